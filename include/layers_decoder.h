// xft::invokeLayerLLaMA, source-compatible with the reference's include/layers_decoder.h:21-28.
// One Llama decoder layer: RMSNorm -> fused QKV -> RoPE -> causal attention over the callee's
// FP16 KV cache -> out-proj + residual -> RMSNorm -> SwiGLU MLP + residual.  fp32 host
// activations, fp32 host weights [in, out] (see layers_attention.h for the Q/K/V layout).
// The declarations follow intel/xFasterTransformer (Apache-2.0, Copyright (c) Intel Corporation).
#pragma once

#include "dtype.h"

namespace xft {

void invokeLayerLLaMA(DataType dt, ActivationType at, NormType nt, int batchSize, int inputSeqLen, int attHeadDim,
        int attHeadNum, int kvHeadNum, int maxPositions, int maxPosEmbed, int pastSeqLen, int currentSeqLen, int step,
        int hiddenSize, int intermediateSize, void *output, int outputStride, const void *input, int inputStride,
        const float *ln1Gamma, const float *ln1Beta, const void *queryWeight, const void *keyWeight,
        const void *valueWeight, const void *attnOutWeight, const float *ln2Gamma, const float *ln2Beta,
        const void *gateWeight, const void *upWeight, const void *downWeight, const float *queryBias = nullptr,
        const float *keyBias = nullptr, const float *valueBias = nullptr, const float *attnOutBias = nullptr);

} // namespace xft
