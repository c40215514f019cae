// xft::invokeAttentionLLaMA, source-compatible with the reference's include/layers_attention.h:61-65.
// output = Attention(input) * Wo + bias + input (no input norm), fp32 host buffers
// [batchSize*inputSeqLen, stride].  query/key/value weights are the three column blocks of one
// fp32 [hiddenSize, (attHeadNum + 2*kvHeadNum) * attHeadDim] host matrix (row stride = that
// width), attnOutWeight is [attHeadNum*attHeadDim, hiddenSize].  The KV cache (FP16) belongs to
// the callee and carries over between calls: pastSeqLen / step are supplied by the caller.
// The declarations follow intel/xFasterTransformer (Apache-2.0, Copyright (c) Intel Corporation).
#pragma once

#include "dtype.h"

namespace xft {

void invokeAttentionLLaMA(DataType dt, int batchSize, int inputSeqLen, int attHeadDim, int attHeadNum, int kvHeadNum,
        int maxPositions, int maxPosEmbed, int pastSeqLen, int currentSeqLen, int step, int hiddenSize, void *output,
        int outputStride, const void *input, int inputStride, const void *queryWeight, const void *keyWeight,
        const void *valueWeight, const void *attnOutWeight, const float *queryBias = nullptr,
        const float *keyBias = nullptr, const float *valueBias = nullptr, const float *attnOutBias = nullptr);

} // namespace xft
