// xft::invokeMLPLLaMA, source-compatible with the reference's include/layers_mlp.h:21-23.
// output = down(silu(gate(input)) * up(input)) + input; input/output are fp32 host buffers
// [numTokens, stride]; the weights are fp32 host matrices [in, out] converted once per distinct
// set of weight addresses.  dt selects the on-device weight format: bf16 (the reference's), or
// the weight-only formats int8 / int4 / nf4 this build adds to the same entry point.
// The declarations follow intel/xFasterTransformer (Apache-2.0, Copyright (c) Intel Corporation).
#pragma once

#include "dtype.h"

namespace xft {

void invokeMLPLLaMA(DataType dt, ActivationType at, int numTokens, int hiddenSize, int intermediateSize, void *output,
        int outputStride, const void *input, int inputStride, const void *gateWeight, const void *upWeight,
        const void *downWeight);

} // namespace xft
