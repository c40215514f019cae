// xft::invokeLayerNorm and xft::invokeRmsNorm, source-compatible with the reference's
// include/layers_norm.h:21-25.  Host buffers of the element type named by dt: fp32 or bf16 (fp16
// activations are not offered: such a call returns without writing, the reference's own behaviour
// for a dt it does not know).
// The declarations follow intel/xFasterTransformer (Apache-2.0, Copyright (c) Intel Corporation).
#pragma once

#include "dtype.h"

namespace xft {

void invokeLayerNorm(DataType dt, void *output, const void *input, const void *gamma, const void *beta, int rows,
        int cols, int iStride = -1, int oStride = -1, float epsilon = 1e-5);

void invokeRmsNorm(DataType dt, void *output, const void *input, const void *weight, int rows, int cols,
        int iStride = -1, int oStride = -1, float epsilon = 1e-6);

} // namespace xft
