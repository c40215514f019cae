// xft::invokeRmsNorm, source-compatible with the reference's include/layers_norm.h:24-25.
// Host buffers of the element type named by dt (fp32, bf16 or fp16 is not offered: bf16/fp32).
// The declarations follow intel/xFasterTransformer (Apache-2.0, Copyright (c) Intel Corporation).
#pragma once

#include "dtype.h"

namespace xft {

void invokeRmsNorm(DataType dt, void *output, const void *input, const void *weight, int rows, int cols,
        int iStride = -1, int oStride = -1, float epsilon = 1e-6);

} // namespace xft
