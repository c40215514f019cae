// xft::invokeRotaryEmbedding, source-compatible with the reference's
// include/layers_rotary_embedding.h:23-33.  In-place rotate-half RoPE on host query / key buffers
// of the element type named by dt (fp32 or bf16); embCos / embSin are [maxPosition, dim] tables in the
// same element type, the second half of a head reading columns [dim/2, dim) (the reference reads them
// this way, src/layers/rotary_embedding_api.cpp:35-47).
// The declaration follows intel/xFasterTransformer (Apache-2.0, Copyright (c) 2024 Intel Corporation).
#pragma once

#include <cmath>
#include <cstdint>
#include <cstring>

#include "dtype.h"

namespace xft {
void invokeRotaryEmbedding(DataType dt,
        const int64_t *positionIds, // [numTokens]
        void *query, // [numTokens, headNum, headSize]
        void *key, // [numTokens, numKvHeads, headSize]
        const void *embCos, // [maxPosition, dim]
        const void *embSin, // [maxPosition, dim]
        const int dim, // rotary dimension
        const int qStride, const int kStride, const int numTokens, const int headNum, const int headSize,
        const int numKvHeads);
} // namespace xft
