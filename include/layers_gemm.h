// xft::invokeGemm, source-compatible with the reference's include/layers_gemm.h:21-22.
// MI355X build: A, B (row-major [K,N], or [N,K] when transB), C, bias and res are HOST buffers
// of the element type named by dt (bf16 or fp16); C = alpha * op(A) * op(B) + beta * C (+ bias)
// (+ res).  B is converted and packed on every call, as the reference does.
// The declarations follow intel/xFasterTransformer (Apache-2.0, Copyright (c) Intel Corporation).
#pragma once

#include "dtype.h"

namespace xft {

void invokeGemm(DataType dt, bool transA, bool transB, int M, int N, int K, float alpha, void *A, int lda, void *packedB, float beta,
        void *C, int ldc, void *bias = nullptr, void *res = nullptr, int ldres = -1);

} // namespace xft
