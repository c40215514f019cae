// Parameter block shared by the weight-only GEMM kernels and their C-ABI entry points.
#pragma once
#include "common.h"

namespace xfthip {

struct SkinnyParams {
    const uint8_t *packed;
    const float *scale;
    const float *zero;
    int KT, NTILES, K, N, M;
    const uint16_t *A; // bf16
    int lda;
    void *C;
    int ldc, c_dtype;
    int epi;
    const float *bias;
    const void *res;
    int ldres, res_dtype;
    float gamma;
    int gateup; // 1: combine tile pairs as silu(gate)*up, N counts cat columns
};

int qgemm_skinny(const PackedWeight &pw, const SkinnyParams &p, hipStream_t stream); // M <= 32
int qgemm_mfma(const PackedWeight &pw, const SkinnyParams &p, hipStream_t stream); // any M, built for M > 32

int gemm_w8a8_from_bf16(xfthip_weight_t w, int M, const void *A, int lda, void *C, int ldc, int c_dtype, int epilogue,
        const float *bias, const void *res, int ldres, int res_dtype, float gamma, hipStream_t stream);

} // namespace xfthip
