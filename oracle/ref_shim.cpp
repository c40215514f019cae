// Thin extern "C" exports over the reference's OWN in-tree sources, compiled where they
// lie (REF_ROOT, normally /root/reference).  Nothing of the reference is copied here:
// this file only includes its headers and forwards calls, so the CPU oracle can be
// checked against the real thing.  TEST INFRASTRUCTURE ONLY; needs an AVX-512 host.
//
// Built by oracle/Makefile into oracle/_ref/libxft_ref.so together with
//   src/kernels/rotary_embedding_kernels.cpp   (RoPE)
//   src/kernels/gemm_kernel_ext3.cpp           (P*V small_gemm, fp32 / fp16 / bf16)
// The remaining kernels of the path need headers of closed or un-vendored libraries
// (xDNN sgemm.h / intrinsic_ext.h / softmax.h, mkl.h, oneDNN) and are not buildable here.
#include <cstdint>
#include <cstring>

#include "bfloat16.h"
#include "float16.h"
#include "uint4x2.h"
#include "bert_util.h"
#include "intrinsics_util.h"
#include "quantize_util.h"
#include "copy_util.h"
#include "rotary_embedding_kernels.h"

namespace xft {
void small_gemm(const float *A, const float *B, float *C, int M, int N, int K, int lda, int ldb, int ldc, bool acc);
void small_gemm(
        const float *A, const float16_t *B, float *C, int M, int N, int K, int lda, int ldb, int ldc, bool acc);
} // namespace xft

extern "C" {

// include/bfloat16.h:40-65 (scalar assignment operator)
uint16_t ref_f32_to_bf16(float f) {
    bfloat16_t b = f;
    uint16_t r;
    std::memcpy(&r, &b, 2);
    return r;
}

// src/utils/intrinsics_util.h:89-92 (store_avx512<bfloat16_t>, vcvtneps2bf16)
void ref_store_bf16(const float *src, uint16_t *dst, int n) {
    for (int i = 0; i < n; i += 16) {
        int remain = n - i;
        __mmask16 mask = (remain >= 16 ? 0xffff : (1 << remain) - 1);
        xft::store_avx512((bfloat16_t *)dst + i, mask, _mm512_maskz_loadu_ps(mask, src + i));
    }
}

// src/utils/intrinsics_util.h:94-97 (store_avx512<float16_t>) and :42-46 (load)
void ref_store_fp16(const float *src, uint16_t *dst, int n) {
    for (int i = 0; i < n; i += 16) {
        int remain = n - i;
        __mmask16 mask = (remain >= 16 ? 0xffff : (1 << remain) - 1);
        xft::store_avx512((float16_t *)dst + i, mask, _mm512_maskz_loadu_ps(mask, src + i));
    }
}
void ref_load_fp16(const uint16_t *src, float *dst, int n) {
    for (int i = 0; i < n; i += 16) {
        int remain = n - i;
        __mmask16 mask = (remain >= 16 ? 0xffff : (1 << remain) - 1);
        _mm512_mask_storeu_ps(dst + i, mask, xft::load_avx512(mask, (const float16_t *)src + i));
    }
}

// src/common/uint4x2.h:43-71
void ref_uint4x2_unpack(const uint8_t *packed, uint8_t *v1, uint8_t *v2, int n) {
    for (int i = 0; i < n; ++i) {
        uint4x2_t p;
        std::memcpy(&p, packed + i, 1);
        v1[i] = p.get_v1();
        v2[i] = p.get_v2();
    }
}
uint8_t ref_uint4x2_pack(uint8_t v1, uint8_t v2) {
    uint4x2_t p(v1, v2);
    uint8_t r;
    std::memcpy(&r, &p, 1);
    return r;
}

// src/utils/bert_util.h:26-75
void ref_vexp(const float *x, float *y, int n) {
    for (int i = 0; i < n; i += 16) {
        int remain = n - i;
        __mmask16 mask = (remain >= 16 ? 0xffff : (1 << remain) - 1);
        __m512 v = _mm512_maskz_loadu_ps(mask, x + i);
        _mm512_mask_storeu_ps(y + i, mask, BertUtil::vexp(v));
    }
}

// src/utils/quantize_util.h:36-51
void ref_kv_quantize(int8_t *dst, float *scale, const float *src, int size) {
    xft::quantize(dst, scale, const_cast<float *>(src), size);
}

// src/kernels/rotary_embedding_kernels.cpp:21-38
void ref_rope_tables(const float *invFreq, float *embCos, float *embSin, int invFreqSize, int maxPos) {
    xft::llamaSetCosSinCache(invFreq, embCos, embSin, invFreqSize, maxPos);
}
// :57-121
void ref_rope_apply_f32(float *q, float *k, int qStride, int kStride, float *embCos, float *embSin, int half,
        const int *qkShape, const int *pos) {
    xft::llamaApplyRotaryPosEmbeding(q, k, qStride, kStride, embCos, embSin, half, qkShape, pos);
}
void ref_rope_apply_bf16(uint16_t *q, uint16_t *k, int qStride, int kStride, float *embCos, float *embSin, int half,
        const int *qkShape, const int *pos) {
    xft::llamaApplyRotaryPosEmbeding(
            (bfloat16_t *)q, (bfloat16_t *)k, qStride, kStride, embCos, embSin, half, qkShape, pos);
}
// :126-199
void ref_rope_apply_tokens_f32(float *q, float *k, float *embCos, float *embSin, int qStride, int kStride, int dim,
        int totSeqLen, int qHeads, int kHeads, const int *pos) {
    xft::llamaApplyRotaryPosEmbed(q, k, embCos, embSin, qStride, kStride, dim, totSeqLen, qHeads, kHeads, pos);
}

// src/kernels/gemm_kernel_ext3.cpp:50-214
void ref_small_gemm_f32(const float *A, const float *B, float *C, int M, int N, int K, int lda, int ldb, int ldc,
        int acc) {
    xft::small_gemm(A, B, C, M, N, K, lda, ldb, ldc, acc != 0);
}
void ref_small_gemm_f16(const float *A, const uint16_t *B, float *C, int M, int N, int K, int lda, int ldb, int ldc,
        int acc) {
    xft::small_gemm(A, (const float16_t *)B, C, M, N, K, lda, ldb, ldc, acc != 0);
}

} // extern "C"
