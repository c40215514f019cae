/*
 * C-ABI of the MI355X (gfx950) implementation of the xFasterTransformer decoder-layer
 * hot path.  Plain C: opaque handles, raw pointers and sizes, int status (0 = ok,
 * non-zero = error, text from xfthip_last_error()).  No HIP, CUDA or torch types.
 *
 * Unless a parameter is marked "host", data pointers are DEVICE pointers
 * (xfthip_malloc, or any hipMalloc'ed memory such as a torch tensor's data_ptr()).
 * `stream` is a hipStream_t passed as void* (NULL = the default stream); every compute
 * call is asynchronous on it.
 *
 * Each entry point cites the interface of the reference (intel/xFasterTransformer
 * v2.1.2, paths relative to its tree) that it replaces.
 */
#ifndef XFT_HIP_H
#define XFT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *xfthip_stream_t;
typedef void *xfthip_event_t;
typedef struct xfthip_weight *xfthip_weight_t;
typedef struct xfthip_kvcache *xfthip_kvcache_t;

/* element types of activation buffers */
enum { XFTHIP_F32 = 0, XFTHIP_BF16 = 1, XFTHIP_FP16 = 2, XFTHIP_INT8 = 3 };

/* weight kinds: the WeiT template argument of MMHelper (src/utils/matmul_helper.h:149-405) */
enum { XFTHIP_W_INT8 = 0, XFTHIP_W_UINT4 = 1, XFTHIP_W_NF4 = 2, XFTHIP_W_W8A8 = 3, XFTHIP_W_BF16 = 4 };

/* GEMM epilogues: MMHelper::compute / compute_bias / compute_silu / compute_gelu /
 * compute_resmul / compute_residential / compute_resext (matmul_helper.h:565-1705) */
enum {
    XFTHIP_EPI_NONE = 0,
    XFTHIP_EPI_BIAS = 1,
    XFTHIP_EPI_SILU = 2,
    XFTHIP_EPI_GELU = 3,
    XFTHIP_EPI_RESMUL = 4,
    XFTHIP_EPI_RESIDENTIAL = 5,
    XFTHIP_EPI_RESEXT = 6
};

/* weight_create flags */
enum {
    XFTHIP_WF_NONE = 0,
    /* the [K, 2I] matrix is cat(gate, up) as LlamaMLP::catGateUpWeights builds it
     * (src/layers/mlp_llama.h:413-454); pack gate/up column tiles interleaved so that
     * xfthip_gemm_gateup_silu can combine them in registers */
    XFTHIP_WF_GATEUP = 1
};

/* ---- runtime ------------------------------------------------------------------------ */
int xfthip_init(int device);
int xfthip_finalize(void);
const char *xfthip_last_error(void);
/* name of the device in use and its compute-unit count (for logs) */
int xfthip_device_info(char *name, int name_len, int *compute_units, size_t *hbm_bytes);

int xfthip_malloc(void **ptr, size_t bytes);
int xfthip_free(void *ptr);
int xfthip_memcpy_h2d(void *dst, const void *src_host, size_t bytes, xfthip_stream_t stream);
int xfthip_memcpy_d2h(void *dst_host, const void *src, size_t bytes, xfthip_stream_t stream);
int xfthip_memcpy_d2d(void *dst, const void *src, size_t bytes, xfthip_stream_t stream);
int xfthip_memset(void *dst, int value, size_t bytes, xfthip_stream_t stream);
int xfthip_stream_create(xfthip_stream_t *stream);
int xfthip_stream_destroy(xfthip_stream_t stream);
int xfthip_stream_synchronize(xfthip_stream_t stream);
int xfthip_device_synchronize(void);
int xfthip_event_create(xfthip_event_t *ev);
int xfthip_event_destroy(xfthip_event_t ev);
int xfthip_event_record(xfthip_event_t ev, xfthip_stream_t stream);
int xfthip_event_synchronize(xfthip_event_t ev);
int xfthip_event_elapsed_ms(xfthip_event_t start, xfthip_event_t stop, float *ms);

/* ---- weights ------------------------------------------------------------------------ */
/*
 * Replaces MMHelper::convertWeight + packWeight for already-quantised weights
 * (matmul_helper.h:284-315 INT8->INT8 / UINT4->UINT4 copies, :407-534 pack).
 * q_host: the reference's pre-pack layout, row-major [K, N]: int8 per element, or two
 * 4-bit codes per byte along N with the even column in the low nibble
 * (src/common/uint4x2.h:43-71); bf16 bit patterns for XFTHIP_W_BF16.
 * scale_host / zero_host: fp32 [N] (w = scale*q + zero; NF4: scale = absmax, zero NULL;
 * zero may be NULL = all zero).  W8A8 also derives the per-column integer sums
 * (matmul_helper.h:362-372).  The device layout is private to this library.
 */
int xfthip_weight_create(int kind, int K, int N, const void *q_host, const float *scale_host,
        const float *zero_host, int flags, xfthip_weight_t *out);
int xfthip_weight_destroy(xfthip_weight_t w);
int xfthip_weight_shape(xfthip_weight_t w, int *kind, int *K, int *N);
/* bytes the GEMM streams from HBM for this weight (packed codes + side vectors) */
size_t xfthip_weight_bytes(xfthip_weight_t w);
/* inverse of the private packing: recovers q in the pre-pack layout (host buffer) */
int xfthip_weight_unpack(xfthip_weight_t w, void *q_host_out);
/*
 * Device dequantisation of the whole matrix to row-major [K, N]:
 * out_dtype XFTHIP_F32 -> fmaf(scale, q, zero);  XFTHIP_BF16 -> that value narrowed as
 * static_cast<bfloat16_t> does (matmul_helper.h:317-346, include/bfloat16.h:40-65).
 */
int xfthip_weight_dequant(xfthip_weight_t w, void *out, int out_dtype, xfthip_stream_t stream);
/*
 * Build-owned weight quantizers (the reference calls xdnn_*_quantize,
 * matmul_helper.h:205-262, whose source is not published).  W_host fp32 [K, N] host;
 * outputs are host buffers in the pre-pack layout accepted by xfthip_weight_create.
 */
int xfthip_quantize_weight(int kind, int K, int N, const float *W_host, void *q_host_out, float *scale_host_out,
        float *zero_host_out);

/* ---- weight-only GEMM --------------------------------------------------------------- */
/*
 * C[M,N] = epilogue(A[M,K] * deq(W)[K,N]).  Replaces MMHelper::compute and its
 * compute_bias/_silu/_gelu/_resmul/_residential/_resext variants
 * (matmul_helper.h:565-1705; W8A8: onednn_amx_gemm_f32s8f32_compute, :2762-2965).
 * A: bf16 [M, lda].  C: c_dtype (XFTHIP_F32 or XFTHIP_BF16) [M, ldc].
 * bias: fp32 [N] or NULL.  res: res_dtype [M, ldres] or NULL; may alias C.
 * gamma: residual scale for XFTHIP_EPI_RESEXT.
 */
int xfthip_gemm(xfthip_weight_t w, int M, const void *A, int lda, void *C, int ldc, int c_dtype, int epilogue,
        const float *bias, const void *res, int ldres, int res_dtype, float gamma, xfthip_stream_t stream);
/*
 * out[M,I] = silu(A*Wgate) * (A*Wup) for a weight created with XFTHIP_WF_GATEUP.
 * Replaces the cat GEMM + DecoderUtil::siluSum pair of LlamaMLP::forward
 * (src/layers/mlp_llama.h:380-411, src/utils/decoder_util.h:550-573).
 */
int xfthip_gemm_gateup_silu(xfthip_weight_t w, int M, const void *A, int lda, void *out, int ldo, int out_dtype,
        xfthip_stream_t stream);


/* ---- RMSNorm ------------------------------------------------------------------------ */
/*
 * y = (x * 1/sqrt(mean(x^2) + eps)) * weight, fp32 accumulation.  Replaces xft::rmsNorm /
 * xft::invokeRmsNorm (src/kernels/rmsnorm_kernels.cpp:27-180).  in/out: XFTHIP_F32 or
 * XFTHIP_BF16; weight: fp32 [cols]; strides in elements (-1 = cols).
 */
int xfthip_rmsnorm(void *out, int out_dtype, const void *in, int in_dtype, const float *weight, int rows, int cols,
        int iStride, int oStride, float eps, xfthip_stream_t stream);

/* ---- rotary embedding --------------------------------------------------------------- */
/*
 * cos/sin tables [maxPos, dim/2] fp32 in device memory, built as LlamaRotaryEmbedding does
 * (src/layers/rotary_embedding.cpp:21-46, src/kernels/rotary_embedding_kernels.cpp:21-38):
 * inv_freq = 1/pow(base, float(2i)/dim) in double, cosf/sinf(float(pos * inv_freq)).
 * Free both with xfthip_free.
 */
int xfthip_rope_tables_create(int dim, int maxPos, int base, float scalingFactor, float **cos_dev, float **sin_dev);
/*
 * In-place rotate-half RoPE on query [numTokens, qStride] and key [numTokens, kStride]
 * (dtype XFTHIP_F32 or XFTHIP_BF16): q' = q*cos - q_half*sin, q_half' = q_half*cos + q*sin.
 * Replaces xft::invokeRotaryEmbedding / llamaApplyRotaryPosEmbed
 * (include/layers_rotary_embedding.h:23-33, rotary_embedding_kernels.cpp:126-199).
 * positions: device int32 [numTokens].
 */
int xfthip_rotary_embedding(int dtype, const int *positions, void *query, void *key, const float *embCos,
        const float *embSin, int dim, int qStride, int kStride, int numTokens, int headNum, int headSize,
        int numKvHeads, xfthip_stream_t stream);

/* ---- KV cache ----------------------------------------------------------------------- */
/*
 * One layer's key and value cache for `batch` sequences.  Replaces KVCacheTensor<float16_t>
 * / KVCacheTensor<int8_t> (src/common/kvcache_tensor.h:65-143): dtype XFTHIP_FP16 stores RNE
 * fp16, XFTHIP_INT8 stores per-(token, head) symmetric int8 with an fp32 scale
 * (xft::quantize, src/utils/quantize_util.h:36-51).  The device layout is private (keys
 * [B][H][S][D]; values blocked by 32 tokens with the token index innermost so that both
 * feed MFMA operands with 128-bit loads); export/import convert from/to the reference's
 * ENABLE_KV_TRANS=1 layout: data [B][H][maxSeq][D], scales [B][H][maxSeq].
 */
int xfthip_kvcache_create(int dtype, int batch, int kvHeads, int maxSeq, int headSize, xfthip_kvcache_t *out);
int xfthip_kvcache_destroy(xfthip_kvcache_t c);
/* which: 0 = keys, 1 = values.  data_dev: fp16 bits or int8 [B][H][maxSeq][D]; scales_dev fp32 [B][H][maxSeq] (INT8 only, may be NULL for FP16) */
int xfthip_kvcache_export(xfthip_kvcache_t c, int which, void *data_dev, float *scales_dev, xfthip_stream_t stream);
int xfthip_kvcache_import(xfthip_kvcache_t c, int which, const void *data_dev, const float *scales_dev,
        xfthip_stream_t stream);
/*
 * RoPE on q and k, then append k and v of S new tokens per sequence to the cache at
 * positions past .. past+S-1.  Replaces the RoPE call of Attention::forward
 * (src/layers/attention.h:357-374) plus storeKVCache (src/kernels/attention_kernels.h:44-69).
 * qkv: [B*S, stride] of dtype (XFTHIP_BF16 or XFTHIP_F32); q at column 0, k at qHeads*D, v at
 * (qHeads+kvHeads)*D.  q is rotated in place; k and v are left untouched in qkv (the rotated k
 * goes to the cache from fp32 registers).  embCos == NULL skips the rotation (plain store).
 * past_dev: optional device int32 [B] overriding `past` (lets a captured graph be replayed
 * while the host advances nothing).
 */
int xfthip_rope_kvstore(xfthip_kvcache_t c, void *qkv, int dtype, int stride, int B, int S, int qHeads,
        const float *embCos, const float *embSin, int past, const int *past_dev, xfthip_stream_t stream);

/* ---- attention over the cache ------------------------------------------------------- */
/*
 * Causal GQA attention of S new query tokens per sequence over cache rows [0, past+S):
 * query token s attends to rows 0 .. past+s.  S == 1 is decode; S > 1 with past == 0 is
 * prefill; S > 1 with past > 0 is chunked prefill.  The cache must already hold the new
 * rows (xfthip_rope_kvstore).  Replaces xft::crossAttnByHead / crossAttnShardedHead /
 * selfScaledDpAttention / selfAttention (src/kernels/attention_kernels.h:139-552,
 * 838-1123, 1283-1408): scores in fp32, online softmax, the KV sequence split across
 * workgroups and merged with the (max, sum) statistics.
 * q: bf16 [B*S, qStride], head h at column h*D.  out: out_dtype (bf16 or f32) [B*S, oStride].
 * past_dev: optional device int32 [B] overriding `past`.  scale: 1/sqrt(D).
 */
int xfthip_attention(xfthip_kvcache_t c, const void *q, int qStride, void *out, int oStride, int out_dtype, int B,
        int S, int qHeads, float scale, int past, const int *past_dev, xfthip_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* XFT_HIP_H */
