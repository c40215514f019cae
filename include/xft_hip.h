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
typedef void *xfthip_graph_t;
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
/* Device-to-device copy by a plain kernel of this library (16 bytes per lane; pointers and size
 * 16-byte aligned): reads `bytes` and writes `bytes`, which makes it the reference point when
 * hardware counters of HBM traffic are scaled.  No counterpart in the reference. */
int xfthip_copy_kernel(void *dst, const void *src, size_t bytes, xfthip_stream_t stream);
/* Reads `bytes` (a multiple of 16, 16-byte aligned) with `blocks` workgroups (0 = two per compute unit) and
 * discards them: the time of a launch is what streaming that many bytes costs on this machine with nothing
 * behind the loads, launch ramp and tail included - the floor bench.py prints beside the weight-streaming
 * kernels.  A measurement aid with no counterpart in the reference. */
int xfthip_read_kernel(const void *src, size_t bytes, int blocks, xfthip_stream_t stream);
int xfthip_memset(void *dst, int value, size_t bytes, xfthip_stream_t stream);
/* Free and total device memory of the current device in bytes (either pointer may be null).  The host layer sizes
 * the cache rows of its sequence pool with it; no counterpart in the reference, whose caches live in host memory. */
int xfthip_device_memory(size_t *free_bytes, size_t *total_bytes);
int xfthip_stream_create(xfthip_stream_t *stream);
int xfthip_stream_destroy(xfthip_stream_t stream);
int xfthip_stream_synchronize(xfthip_stream_t stream);
int xfthip_device_synchronize(void);
/* Stream capture for callers that replay a fixed sequence of this library's calls (the reference has no
 * counterpart: its CPU kernels are called directly).  Between begin and end, calls on `stream` are recorded
 * instead of run; only calls that neither allocate nor wait for the device may be recorded.  The graph that
 * comes back is ready to launch on any stream. */
int xfthip_graph_begin(xfthip_stream_t stream);
int xfthip_graph_end(xfthip_stream_t stream, xfthip_graph_t *graph);
int xfthip_graph_launch(xfthip_graph_t graph, xfthip_stream_t stream);
int xfthip_graph_destroy(xfthip_graph_t graph);
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

/*
 * The two decode-step fusions of the M <= 32 kernel, for up to 4 activation rows (the model
 * driver uses them when it decodes; they are entry points of their own so that they can be
 * tested and timed alone).  The reference runs the norm, the projection, the rotation and the
 * cache write as separate calls (src/layers/rms_norm.cpp:54-110, src/layers/attention.h:322-460,
 * src/layers/mlp_llama.h:200-260); the bf16 hand-over points between them are kept.
 *
 * xfthip_gemm_gateup_silu_rmsnorm: out = silu(n W_gate) * (n W_up) with
 *   n = bf16(x * rsqrt(mean(x^2) + eps) * norm_weight), x fp32 [M, K] with row pitch ldx.
 *
 * xfthip_gemm_qkv_rmsnorm_rope: one new token per sequence (row m belongs to sequence m of the
 * cache).  qkv = bf16(n W); the query heads are rotated (tables of xfthip_rope_tables_create,
 * 64 entries a row) and written as bf16 to q_out [M, q_heads * 128] (row pitch ldq); the rotated
 * key heads and the value heads are appended to `cache` (FP16 cache, head size 128) at
 * position_dev[m], or at `position` for every row when position_dev is NULL.
 */
int xfthip_gemm_gateup_silu_rmsnorm(xfthip_weight_t w, int M, const float *x, int ldx, const float *norm_weight, float eps,
        void *out, int ldo, int out_dtype, xfthip_stream_t stream);
int xfthip_gemm_qkv_rmsnorm_rope(xfthip_weight_t w, xfthip_kvcache_t cache, int M, const float *x, int ldx,
        const float *norm_weight, float eps, void *q_out, int ldq, int q_heads, const float *cos_table,
        const float *sin_table, int position, const int *position_dev, xfthip_stream_t stream);


/*
 * W8A8 pieces (matmul_helper.h:2762-2965).  quantize_rows: per-row asymmetric INT8 quantisation of
 * A (f32 or bf16): zero = (min+max)/2, scale = max(|max-zero|,|zero-min|)/127,
 * q = rne(fma(x, 1/scale, -zero/scale)), sum = (sum q)*scale + K*zero.  gemm_w8a8: int8 x int8 ->
 * int32 GEMM against an XFTHIP_W_W8A8 weight, then C = s32*sA*sB + sumB*sB*zA + sumA*zB and the
 * epilogue.  qa: int8 [M, ldq], 16-byte aligned, ldq % 16 == 0.  xfthip_gemm on a W8A8 weight runs
 * both, quantising its bf16 A into the scratch of the call's stream (grown on demand: a first call of a size is not
 * for use under stream capture).
 */
int xfthip_w8a8_quantize_rows(const void *A, int a_dtype, int M, int K, int lda, int8_t *qa, int ldq, float *scale,
        float *zero, float *sum, xfthip_stream_t stream);
int xfthip_gemm_w8a8(xfthip_weight_t w, int M, const int8_t *qa, int ldq, const float *scaleA, const float *zeroA,
        const float *sumA, void *C, int ldc, int c_dtype, int epilogue, const float *bias, const void *res, int ldres,
        int res_dtype, float gamma, xfthip_stream_t stream);

/* ---- RMSNorm ------------------------------------------------------------------------ */
/*
 * y = (x * 1/sqrt(mean(x^2) + eps)) * weight, fp32 accumulation.  Replaces xft::rmsNorm /
 * xft::invokeRmsNorm (src/kernels/rmsnorm_kernels.cpp:27-180).  in/out: XFTHIP_F32 or
 * XFTHIP_BF16; weight: fp32 [cols]; strides in elements (-1 = cols).
 */
int xfthip_rmsnorm(void *out, int out_dtype, const void *in, int in_dtype, const float *weight, int rows, int cols,
        int iStride, int oStride, float eps, xfthip_stream_t stream);

/* ---- LayerNorm ---------------------------------------------------------------------- */
/*
 * y = (x - mean) * gamma / sqrt(E[x^2] - mean^2 + eps) + beta, fp32 arithmetic.  Replaces
 * xft::invokeLayerNorm / LayerNorm::forward (src/kernels/layernorm_kernels.cpp:27-160).  in/out:
 * XFTHIP_F32 or XFTHIP_BF16; gamma, beta: fp32 [cols]; strides in elements (-1 = cols).
 */
int xfthip_layernorm(void *out, int out_dtype, const void *in, int in_dtype, const float *gamma, const float *beta, int rows,
        int cols, int iStride, int oStride, float eps, xfthip_stream_t stream);

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

/*
 * Same rotation with tables laid out as the public xft::invokeRotaryEmbedding takes them:
 * [maxPosition, dim], the second half of a head reading columns [dim/2, dim)
 * (src/layers/rotary_embedding_api.cpp:20-50).
 */
int xfthip_rotary_embedding_full(int dtype, const int *positions, void *query, void *key, const float *embCos,
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
/* Rows of one cache copied / re-mapped (beam search; KVCacheTensor::reorder, reference
 * src/common/kvcache_tensor.h:196-286, and ::expandAllSequence, :147-173): row dst_rows_host[i] becomes a
 * copy of row src_rows_host[i] over the positions [pos0, pos1), widened to whole 32-token blocks.  A row
 * may be source and destination at once. */
int xfthip_kvcache_reorder(xfthip_kvcache_t cache, const int *dst_rows_host, const int *src_rows_host, int n, int pos0, int pos1,
        xfthip_stream_t stream);
/* which: 0 = keys, 1 = values.  data_dev: fp16 bits or int8 [B][H][maxSeq][D]; scales_dev fp32 [B][H][maxSeq] (INT8 only, may be NULL for FP16) */
int xfthip_kvcache_export(xfthip_kvcache_t c, int which, void *data_dev, float *scales_dev, xfthip_stream_t stream);
int xfthip_kvcache_import(xfthip_kvcache_t c, int which, const void *data_dev, const float *scales_dev,
        xfthip_stream_t stream);
/* the same with data_dev laid out [maxSeq][B][H][D], the reference's layout when ENABLE_KV_TRANS is off
 * (src/common/kvcache_tensor.h:113-117); the scales stay [B][H][maxSeq] as there */
int xfthip_kvcache_export_sbhd(xfthip_kvcache_t c, int which, void *data_dev, float *scales_dev, xfthip_stream_t stream);
int xfthip_kvcache_import_sbhd(xfthip_kvcache_t c, int which, const void *data_dev, const float *scales_dev,
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

/*
 * xfthip_attention for callers that cannot allocate (code under HIP graph capture, serving loops
 * and harnesses that forbid hipMalloc): same arguments, same kernel and same split of the KV
 * sequence, but the partial results and tickets of the split merge live in a statically allocated
 * device array of the library (1024 partial-result slots, about 8.5 MB per GPU, held until the
 * process ends) instead of the workspace xfthip_attention allocates on first use.  The call
 * allocates and frees nothing.  A shape whose split needs more than 1024 slots (column groups
 * B * kvHeads * ceil(S * qHeads / kvHeads / 16) times sequence splits) is rejected with an error
 * that says so; the split rule makes at most two slots a compute unit, so that on a device of up to
 * 512 compute units no shape is.  All calls on one GPU share the array: calls that overlap on one GPU (two streams)
 * race; calls on one stream do not.  No counterpart in the reference.
 */
int xfthip_attention_static(xfthip_kvcache_t c, const void *q, int qStride, void *out, int oStride, int out_dtype, int B,
        int S, int qHeads, float scale, int past, const int *past_dev, xfthip_stream_t stream);


/*
 * Attention over a block-paged BF16 KV cache: the device side of xft::invokeAttention
 * (include/layers_attention.h:22-59, src/kernels/attention_kernels.cpp:24-157).  Caches are
 * [block_num][block_size][kv_heads][head_size] bf16 in device memory; slot = block * block_size + row.
 * Decode: one new token per sequence.  key / value row b is stored at slot_mapping[b], then query row b
 * attends to the context_lens[b] + 1 tokens that block_tables row b (table_stride entries a row)
 * maps, new token included: fp32 scores, softmax(scale * s), fp32 P.V, bf16 out [batch, o_stride].
 * max_context: the largest context_lens value (host copy); every table row must hold
 * max_context / block_size + 1 valid entries.  All pointers but none of the integers are device memory.
 * The reference reads query / key / value row 0 for every sequence and indexes the KV head with the
 * query head (attention_kernels.cpp:51-61); this entry point uses row b and head hq / (q_heads / kv_heads),
 * the same for batch 1 without grouped heads.
 */
int xfthip_paged_attention_decode(void *out, const void *q, const void *k, const void *v, int q_heads, int kv_heads,
        int head_size, int q_stride, int kv_stride, int o_stride, float scale, int batch, void *kcache, void *vcache,
        int block_num, int block_size, const int *block_tables, int table_stride, const int *context_lens,
        const int *slot_mapping, int max_context, xfthip_stream_t stream);
/*
 * Prefill: sequences lie back to back in q / k / v (token_lens_host[b] rows each, host array); causal
 * self-attention per sequence (the reference's selfAttention call, attention_kernels.cpp:141-151) and
 * every token's key / value row stored at slot_mapping[token] (device int32, one entry per token).
 */
int xfthip_paged_attention_prefill(void *out, const void *q, const void *k, const void *v, int q_heads, int kv_heads,
        int head_size, int q_stride, int kv_stride, int o_stride, float scale, int batch, const int *token_lens_host,
        void *kcache, void *vcache, int block_num, int block_size, const int *slot_mapping, xfthip_stream_t stream);

/* ---- decoder layers and the model driver -------------------------------------------- */
typedef struct xfthip_model *xfthip_model_t;

typedef struct {
    int layers; /* number of decoder layers */
    int hidden; /* hidden size */
    int intermediate; /* MLP intermediate size */
    int q_heads, kv_heads, head_size;
    int vocab; /* 0: no embedding / lm_head (layer-only use) */
    int max_batch; /* sequences held by the KV caches */
    int max_seq; /* KV cache length per sequence (the reference's maxPositions) */
    int max_tokens; /* largest batch*inputSeqLen a forward call will carry */
    int max_pos_embed; /* rows of the RoPE tables */
    int rope_base; /* rope_theta (an int in the reference, rotary_embedding.h:63) */
    int kv_dtype; /* XFTHIP_FP16 or XFTHIP_INT8 */
    float rms_eps; /* epsilon of the attention-side RMSNorm; the MLP side uses 1e-6 as the
                      reference hard-codes it (src/layers/mlp_llama.h:212) */
} xfthip_model_config;

/*
 * A Llama-family decoder stack resident in HBM: per-layer KV caches, RoPE tables and the
 * activation scratch.  Replaces DecoderContext + KVCacheManager + DecoderBlock
 * (src/common/transformer_ctx.h:63-459, src/models/kvcache_manager.h, src/layers/decoder_block.h:28-150).
 */
int xfthip_model_create(const xfthip_model_config *cfg, xfthip_model_t *out);
int xfthip_model_destroy(xfthip_model_t m);
/*
 * Attach the weights of layer `idx` (handles stay owned by the caller and must outlive the
 * model).  qkv: [hidden, (q+2kv)*head] as Attention::setWeights concatenates it
 * (src/layers/attention.h:94-242); o: [q*head, hidden]; gateup: [hidden, 2*intermediate]
 * created with XFTHIP_WF_GATEUP (LlamaMLP::setWeights, src/layers/mlp_llama.h:63-139);
 * down: [intermediate, hidden].  ln1/ln2: host fp32 [hidden] RMSNorm weights.
 * qkv_bias / o_bias: host fp32 or NULL.
 */
int xfthip_model_set_layer(xfthip_model_t m, int idx, xfthip_weight_t qkv, xfthip_weight_t o, xfthip_weight_t gateup,
        xfthip_weight_t down, const float *ln1_host, const float *ln2_host, const float *qkv_bias_host,
        const float *o_bias_host);
/* the two halves of xfthip_model_set_layer, for callers that drive only one block of a layer
 * (ln*_host may be NULL when that block is always run with do_norm = 0) */
int xfthip_model_set_attention(xfthip_model_t m, int idx, xfthip_weight_t qkv, xfthip_weight_t o, const float *ln1_host,
        const float *qkv_bias_host, const float *o_bias_host);
int xfthip_model_set_mlp(xfthip_model_t m, int idx, xfthip_weight_t gateup, xfthip_weight_t down, const float *ln2_host);
/* NormType::LN of the layer API (src/layers/decoder_layer.cpp:179-181, 195-197: the layer built over
 * LayerNorm instead of RmsNorm): with shifts set, layer idx runs its two norms as LayerNorms with the
 * weights given to xfthip_model_set_layer as gamma and these fp32 [hidden] host arrays as beta (as
 * kernels of their own: the norm prologue of the decode GEMVs is RMSNorm only).  Null pointers turn the
 * layer back into an RMSNorm layer. */
int xfthip_model_set_layer_norm_shifts(xfthip_model_t m, int idx, const float *ln1_beta_host, const float *ln2_beta_host);
/* A second weight set for layer idx that only the prompt pass (xfthip_model_prefill / _seq_prefill) uses; the
 * decode steps keep the layer's own set.  The reference's HybridModel (src/models/hybrid_model.h:25-84: one
 * model per weight type sharing context and KV cache, behind the "bf16_int8"-style type names).  Shapes as in
 * xfthip_model_set_layer, which must have been called for the layer; four NULLs drop the second set. */
int xfthip_model_set_first_token_weights(xfthip_model_t m, int idx, xfthip_weight_t qkv, xfthip_weight_t o, xfthip_weight_t gateup,
        xfthip_weight_t down);
/*
 * Embedding table (host fp16 bit patterns [vocab, hidden], the reference keeps it in FP16:
 * src/layers/token_embedding.h:49-52), final RMSNorm weight (host fp32 [hidden]) and the
 * lm_head weight handle ([hidden, vocab], XFTHIP_W_BF16: never quantised in the reference,
 * src/models/common_decoder.h:1000-1001).
 */
int xfthip_model_set_head(xfthip_model_t m, const uint16_t *embedding_fp16_host, const float *final_norm_host,
        xfthip_weight_t lm_head);
/*
 * One decoder layer: x_out = layer(x_in) for B sequences of S new tokens each at positions
 * past .. past+S-1 (fp32 device buffers [B*S, stride], may alias).  Replaces
 * Decoder::forwardAttention + forwardFFN (src/layers/decoder_layer.h:101-170), the body of
 * xft::invokeLayerLLaMA (src/layers/decoder_layer.cpp:29-160).
 */
int xfthip_model_layer_forward(xfthip_model_t m, int idx, const float *x_in, int in_stride, float *x_out,
        int out_stride, int B, int S, int past, xfthip_stream_t stream);
/*
 * The attention block alone: x_out = Attention(norm?(x_in)) * Wo + bias + x_in.  Replaces
 * Attention::forward as xft::invokeAttentionLLaMA drives it (src/layers/attention.cpp:28-129:
 * do_norm = 0 there; the decoder layer passes 1).
 */
int xfthip_model_attention_forward(xfthip_model_t m, int idx, const float *x_in, int in_stride, float *x_out,
        int out_stride, int B, int S, int past, int do_norm, xfthip_stream_t stream);
/*
 * The MLP block alone: x_out = down(silu(gate(xn)) * up(xn)) + x_in with xn = norm?(x_in).
 * Replaces LlamaMLP::forward as xft::invokeMLPLLaMA drives it (src/layers/mlp_llama.cpp:22-73:
 * do_norm = 0 there).
 */
int xfthip_model_mlp_forward(xfthip_model_t m, int idx, const float *x_in, int in_stride, float *x_out, int out_stride,
        int tokens, int do_norm, xfthip_stream_t stream);
/*
 * Prefill: embeds ids_host [B, S] (host int32), runs every layer at positions 0..S-1, final
 * norm + lm_head on the last token of each sequence and greedy argmax (first maximum wins,
 * src/searchers/sampling.cpp:22-131).  The chosen ids stay on the device as the input of
 * the next decode step.  Replaces CommonDecoder::forward for the first token
 * (src/models/common_decoder.h:315-589).  logits_host (fp32 [B, vocab]) may be NULL.
 */
int xfthip_model_prefill(xfthip_model_t m, const int *ids_host, int B, int S, float *logits_host, xfthip_stream_t stream);
/*
 * Prefix sharing (CommonDecoder::setPrefix / prefixForward, src/models/common_decoder.h:695-768, and the step-0 branch
 * of forward, :337-350, 440-443).  set_prefix runs the n prefix tokens once, as one sequence, into cache row 0.
 * prefill_after_prefix is the prompt pass of B sequences whose first n tokens are that prefix: ids_host [B, S] holds
 * only what follows the prefix; every sequence's cache row starts as a copy of the prefix's positions
 * (KVCacheManager::expandPrefixCache) and the S new tokens run at positions n .. n + S - 1; decode steps follow as after
 * xfthip_model_prefill.  The prefix stays usable for further prefill_after_prefix calls until a plain prompt pass writes
 * row 0 again (xfthip_model_prefill, xfthip_model_seq_prefill into row 0).
 */
int xfthip_model_set_prefix(xfthip_model_t m, const int *ids_host, int n, xfthip_stream_t stream);
int xfthip_model_prefill_after_prefix(xfthip_model_t m, const int *ids_host, int B, int S, float *logits_host, xfthip_stream_t stream);
/*
 * `steps` greedy decode steps, each one replay of a captured HIP graph (embedding of the
 * previous ids, all layers, lm_head, argmax, position advance).  ids_out_host: int32
 * [steps, B] or NULL.  Must follow xfthip_model_prefill with the same B.
 */
int xfthip_model_decode(xfthip_model_t m, int steps, int *ids_out_host, xfthip_stream_t stream);
/*
 * Continuous batching: every sequence lives in one of the model's max_batch cache rows, at its own
 * position; sequences start, step and end independently.  Replaces what the reference's second
 * Attention::forward overload (src/layers/attention.h:501-730) and its per-sequence KV manager
 * (src/common/kvcache_mgr.h:37-194, src/common/sequence.h) give CommonDecoder::forward(seqs):
 * prompts of different lengths in one batch and decode steps over any subset of the live sequences.
 * The caller assigns rows (the host layer's Model class keeps the sequence-id -> row map).
 *   _seq_prefill: the prompt of ONE sequence (ids_host int32 [S]) into `row`: its first token becomes the
 *       row's next input, its position S; logits_host (fp32 [vocab]) may be NULL.
 *   _seq_decode: one step for the listed rows (each must hold a sequence); every other row keeps its
 *       token, position and cache.  ids_out_host int32 [n], in the order of rows_host.  All rows up to
 *       the highest live one run through the kernels (the step is one graph over a dense batch);
 *       the rows that sit out are masked when ids and positions are updated.
 *   _seq_set_next_id / _seq_logits: the searcher's hooks (replace the token a row feeds next; read
 *       the row's last logits).
 *   _seq_reorder: cache row dst_rows_host[i] becomes a copy of row src_rows_host[i] over the positions
 *       [pos0, pos1) (whole 32-token blocks), with its position and next token: the beam searcher's
 *       KVCacheTensor::expandAllSequence (pos0 = 0, beams filled from the row that ran the prompt) and
 *       ::reorder (pos0 = prompt length; src/common/kvcache_tensor.h:147-286).  A row may be source and
 *       destination at once: everything is read before anything is written.
 *   _seq_release: frees the row.
 * xfthip_model_prefill resets this state (all rows in lockstep again).
 */
/* Logits of every prompt position (Model::forward(logitsAll = true), src/models/models.cpp:760-830,
 * CommonDecoder::forward's logitsAll branch): final norm + lm_head over rows [first_row, first_row + rows)
 * of the last prompt pass (xfthip_model_prefill: B * S rows, sequence after sequence; xfthip_model_seq_prefill:
 * S rows), fp32 [rows, vocab] to host memory.  Valid until the next forward call of the model. */
int xfthip_model_prompt_logits(xfthip_model_t m, int first_row, int rows, float *logits_host, xfthip_stream_t stream);
int xfthip_model_seq_prefill(xfthip_model_t m, int row, const int *ids_host, int S, float *logits_host, xfthip_stream_t stream);
int xfthip_model_seq_decode(xfthip_model_t m, const int *rows_host, int n, int *ids_out_host, xfthip_stream_t stream);
int xfthip_model_seq_set_next_id(xfthip_model_t m, int row, int id);
int xfthip_model_seq_logits(xfthip_model_t m, int row, float *logits_host);
int xfthip_model_seq_reorder(xfthip_model_t m, const int *dst_rows_host, const int *src_rows_host, int n, int pos0, int pos1,
        xfthip_stream_t stream);
int xfthip_model_seq_release(xfthip_model_t m, int row);
/* enable (default) or disable replaying the decode step as a captured HIP graph; with 0 every
 * step launches its kernels one by one (for per-kernel profiling) */
int xfthip_model_use_graph(xfthip_model_t m, int enable);
/* enable (default) or disable the decode-step fusions: RMSNorm as the prologue of the QKV and
 * gate/up GEMVs (up to 4 rows) and RoPE + cache append as the epilogue of the QKV GEMV (one new
 * token per sequence, FP16 cache).  Disabled, the step runs xfthip_rmsnorm / xfthip_gemm /
 * xfthip_rope_kvstore one after the other; results agree to the last bit of the bf16 hand-over
 * points except for the fp32 summation order inside the norm.  The reference keeps these as
 * separate calls (src/layers/attention.h:322-460, src/layers/mlp_llama.h:200-260). */
int xfthip_model_use_fusion(xfthip_model_t m, int enable);
/* How the last xfthip_model_decode ran: 1 = graph replay, 0 = eager launches. */
int xfthip_model_decode_mode(xfthip_model_t m);
/* ids chosen by the last prefill / decode call (host int32 [B]) and the current position */
int xfthip_model_last_ids(xfthip_model_t m, int *ids_host, int *position);
/* Replace the ids the next decode step embeds (host int32 [B], each inside the vocabulary): for
 * searchers that do not take the arg-max of the raw logits (sampling, repetition penalty, padding of
 * finished sequences: the nextTokens vector GreedySearch / SampleSearch feed back,
 * src/searchers/greedy_search.cpp:112-119, sample_search.cpp:74-90). */
int xfthip_model_set_next_ids(xfthip_model_t m, const int *ids_host, xfthip_stream_t stream);
/* fp32 logits of the last step, device pointer [B, vocab] (valid until the next call) */
int xfthip_model_logits(xfthip_model_t m, const float **logits_dev);

/* first-maximum argmax over rows of fp32 logits [rows, cols] (sampling.cpp:22-131) */
int xfthip_argmax(const float *logits, int rows, int cols, int *ids_dev, xfthip_stream_t stream);


/* ---- Mixtral-style sparse MLP ------------------------------------------------------- */
typedef struct xfthip_moe *xfthip_moe_t;
/*
 * Top-2 expert selection per token over fp32 logits [M, E]: strict '>' scan (the lower index wins
 * ties), weights = softmax over the two selected logits.  sel: int32 [M, 2], weights: fp32 [M, 2]
 * (device).  Replaces MixtralMLP::selectTop2Experts (src/layers/mlp_mixtral.h:221-283).
 */
int xfthip_moe_top2(const float *logits, int M, int E, int *sel, float *weights, xfthip_stream_t stream);
/*
 * One sparse MLP block: RMSNorm (eps 1e-6) -> router GEMM (fp32 router weights, host
 * [hidden, experts]) -> top-2 -> per expert: gather, SwiGLU MLP, out += w * expert_out; the output
 * starts as the input (residual).  Replaces MixtralMLP::forward (mlp_mixtral.h:85-187).  Expert
 * weights: gateup [hidden, 2*intermediate] created with XFTHIP_WF_GATEUP, down [intermediate, hidden].
 * logits_override: optional device fp32 [tokens, experts] used instead of the router GEMM.
 * sel_host_out / w_host_out: optional host copies of the routing decision; asking for either makes the call
 * wait for the stream once.  Without them the call only enqueues work (the per-expert row counts stay in device
 * memory, where the expert GEMMs read them) and may be recorded into a graph.  The workspace of one xfthip_moe
 * serves one call at a time: calls on the same object must be ordered on one stream.  x_out may be x_in itself
 * (same pointer and stride: the result is then written over the input); buffers that overlap in any other way are
 * not supported.
 */
int xfthip_moe_create(int hidden, int intermediate, int experts, int max_tokens, const float *router_host, const float *ln_host,
        xfthip_moe_t *out);
/* A further sparse MLP of the same shape that works in the per-call buffers of `first` (the layers of one model run
 * one after the other on one stream): only the router, the norm weight and the experts' table are its own.  `first`
 * must outlive it. */
int xfthip_moe_create_beside(xfthip_moe_t first, const float *router_host, const float *ln_host, xfthip_moe_t *out);
int xfthip_moe_shape(xfthip_moe_t m, int *hidden, int *intermediate, int *experts, int *max_tokens);
int xfthip_moe_destroy(xfthip_moe_t m);
int xfthip_moe_set_expert(xfthip_moe_t m, int e, xfthip_weight_t gateup, xfthip_weight_t down);
int xfthip_moe_forward(xfthip_moe_t m, const float *x_in, int in_stride, float *x_out, int out_stride, int tokens, int do_norm,
        const float *logits_override, int *sel_host_out, float *w_host_out, xfthip_stream_t stream);
/*
 * Layer idx of a model takes this sparse MLP in place of its gate/up/down weights (set its attention half with
 * xfthip_model_set_attention): the layer of MixtralLLM (src/models/mixtral.h:25-54: CommonDecoder over Attention +
 * MixtralMLP).  The object must have been created for at least the model's max_tokens and outlive the model; prompt
 * pass, decode steps (graph replay included) and the per-sequence entry points run it like any other layer.
 */
int xfthip_model_set_moe(xfthip_model_t m, int idx, xfthip_moe_t moe);

#ifdef __cplusplus
}
#endif
#endif /* XFT_HIP_H */
