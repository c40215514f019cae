// Decoder-layer and whole-model drivers: the order of kernels one Llama-family layer runs,
// the prefill pass and the graph-captured greedy decode step.  Replaces
// Decoder::forwardAttention / forwardFFN, CommonDecoder::forward and greedySearch of the
// reference (src/layers/decoder_layer.h, src/models/common_decoder.h:315-589,
// src/searchers/sampling.cpp:22-131).
//
// Activation flow of one layer (residual stream x in fp32, GEMM operands in bf16):
//   xn  = rmsnorm(x)                       bf16
//   qkv = xn * Wqkv (+bias)                bf16   [tokens, (q + 2 kv) * head]
//   rope(q, k); append k, v to the cache   (k goes to the cache from fp32 registers)
//   att = attention(q, cache)              bf16
//   x   = att * Wo (+bias) + x             fp32   (residual epilogue)
//   xn  = rmsnorm(x, eps 1e-6)             bf16
//   h   = silu(xn * Wgate) * (xn * Wup)    bf16   (fused into the cat GEMM's epilogue)
//   x   = h * Wdown + x                    fp32
#include <string.h>

#include <utility>
#include <vector>

#include "attention_dev.h"
#include "kvcache.h"
#include "qgemm.h"

namespace xfthip {

struct LayerW {
    xfthip_weight_t qkv = nullptr, o = nullptr, gateup = nullptr, down = nullptr;
    // optional second set used by the prompt pass only (the reference's HybridModel: one weight type for the
    // first token, another for the following ones, src/models/hybrid_model.h:25-84)
    xfthip_weight_t first_qkv = nullptr, first_o = nullptr, first_gateup = nullptr, first_down = nullptr;
    float *ln1 = nullptr, *ln2 = nullptr, *qkv_bias = nullptr, *o_bias = nullptr;
    // set: the layer's two norms are LayerNorms with these shifts (NormType::LN of the layer API) instead of RMSNorms
    float *ln1_beta = nullptr, *ln2_beta = nullptr;
    // set: the layer's MLP is this sparse one (MixtralMLP; it carries its own norm weight and router), not gateup / down
    xfthip_moe_t moe = nullptr;
};

__global__ void embed_kernel(const uint16_t *__restrict__ table, const int *__restrict__ ids, float *__restrict__ x,
        int hidden, int vocab) {
    const int tok = blockIdx.x;
    int id = ids[tok];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const uint16_t *row = table + (size_t)id * hidden;
    for (int c = threadIdx.x; c < hidden; c += blockDim.x) x[(size_t)tok * hidden + c] = fp16_bits_to_f32(row[c]);
}

// rows of the last token of every sequence -> compact [B, hidden]
__global__ void gather_last_kernel(const float *__restrict__ x, float *__restrict__ out, int S, int hidden) {
    const int b = blockIdx.x;
    const float *row = x + ((size_t)b * S + S - 1) * hidden;
    for (int c = threadIdx.x; c < hidden; c += blockDim.x) out[(size_t)b * hidden + c] = row[c];
}

// first maximum per row: strict '>' inside a thread's ascending scan, lower index wins ties
// across threads
// advance_pos / advance_step (may be null): the decode step's position and step counters, bumped
// here so that the step needs no launches of its own for them
// active: optional per-row flags; a row whose flag is 0 keeps its id and its position (a sequence
// that sits out this step of a continuously batched decode)
__global__ __launch_bounds__(1024) void argmax_kernel(const float *__restrict__ logits, int cols, int *__restrict__ ids,
        int *advance_pos, int *advance_step, const int *__restrict__ active) {
    __shared__ float sv[1024];
    __shared__ int si[1024];
    const float *p = logits + (size_t)blockIdx.x * cols;
    float bv = -INFINITY;
    int bi = 0x7FFFFFFF;
    auto take = [&](float v, int j) {
        if (v > bv || bi == 0x7FFFFFFF) {
            bv = v;
            bi = j;
        }
    };
    const bool vec = ((cols & 3) == 0) && ((((uintptr_t)p) & 15) == 0);
    if (vec) {
        for (int j = threadIdx.x * 4; j < cols; j += blockDim.x * 4) {
            const float4 v = *(const float4 *)(p + j);
            take(v.x, j), take(v.y, j + 1), take(v.z, j + 2), take(v.w, j + 3);
        }
    } else {
        for (int j = threadIdx.x; j < cols; j += blockDim.x) take(p[j], j);
    }
    sv[threadIdx.x] = bv;
    si[threadIdx.x] = bi;
    __syncthreads();
    for (int s = blockDim.x >> 1; s > 0; s >>= 1) {
        if (threadIdx.x < s) {
            const float ov = sv[threadIdx.x + s];
            const int oi = si[threadIdx.x + s];
            if (ov > sv[threadIdx.x] || (ov == sv[threadIdx.x] && oi < si[threadIdx.x])) {
                sv[threadIdx.x] = ov;
                si[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const bool on = active == nullptr || active[blockIdx.x] != 0;
        if (on) ids[blockIdx.x] = si[0];
        if (advance_pos && on) advance_pos[blockIdx.x] += 1;
        if (advance_step && blockIdx.x == 0) advance_step[0] += 1;
    }
}

// start of a decode step: log the input id of sequence blockIdx.x and embed it
__global__ void decode_begin_kernel(const uint16_t *__restrict__ table, const int *__restrict__ ids, float *__restrict__ x, int hidden,
        int vocab, int *__restrict__ log, const int *__restrict__ step) {
    const int b = blockIdx.x;
    int id = ids[b];
    if (threadIdx.x == 0) log[(size_t)step[0] * gridDim.x + b] = id;
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const uint16_t *row = table + (size_t)id * hidden;
    for (int c = threadIdx.x; c < hidden; c += blockDim.x) x[(size_t)b * hidden + c] = fp16_bits_to_f32(row[c]);
}

// Cache rows copied through a staging buffer (beam search: KVCacheTensor::expandAllSequence and ::reorder,
// reference src/common/kvcache_tensor.h:147-286).  Entry i moves the 32-token blocks [blk0, blk0 + nblk) of
// every head of cache row rows[i]: TO_STAGE reads them into stage[i], otherwise stage[i] is written over them.
// Keys [B][H][S][D] and values [B][H][S/32][D][32] keep a token block at the same offset of a head's
// segment, so one index serves both.  grid (16-byte chunks / 256, heads, 2 * entries), 256 threads.
template <bool TO_STAGE>
__global__ __launch_bounds__(256) void kv_rows_move_kernel(KvView kv, const int *__restrict__ rows, int blk0, int nblk,
        unsigned char *__restrict__ stage) {
    const int esz = kv.int8 ? 1 : 2;
    const size_t seg = (size_t)nblk * 32 * kv.D * esz; // bytes of a head's blocks
    const size_t at = ((size_t)blockIdx.x * 256 + threadIdx.x) * 16;
    if (at >= seg) return;
    const int head = blockIdx.y, i = blockIdx.z >> 1, which = blockIdx.z & 1;
    const int row = rows[i];
    unsigned char *cache = (unsigned char *)(which ? kv.v : kv.k) + (((size_t)row * kv.H + head) * kv.S + (size_t)blk0 * 32) * kv.D * esz + at;
    unsigned char *st = stage + (((size_t)i * 2 + which) * kv.H + head) * seg + at;
    if (TO_STAGE)
        *(uint4 *)st = *(const uint4 *)cache;
    else
        *(uint4 *)cache = *(const uint4 *)st;
}

// the per-token scales of an INT8 cache, same staging scheme; grid (ceil(nblk * 32 / 256), heads, 2 * entries)
template <bool TO_STAGE>
__global__ __launch_bounds__(256) void kv_scales_move_kernel(KvView kv, const int *__restrict__ rows, int blk0, int nblk,
        float *__restrict__ stage) {
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t >= nblk * 32) return;
    const int head = blockIdx.y, i = blockIdx.z >> 1, which = blockIdx.z & 1;
    float *cache = (which ? kv.vscale : kv.kscale) + ((size_t)rows[i] * kv.H + head) * kv.S + (size_t)blk0 * 32 + t;
    float *st = stage + (((size_t)i * 2 + which) * kv.H + head) * ((size_t)nblk * 32) + t;
    if (TO_STAGE)
        *st = *cache;
    else
        *cache = *st;
}

__global__ void fill_int_kernel(int *p, int n, int v) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}


} // namespace xfthip

using namespace xfthip;

struct xfthip_model {
    xfthip_model_config cfg;
    std::vector<LayerW> layers;
    std::vector<xfthip_kvcache_t> caches;
    // INT8 KV: the first-token pass attends over unquantised keys/values, as the reference's
    // flash path does on its bf16 copies (src/layers/attention.h:1121-1188); they live here
    xfthip_kvcache_t prefill_cache = nullptr;
    AttnWorkspace attn_ws; // split-KV partials and tickets of this model's attention launches
    // W8A8 layers: int8 activation rows + per-row (scale, zero, sum), and the [tokens, 2 * inter]
    // bf16 result of the gate/up projection (which runs as a plain GEMM for this kind)
    int8_t *w8a8_qa = nullptr;
    size_t w8a8_qa_bytes = 0;
    float *w8a8_stat = nullptr;
    uint16_t *gu = nullptr;
    float *cosT = nullptr, *sinT = nullptr;
    // scratch
    uint16_t *xn = nullptr, *qkv = nullptr, *att = nullptr, *h = nullptr;
    float *x = nullptr, *xlast = nullptr, *logits = nullptr;
    int *ids = nullptr, *pos = nullptr, *step = nullptr, *idlog = nullptr;
    int idlog_cap = 0;
    // head
    uint16_t *embedding = nullptr;
    float *final_norm = nullptr;
    xfthip_weight_t lm_head = nullptr;
    // decode state
    int cur_B = 0, cur_pos = 0;
    int prompt_rows = 0; // rows of `x` that hold the last layer's output of the most recent prompt pass (0 after a decode step)
    int prefix_len = 0; // positions [0, prefix_len) of cache row 0 hold a shared prefix (xfthip_model_set_prefix)
    // continuous batching: sequences live in cache rows of their own, each at its own position
    int row0 = 0; // cache row of the first sequence of the forward call in flight
    bool ragged = false; // rows may differ in position or sit out a step (set by the xfthip_model_seq_* calls)
    int *active = nullptr; // device [max_batch]: rows taking part in the next decode call
    int *prompt_ids = nullptr; // device [max_tokens]: prompt of a single-sequence prefill
    std::vector<int> row_pos; // host copy of every row's position (-1 = free row)
    unsigned char *kv_stage = nullptr; // staging buffer of xfthip_model_seq_reorder (grown on demand)
    size_t kv_stage_bytes = 0;
    int *reorder_rows = nullptr; // device [2 * max_batch]: source rows, destination rows
    hipGraphExec_t graph = nullptr;
    int graph_B = 0;
    int graph_nsplit = 0; // attention split count the captured step was built with
    bool graph_ragged = false; // the captured step's last node holds the `active` mask only in this mode
    int len_hint = 0; // upper bound of the sequence length during the current decode call (0 = unknown)
    hipStream_t graph_stream = nullptr;
    bool use_graph = true;
    bool fuse_decode = true; // RMSNorm prologue / RoPE + cache-append epilogue inside the decode GEMVs
};

// While one of these lives, the layers that hold first-token weights run with them.
struct FirstTokenWeights {
    xfthip_model *m;
    explicit FirstTokenWeights(xfthip_model *model) : m(model) { swap_all(); }
    ~FirstTokenWeights() { swap_all(); }
    FirstTokenWeights(const FirstTokenWeights &) = delete;
    FirstTokenWeights &operator=(const FirstTokenWeights &) = delete;
    void swap_all() {
        for (LayerW &L : m->layers) {
            if (!L.first_qkv) continue;
            std::swap(L.qkv, L.first_qkv), std::swap(L.o, L.first_o);
            std::swap(L.gateup, L.first_gateup), std::swap(L.down, L.first_down);
        }
    }
};

static int upload_f32(float **dst, const float *src, size_t n) {
    if (*dst) {
        (void)hipFree(*dst);
        *dst = nullptr;
    }
    if (!src) return 0;
    XFT_CHECK_HIP(hipMalloc((void **)dst, n * sizeof(float)));
    XFT_CHECK_HIP(hipMemcpy(*dst, src, n * sizeof(float), hipMemcpyHostToDevice));
    return 0;
}

// fp32 -> bf16 copy of activation rows (the un-normalised GEMM input of the block-level entry points)
__global__ void narrow_rows_kernel(const float *__restrict__ in, int in_stride, uint16_t *__restrict__ out, int cols) {
    const float *row = in + (size_t)blockIdx.x * in_stride;
    uint16_t *orow = out + (size_t)blockIdx.x * cols;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) orow[c] = xfthip::f32_to_bf16_ref(row[c]);
}

// h[t][i] = silu(gu[t][i]) * gu[t][inter + i] on bf16 rows: the SwiGLU of a gate/up projection that
// ran as a plain GEMM (DecoderUtil::siluSum, src/utils/decoder_util.h:550-573)
__global__ void silu_mul_kernel(const uint16_t *__restrict__ gu, uint16_t *__restrict__ h, int inter) {
    const uint16_t *row = gu + (size_t)blockIdx.x * 2 * inter;
    for (int i = threadIdx.x; i < inter; i += blockDim.x) {
        const float g = bf16_to_f32(row[i]), u = bf16_to_f32(row[inter + i]);
        h[(size_t)blockIdx.x * inter + i] = f32_to_bf16_ref(u * (g / (1.0f + fast_exp(-g))));
    }
}

// xfthip_gemm for the model: W8A8 weights quantise their activation rows into the model's own
// scratch (sized at attach time, so nothing is allocated or freed while a captured step exists)
static int model_gemm(xfthip_model *m, xfthip_weight_t w, int M, const void *A, int lda, void *C, int ldc, int c_dtype, int epi,
        const float *bias, const void *res, int ldres, int res_dtype, hipStream_t st) {
    if (w->pw.kind == XFTHIP_W_W8A8) {
        XFT_REQUIRE(m->w8a8_qa != nullptr, "model has a W8A8 weight but no activation scratch");
        const int K = w->pw.K, ldq = (K + 15) / 16 * 16;
        XFT_REQUIRE((size_t)M * ldq <= m->w8a8_qa_bytes, "W8A8 scratch too small for %d rows of %d", M, K);
        float *sA = m->w8a8_stat, *zA = sA + m->cfg.max_tokens, *sumA = zA + m->cfg.max_tokens;
        if (int rc = xfthip_w8a8_quantize_rows(A, XFTHIP_BF16, M, K, lda, m->w8a8_qa, ldq, sA, zA, sumA, st)) return rc;
        return xfthip_gemm_w8a8(w, M, m->w8a8_qa, ldq, sA, zA, sumA, C, ldc, c_dtype, epi, bias, res, ldres, res_dtype, 1.0f, st);
    }
    return xfthip_gemm(w, M, A, lda, C, ldc, c_dtype, epi, bias, res, ldres, res_dtype, 1.0f, st);
}

// grows the model's W8A8 scratch for a weight with K input rows (called when weights are attached)
static int w8a8_reserve(xfthip_model *m, const PackedWeight &pw, bool gateup) {
    if (pw.kind != XFTHIP_W_W8A8) return 0;
    const size_t need = (size_t)m->cfg.max_tokens * ((pw.K + 15) / 16 * 16);
    if (need > m->w8a8_qa_bytes) {
        XFT_CHECK_HIP(hipDeviceSynchronize());
        if (m->w8a8_qa) (void)hipFree(m->w8a8_qa);
        m->w8a8_qa = nullptr;
        XFT_CHECK_HIP(hipMalloc((void **)&m->w8a8_qa, need));
        m->w8a8_qa_bytes = need;
    }
    if (!m->w8a8_stat) XFT_CHECK_HIP(hipMalloc((void **)&m->w8a8_stat, (size_t)m->cfg.max_tokens * 3 * sizeof(float)));
    if (gateup && !m->gu) XFT_CHECK_HIP(hipMalloc((void **)&m->gu, (size_t)m->cfg.max_tokens * pw.N * 2));
    return 0;
}

// attention half of a layer: x_out = Attn(norm?(x_in)) * Wo + bias + x_in
static int attention_block(xfthip_model *m, int idx, const float *x_in, int in_stride, float *x_out, int out_stride, int B,
        int S, int past, const int *past_dev, bool do_norm, hipStream_t st) {
    const xfthip_model_config &c = m->cfg;
    const LayerW &L = m->layers[idx];
    XFT_REQUIRE(L.qkv && L.o, "layer %d has no attention weights attached", idx);
    XFT_REQUIRE(!do_norm || L.ln1, "layer %d has no attention norm weight", idx);
    const int T = B * S;
    const int qcols = c.q_heads * c.head_size, kvcols = c.kv_heads * c.head_size;
    const int qkv_cols = qcols + 2 * kvcols;
    int rc;
    // the B sequences of this call live in cache rows row0 .. row0 + B - 1
    auto rows_of = [&](xfthip_kvcache_t full) {
        xfthip_kvcache v = *full;
        const size_t per_row = (size_t)v.kv.H * v.kv.S * v.kv.D;
        v.kv.k = (char *)v.kv.k + (size_t)m->row0 * per_row * (v.kv.int8 ? 1 : 2);
        v.kv.v = (char *)v.kv.v + (size_t)m->row0 * per_row * (v.kv.int8 ? 1 : 2);
        if (v.kv.kscale) v.kv.kscale += (size_t)m->row0 * v.kv.H * v.kv.S, v.kv.vscale += (size_t)m->row0 * v.kv.H * v.kv.S;
        v.kv.B = full->kv.B - m->row0;
        return v;
    };
    xfthip_kvcache layer_cache = rows_of(m->caches[idx]);
    // Decode step (one new token per sequence, a handful of rows): the norm runs as the QKV
    // GEMV's prologue and the rotation + cache append as its epilogue, which takes two launches
    // (and their gaps) out of every layer.
    const PackedWeight &wq = L.qkv->pw;
    const bool small = m->fuse_decode && wq.kind != XFTHIP_W_W8A8;
    const bool fuse_norm = small && do_norm && !L.ln1_beta && skinny_can_fuse_norm(wq, T);
    const bool fuse_rope = small && S == 1 && T <= 32 && c.kv_dtype == XFTHIP_FP16 && !L.qkv_bias && c.head_size == 128
            && wq.KT * ktile_of(wq.kind) == wq.K;
    if (!fuse_norm) {
        if (do_norm && L.ln1_beta) {
            if ((rc = xfthip_layernorm(m->xn, XFTHIP_BF16, x_in, XFTHIP_F32, L.ln1, L.ln1_beta, T, c.hidden, in_stride, c.hidden, c.rms_eps, st)))
                return rc;
        } else if (do_norm) {
            if ((rc = xfthip_rmsnorm(m->xn, XFTHIP_BF16, x_in, XFTHIP_F32, L.ln1, T, c.hidden, in_stride, c.hidden, c.rms_eps, st))) return rc;
        } else {
            hipLaunchKernelGGL(narrow_rows_kernel, dim3(T), dim3(256), 0, st, x_in, in_stride, m->xn, c.hidden);
        }
    }
    if (fuse_norm || fuse_rope) {
        SkinnyParams sp = {};
        sp.M = T;
        sp.A = m->xn;
        sp.lda = c.hidden;
        sp.C = m->qkv;
        sp.ldc = qkv_cols;
        sp.c_dtype = XFTHIP_BF16;
        sp.epi = L.qkv_bias ? XFTHIP_EPI_BIAS : XFTHIP_EPI_NONE;
        sp.bias = L.qkv_bias;
        sp.gamma = 1.0f;
        if (fuse_norm) {
            sp.norm_x = x_in, sp.ldx = in_stride, sp.norm_w = L.ln1, sp.norm_eps = c.rms_eps;
        }
        if (fuse_rope) {
            sp.rope = 1, sp.cosT = m->cosT, sp.sinT = m->sinT, sp.pos_dev = past_dev, sp.pos_host = past;
            sp.qH = c.q_heads, sp.kvH = c.kv_heads, sp.kv = layer_cache.kv;
        }
        if ((rc = qgemm_skinny(wq, sp, st))) return rc;
    } else {
        if ((rc = model_gemm(m, L.qkv, T, m->xn, c.hidden, m->qkv, qkv_cols, XFTHIP_BF16, L.qkv_bias ? XFTHIP_EPI_BIAS : XFTHIP_EPI_NONE,
                     L.qkv_bias, nullptr, 0, XFTHIP_F32, st)))
            return rc;
    }
    if (!fuse_rope)
        if ((rc = xfthip_rope_kvstore(&layer_cache, m->qkv, XFTHIP_BF16, qkv_cols, B, S, c.q_heads, m->cosT, m->sinT, past, past_dev, st)))
            return rc;
    xfthip_kvcache_t attend = &layer_cache;
    xfthip_kvcache first_pass;
    if (c.kv_dtype == XFTHIP_INT8 && S > 1 && past == 0 && past_dev == nullptr) {
        first_pass = rows_of(m->prefill_cache);
        if ((rc = rope_kvstore_impl(&first_pass, m->qkv, XFTHIP_BF16, qkv_cols, B, S, c.q_heads, m->cosT, m->sinT, 0, nullptr,
                     false, st)))
            return rc;
        attend = &first_pass;
    }
    if ((rc = attention_launch(attend, m->qkv, qkv_cols, m->att, qcols, XFTHIP_BF16, B, S, c.q_heads, 1.0f / sqrtf((float)c.head_size), past,
                 past_dev, past_dev ? m->len_hint : 0, st, &m->attn_ws)))
        return rc;
    return model_gemm(m, L.o, T, m->att, qcols, x_out, out_stride, XFTHIP_F32, XFTHIP_EPI_RESIDENTIAL, L.o_bias, x_in, in_stride,
            XFTHIP_F32, st);
}

// MLP half of a layer: x_out = (silu(xn Wgate) * (xn Wup)) Wdown + x_in, xn = norm?(x_in)
static int mlp_block(xfthip_model *m, int idx, const float *x_in, int in_stride, float *x_out, int out_stride, int T,
        bool do_norm, hipStream_t st) {
    const xfthip_model_config &c = m->cfg;
    const LayerW &L = m->layers[idx];
    if (L.moe) // router, top-2, expert GEMMs and the weighted sum over the residual: only enqueues work
        return xfthip_moe_forward(L.moe, x_in, in_stride, x_out, out_stride, T, do_norm ? 1 : 0, nullptr, nullptr, nullptr, st);
    XFT_REQUIRE(L.gateup && L.down, "layer %d has no MLP weights attached", idx);
    XFT_REQUIRE(!do_norm || L.ln2, "layer %d has no MLP norm weight", idx);
    int rc;
    const PackedWeight &wg = L.gateup->pw;
    // epsilon 1e-6 is hard-coded on the MLP side of the reference (src/layers/mlp_llama.h:212)
    if (m->fuse_decode && do_norm && !L.ln2_beta && wg.kind != XFTHIP_W_W8A8 && skinny_can_fuse_norm(wg, T)) {
        SkinnyParams sp = {};
        sp.M = T;
        sp.A = m->xn;
        sp.lda = c.hidden;
        sp.C = m->h;
        sp.ldc = c.intermediate;
        sp.c_dtype = XFTHIP_BF16;
        sp.gateup = 1;
        sp.norm_x = x_in, sp.ldx = in_stride, sp.norm_w = L.ln2, sp.norm_eps = 1e-6f;
        if ((rc = qgemm_skinny(wg, sp, st))) return rc;
    } else {
        if (do_norm && L.ln2_beta) {
            if ((rc = xfthip_layernorm(m->xn, XFTHIP_BF16, x_in, XFTHIP_F32, L.ln2, L.ln2_beta, T, c.hidden, in_stride, c.hidden, 1e-6f, st)))
                return rc;
        } else if (do_norm) {
            if ((rc = xfthip_rmsnorm(m->xn, XFTHIP_BF16, x_in, XFTHIP_F32, L.ln2, T, c.hidden, in_stride, c.hidden, 1e-6f, st))) return rc;
        } else {
            hipLaunchKernelGGL(narrow_rows_kernel, dim3(T), dim3(256), 0, st, x_in, in_stride, m->xn, c.hidden);
        }
        if (wg.kind == XFTHIP_W_W8A8) {
            // cat(gate, up) as one plain int8 GEMM, then SwiGLU (the reference's own order of work)
            if ((rc = model_gemm(m, L.gateup, T, m->xn, c.hidden, m->gu, 2 * c.intermediate, XFTHIP_BF16, XFTHIP_EPI_NONE, nullptr, nullptr, 0,
                         XFTHIP_F32, st)))
                return rc;
            hipLaunchKernelGGL(silu_mul_kernel, dim3(T), dim3(256), 0, st, m->gu, m->h, c.intermediate);
        } else if ((rc = xfthip_gemm_gateup_silu(L.gateup, T, m->xn, c.hidden, m->h, c.intermediate, XFTHIP_BF16, st))) {
            return rc;
        }
    }
    return model_gemm(m, L.down, T, m->h, c.intermediate, x_out, out_stride, XFTHIP_F32, XFTHIP_EPI_RESIDENTIAL, nullptr, x_in, in_stride,
            XFTHIP_F32, st);
}

// one layer on device buffers (x_in may alias x_out)
static int layer_forward(xfthip_model *m, int idx, const float *x_in, int in_stride, float *x_out, int out_stride, int B,
        int S, int past, const int *past_dev, hipStream_t st) {
    if (int rc = attention_block(m, idx, x_in, in_stride, x_out, out_stride, B, S, past, past_dev, true, st)) return rc;
    return mlp_block(m, idx, x_out, out_stride, x_out, out_stride, B * S, true, st);
}

// final norm + lm_head + greedy pick; advance: also bump the decode step's position / step counters
static int head_forward(xfthip_model *m, const float *xrows, int B, bool advance, hipStream_t st) {
    const xfthip_model_config &c = m->cfg;
    int rc;
    const int r0 = m->row0; // logits, ids and positions of row r0 + b
    // (the norm stays a kernel of its own here: as a prologue of the 2000-tile lm_head GEMV it cost
    // 3 us more than it saved)
    if ((rc = xfthip_rmsnorm(m->xn, XFTHIP_BF16, xrows, XFTHIP_F32, m->final_norm, B, c.hidden, c.hidden, c.hidden, c.rms_eps, st))) return rc;
    if ((rc = xfthip_gemm(m->lm_head, B, m->xn, c.hidden, m->logits + (size_t)r0 * c.vocab, c.vocab, XFTHIP_F32, XFTHIP_EPI_NONE, nullptr,
                 nullptr, 0, XFTHIP_F32, 1.0f, st)))
        return rc;
    hipLaunchKernelGGL(argmax_kernel, dim3(B), dim3(1024), 0, st, m->logits + (size_t)r0 * c.vocab, c.vocab, m->ids + r0,
            advance ? m->pos + r0 : nullptr, advance ? m->step : nullptr, (advance && m->ragged) ? m->active + r0 : nullptr);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

// the decode step that gets captured: everything reads its position from device memory
static int decode_step(xfthip_model *m, int B, hipStream_t st) {
    const xfthip_model_config &c = m->cfg;
    hipLaunchKernelGGL(decode_begin_kernel, dim3(B), dim3(256), 0, st, m->embedding, m->ids, m->x, c.hidden, c.vocab, m->idlog, m->step);
    for (int l = 0; l < c.layers; ++l)
        if (int rc = layer_forward(m, l, m->x, c.hidden, m->x, c.hidden, B, 1, 0, m->pos, st)) return rc;
    return head_forward(m, m->x, B, true, st);
}

extern "C" {

int xfthip_argmax(const float *logits, int rows, int cols, int *ids_dev, xfthip_stream_t stream) {
    XFT_REQUIRE(logits && ids_dev && rows > 0 && cols > 0, "xfthip_argmax: bad argument");
    hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(1024), 0, (hipStream_t)stream, logits, cols, ids_dev, (int *)nullptr, (int *)nullptr,
            (const int *)nullptr);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

int xfthip_model_create(const xfthip_model_config *cfg, xfthip_model_t *out) {
    XFT_REQUIRE(cfg && out, "xfthip_model_create: null argument");
    const xfthip_model_config &c = *cfg;
    XFT_REQUIRE(c.layers > 0 && c.hidden > 0 && c.intermediate > 0, "xfthip_model_create: bad sizes");
    XFT_REQUIRE(c.head_size == 128, "xfthip_model_create: head size %d unsupported (128 only)", c.head_size);
    XFT_REQUIRE(c.q_heads > 0 && c.kv_heads > 0 && c.q_heads % c.kv_heads == 0, "xfthip_model_create: bad head counts");
    XFT_REQUIRE(c.q_heads / c.kv_heads <= 16, "xfthip_model_create: more than 16 query heads per KV head");
    XFT_REQUIRE(c.hidden % 8 == 0 && c.intermediate % 16 == 0, "xfthip_model_create: hidden %% 8 and intermediate %% 16 must be 0");
    XFT_REQUIRE(c.max_batch > 0 && c.max_seq > 0 && c.max_tokens >= c.max_batch, "xfthip_model_create: bad batch/sequence limits");
    XFT_REQUIRE(c.max_pos_embed >= c.max_seq, "xfthip_model_create: max_pos_embed %d < max_seq %d", c.max_pos_embed, c.max_seq);
    xfthip_model *m = new xfthip_model();
    m->cfg = c;
    m->layers.resize(c.layers);
    m->caches.assign(c.layers, nullptr);
    auto fail = [&](int rc) {
        xfthip_model_destroy(m);
        return rc;
    };
    for (int l = 0; l < c.layers; ++l)
        if (int rc = xfthip_kvcache_create(c.kv_dtype, c.max_batch, c.kv_heads, c.max_seq, c.head_size, &m->caches[l])) return fail(rc);
    if (int rc = attention_workspace_create(&m->attn_ws, kWsSlots)) return fail(rc);
    if (c.kv_dtype == XFTHIP_INT8)
        if (int rc = xfthip_kvcache_create(XFTHIP_FP16, c.max_batch, c.kv_heads, c.max_seq, c.head_size, &m->prefill_cache)) return fail(rc);
    // (the tables cover the cache rows up to their padded length: a clamped device position stays inside both)
    const int table_rows = c.max_pos_embed > (c.max_seq + 31) / 32 * 32 ? c.max_pos_embed : (c.max_seq + 31) / 32 * 32;
    if (int rc = xfthip_rope_tables_create(c.head_size, table_rows, c.rope_base, 1.0f, &m->cosT, &m->sinT)) return fail(rc);
    const size_t T = c.max_tokens;
    const size_t qkv_cols = (size_t)(c.q_heads + 2 * c.kv_heads) * c.head_size;
    bool ok = hipMalloc((void **)&m->xn, T * (c.hidden > c.intermediate ? c.hidden : c.intermediate) * 2) == hipSuccess
            && hipMalloc((void **)&m->qkv, T * qkv_cols * 2) == hipSuccess
            && hipMalloc((void **)&m->att, T * c.q_heads * c.head_size * 2) == hipSuccess
            && hipMalloc((void **)&m->h, T * c.intermediate * 2) == hipSuccess
            && hipMalloc((void **)&m->x, T * c.hidden * 4) == hipSuccess
            && hipMalloc((void **)&m->xlast, (size_t)c.max_batch * c.hidden * 4) == hipSuccess
            && hipMalloc((void **)&m->ids, (size_t)(T > 64 ? T : 64) * 4) == hipSuccess
            && hipMalloc((void **)&m->pos, (size_t)c.max_batch * 4) == hipSuccess
            && hipMalloc((void **)&m->step, 64) == hipSuccess;
    if (ok && c.vocab > 0) ok = hipMalloc((void **)&m->logits, (size_t)c.max_batch * c.vocab * 4) == hipSuccess;
    if (!ok) {
        set_error("xfthip_model_create: scratch allocation failed");
        return fail(1);
    }
    // every row starts at position 0 with token 0: a decode step may run over rows that hold no sequence
    if (hipMemset(m->ids, 0, (size_t)(T > 64 ? T : 64) * 4) != hipSuccess || hipMemset(m->pos, 0, (size_t)c.max_batch * 4) != hipSuccess
            || hipMemset(m->step, 0, 64) != hipSuccess) {
        set_error("xfthip_model_create: clearing the position buffers failed");
        return fail(1);
    }
    m->idlog_cap = c.max_seq + 1;
    if (hipMalloc((void **)&m->idlog, (size_t)m->idlog_cap * c.max_batch * 4) != hipSuccess) {
        set_error("xfthip_model_create: id log allocation failed");
        return fail(1);
    }
    *out = m;
    return 0;
}

int xfthip_model_destroy(xfthip_model_t m) {
    if (!m) return 0;
    if (m->graph) (void)hipGraphExecDestroy(m->graph);
    for (auto c : m->caches) xfthip_kvcache_destroy(c);
    xfthip_kvcache_destroy(m->prefill_cache);
    attention_workspace_destroy(&m->attn_ws);
    for (auto &L : m->layers) {
        if (L.ln1) (void)hipFree(L.ln1);
        if (L.ln2) (void)hipFree(L.ln2);
        if (L.ln1_beta) (void)hipFree(L.ln1_beta);
        if (L.ln2_beta) (void)hipFree(L.ln2_beta);
        if (L.qkv_bias) (void)hipFree(L.qkv_bias);
        if (L.o_bias) (void)hipFree(L.o_bias);
    }
    void *bufs[] = {m->w8a8_qa, m->w8a8_stat, m->gu, m->cosT, m->sinT, m->xn, m->qkv, m->att, m->h, m->x, m->xlast, m->logits, m->ids, m->pos, m->step, m->idlog,
            m->embedding, m->final_norm, m->active, m->prompt_ids, m->kv_stage, m->reorder_rows};
    for (void *b : bufs)
        if (b) (void)hipFree(b);
    delete m;
    return 0;
}

int xfthip_model_set_attention(xfthip_model_t m, int idx, xfthip_weight_t qkv, xfthip_weight_t o, const float *ln1_host,
        const float *qkv_bias_host, const float *o_bias_host) {
    XFT_REQUIRE(m && qkv && o, "xfthip_model_set_attention: null argument");
    XFT_REQUIRE(idx >= 0 && idx < m->cfg.layers, "xfthip_model_set_attention: layer %d out of range", idx);
    const xfthip_model_config &c = m->cfg;
    const int qcols = c.q_heads * c.head_size, qkv_cols = qcols + 2 * c.kv_heads * c.head_size;
    XFT_REQUIRE(qkv->pw.K == c.hidden && qkv->pw.N == qkv_cols, "xfthip_model_set_attention: qkv weight is [%d,%d], expected [%d,%d]",
            qkv->pw.K, qkv->pw.N, c.hidden, qkv_cols);
    XFT_REQUIRE(o->pw.K == qcols && o->pw.N == c.hidden, "xfthip_model_set_attention: o weight is [%d,%d], expected [%d,%d]", o->pw.K,
            o->pw.N, qcols, c.hidden);
    LayerW &L = m->layers[idx];
    L.qkv = qkv;
    L.o = o;
    if (int rc = w8a8_reserve(m, qkv->pw, false)) return rc;
    if (int rc = w8a8_reserve(m, o->pw, false)) return rc;
    int rc;
    if ((rc = upload_f32(&L.ln1, ln1_host, c.hidden))) return rc;
    if ((rc = upload_f32(&L.qkv_bias, qkv_bias_host, qkv_cols))) return rc;
    if ((rc = upload_f32(&L.o_bias, o_bias_host, c.hidden))) return rc;
    if (m->graph) {
        (void)hipGraphExecDestroy(m->graph);
        m->graph = nullptr;
    }
    return 0;
}

int xfthip_model_set_mlp(xfthip_model_t m, int idx, xfthip_weight_t gateup, xfthip_weight_t down, const float *ln2_host) {
    XFT_REQUIRE(m && gateup && down, "xfthip_model_set_mlp: null argument");
    XFT_REQUIRE(idx >= 0 && idx < m->cfg.layers, "xfthip_model_set_mlp: layer %d out of range", idx);
    const xfthip_model_config &c = m->cfg;
    // W8A8 gate/up weights stay in plain cat(gate, up) column order: the int8 GEMM has no fused SwiGLU
    const bool gu_w8a8 = gateup->pw.kind == XFTHIP_W_W8A8;
    XFT_REQUIRE(gateup->pw.K == c.hidden && gateup->pw.N == 2 * c.intermediate
                    && (gu_w8a8 ? !(gateup->pw.flags & XFTHIP_WF_GATEUP) : (gateup->pw.flags & XFTHIP_WF_GATEUP) != 0),
            "xfthip_model_set_mlp: gate/up weight must be [%d,%d] created with XFTHIP_WF_GATEUP (W8A8: without it)", c.hidden,
            2 * c.intermediate);
    XFT_REQUIRE(down->pw.K == c.intermediate && down->pw.N == c.hidden, "xfthip_model_set_mlp: down weight is [%d,%d], expected [%d,%d]",
            down->pw.K, down->pw.N, c.intermediate, c.hidden);
    LayerW &L = m->layers[idx];
    L.gateup = gateup;
    L.down = down;
    L.moe = nullptr;
    if (int rc = upload_f32(&L.ln2, ln2_host, c.hidden)) return rc;
    if (int rc = w8a8_reserve(m, gateup->pw, true)) return rc;
    if (int rc = w8a8_reserve(m, down->pw, false)) return rc;
    if (m->graph) {
        (void)hipGraphExecDestroy(m->graph);
        m->graph = nullptr;
    }
    return 0;
}

int xfthip_model_set_moe(xfthip_model_t m, int idx, xfthip_moe_t moe) {
    XFT_REQUIRE(m && moe, "xfthip_model_set_moe: null argument");
    XFT_REQUIRE(idx >= 0 && idx < m->cfg.layers, "xfthip_model_set_moe: layer %d out of range", idx);
    const xfthip_model_config &c = m->cfg;
    int hidden = 0, inter = 0, experts = 0, max_tokens = 0;
    if (int rc = xfthip_moe_shape(moe, &hidden, &inter, &experts, &max_tokens)) return rc;
    XFT_REQUIRE(hidden == c.hidden && inter == c.intermediate, "xfthip_model_set_moe: the sparse MLP is %d x %d, the model %d x %d", hidden, inter,
            c.hidden, c.intermediate);
    XFT_REQUIRE(max_tokens >= c.max_tokens, "xfthip_model_set_moe: the sparse MLP takes %d tokens a call, the model up to %d", max_tokens,
            c.max_tokens);
    LayerW &L = m->layers[idx];
    L.moe = moe;
    L.gateup = L.down = nullptr;
    if (m->graph) {
        (void)hipGraphExecDestroy(m->graph);
        m->graph = nullptr;
    }
    return 0;
}

int xfthip_model_set_layer(xfthip_model_t m, int idx, xfthip_weight_t qkv, xfthip_weight_t o, xfthip_weight_t gateup,
        xfthip_weight_t down, const float *ln1_host, const float *ln2_host, const float *qkv_bias_host,
        const float *o_bias_host) {
    XFT_REQUIRE(ln1_host && ln2_host, "xfthip_model_set_layer: norm weights are required");
    if (int rc = xfthip_model_set_attention(m, idx, qkv, o, ln1_host, qkv_bias_host, o_bias_host)) return rc;
    return xfthip_model_set_mlp(m, idx, gateup, down, ln2_host);
}

int xfthip_model_set_layer_norm_shifts(xfthip_model_t m, int idx, const float *ln1_beta_host, const float *ln2_beta_host) {
    XFT_REQUIRE(m && idx >= 0 && idx < m->cfg.layers, "xfthip_model_set_layer_norm_shifts: bad model or layer");
    LayerW &L = m->layers[idx];
    // a captured decode step holds the kernels of the other norm
    if (m->graph) {
        XFT_CHECK_HIP(hipDeviceSynchronize());
        (void)hipGraphExecDestroy(m->graph);
        m->graph = nullptr;
    }
    XFT_CHECK_HIP(hipDeviceSynchronize());
    if (int rc = upload_f32(&L.ln1_beta, ln1_beta_host, m->cfg.hidden)) return rc; // (a null pointer drops the shift)
    return upload_f32(&L.ln2_beta, ln2_beta_host, m->cfg.hidden);
}

int xfthip_model_set_first_token_weights(xfthip_model_t m, int idx, xfthip_weight_t qkv, xfthip_weight_t o, xfthip_weight_t gateup,
        xfthip_weight_t down) {
    XFT_REQUIRE(m && idx >= 0 && idx < m->cfg.layers, "xfthip_model_set_first_token_weights: bad model or layer");
    LayerW &L = m->layers[idx];
    if (!qkv && !o && !gateup && !down) { // back to one weight set
        L.first_qkv = L.first_o = L.first_gateup = L.first_down = nullptr;
        return 0;
    }
    XFT_REQUIRE(qkv && o && gateup && down, "xfthip_model_set_first_token_weights: all four weights or none");
    XFT_REQUIRE(L.qkv && L.o && L.gateup && L.down, "xfthip_model_set_first_token_weights: set the layer's own weights first");
    const xfthip_model_config &c = m->cfg;
    const bool gu_w8a8 = gateup->pw.kind == XFTHIP_W_W8A8;
    XFT_REQUIRE(qkv->pw.K == L.qkv->pw.K && qkv->pw.N == L.qkv->pw.N && o->pw.K == L.o->pw.K && o->pw.N == L.o->pw.N
                    && gateup->pw.K == c.hidden && gateup->pw.N == 2 * c.intermediate && down->pw.K == c.intermediate && down->pw.N == c.hidden,
            "xfthip_model_set_first_token_weights: shapes differ from the layer's own weights");
    XFT_REQUIRE(gu_w8a8 ? !(gateup->pw.flags & XFTHIP_WF_GATEUP) : (gateup->pw.flags & XFTHIP_WF_GATEUP) != 0,
            "xfthip_model_set_first_token_weights: gate/up weight must be created with XFTHIP_WF_GATEUP (W8A8: without it)");
    if (int rc = w8a8_reserve(m, qkv->pw, false)) return rc;
    if (int rc = w8a8_reserve(m, o->pw, false)) return rc;
    if (int rc = w8a8_reserve(m, gateup->pw, true)) return rc;
    if (int rc = w8a8_reserve(m, down->pw, false)) return rc;
    L.first_qkv = qkv, L.first_o = o, L.first_gateup = gateup, L.first_down = down;
    return 0;
}

int xfthip_model_set_head(xfthip_model_t m, const uint16_t *embedding_fp16_host, const float *final_norm_host,
        xfthip_weight_t lm_head) {
    XFT_REQUIRE(m && embedding_fp16_host && final_norm_host && lm_head, "xfthip_model_set_head: null argument");
    const xfthip_model_config &c = m->cfg;
    XFT_REQUIRE(c.vocab > 0, "xfthip_model_set_head: model was created without a vocabulary");
    XFT_REQUIRE(lm_head->pw.K == c.hidden && lm_head->pw.N == c.vocab, "xfthip_model_set_head: lm_head is [%d,%d], expected [%d,%d]",
            lm_head->pw.K, lm_head->pw.N, c.hidden, c.vocab);
    // a captured decode step holds the addresses of the buffers replaced below
    if (m->graph) {
        XFT_CHECK_HIP(hipDeviceSynchronize());
        (void)hipGraphExecDestroy(m->graph);
        m->graph = nullptr;
    }
    if (m->embedding) (void)hipFree(m->embedding);
    m->embedding = nullptr;
    const size_t eb = (size_t)c.vocab * c.hidden * 2;
    XFT_CHECK_HIP(hipMalloc((void **)&m->embedding, eb));
    XFT_CHECK_HIP(hipMemcpy(m->embedding, embedding_fp16_host, eb, hipMemcpyHostToDevice));
    if (int rc = upload_f32(&m->final_norm, final_norm_host, c.hidden)) return rc;
    m->lm_head = lm_head;
    return 0;
}

static int check_forward(xfthip_model_t m, const char *fn, int idx, const void *x_in, const void *x_out, int in_stride,
        int out_stride, int B, int S, int past) {
    XFT_REQUIRE(m && x_in && x_out, "%s: null argument", fn);
    XFT_REQUIRE(idx >= 0 && idx < m->cfg.layers, "%s: layer %d out of range", fn, idx);
    XFT_REQUIRE(B > 0 && B <= m->cfg.max_batch && S > 0 && B * S <= m->cfg.max_tokens, "%s: B=%d S=%d exceed max_batch=%d / max_tokens=%d",
            fn, B, S, m->cfg.max_batch, m->cfg.max_tokens);
    XFT_REQUIRE(past >= 0 && past + S <= m->cfg.max_seq, "%s: past %d + S %d exceeds max_seq %d", fn, past, S, m->cfg.max_seq);
    XFT_REQUIRE(in_stride >= m->cfg.hidden && out_stride >= m->cfg.hidden, "%s: stride smaller than hidden", fn);
    return 0;
}

int xfthip_model_layer_forward(xfthip_model_t m, int idx, const float *x_in, int in_stride, float *x_out,
        int out_stride, int B, int S, int past, xfthip_stream_t stream) {
    if (int rc = check_forward(m, "xfthip_model_layer_forward", idx, x_in, x_out, in_stride, out_stride, B, S, past)) return rc;
    return layer_forward(m, idx, x_in, in_stride, x_out, out_stride, B, S, past, nullptr, (hipStream_t)stream);
}

int xfthip_model_attention_forward(xfthip_model_t m, int idx, const float *x_in, int in_stride, float *x_out,
        int out_stride, int B, int S, int past, int do_norm, xfthip_stream_t stream) {
    if (int rc = check_forward(m, "xfthip_model_attention_forward", idx, x_in, x_out, in_stride, out_stride, B, S, past)) return rc;
    return attention_block(m, idx, x_in, in_stride, x_out, out_stride, B, S, past, nullptr, do_norm != 0, (hipStream_t)stream);
}

int xfthip_model_mlp_forward(xfthip_model_t m, int idx, const float *x_in, int in_stride, float *x_out, int out_stride,
        int tokens, int do_norm, xfthip_stream_t stream) {
    if (int rc = check_forward(m, "xfthip_model_mlp_forward", idx, x_in, x_out, in_stride, out_stride, 1, 1, 0)) return rc;
    XFT_REQUIRE(tokens > 0 && tokens <= m->cfg.max_tokens, "xfthip_model_mlp_forward: %d tokens exceed max_tokens %d", tokens,
            m->cfg.max_tokens);
    return mlp_block(m, idx, x_in, in_stride, x_out, out_stride, tokens, do_norm != 0, (hipStream_t)stream);
}

// the prompt pass of B sequences of S tokens whose cache rows already hold `past` positions each
static int prompt_pass(xfthip_model_t m, const char *who, const int *ids_host, int B, int S, int past, float *logits_host, hipStream_t st) {
    const xfthip_model_config &c = m->cfg;
    XFT_REQUIRE(m->embedding && m->lm_head, "%s: embedding / lm_head not set", who);
    XFT_REQUIRE(B > 0 && B <= c.max_batch && S > 0 && B * S <= c.max_tokens && past + S <= c.max_seq, "%s: B=%d S=%d past=%d exceed the model limits",
            who, B, S, past);
    FirstTokenWeights first_token(m);
    m->row0 = 0;
    m->ragged = false;
    m->row_pos.assign(c.max_batch, -1);
    for (int b = 0; b < B; ++b) m->row_pos[b] = past + S;
    XFT_CHECK_HIP(hipMemcpyAsync(m->ids, ids_host, (size_t)B * S * 4, hipMemcpyHostToDevice, st));
    hipLaunchKernelGGL(embed_kernel, dim3(B * S), dim3(256), 0, st, m->embedding, m->ids, m->x, c.hidden, c.vocab);
    for (int l = 0; l < c.layers; ++l)
        if (int rc = layer_forward(m, l, m->x, c.hidden, m->x, c.hidden, B, S, past, nullptr, st)) return rc;
    hipLaunchKernelGGL(gather_last_kernel, dim3(B), dim3(256), 0, st, m->x, m->xlast, S, c.hidden);
    if (int rc = head_forward(m, m->xlast, B, false, st)) return rc;
    hipLaunchKernelGGL(fill_int_kernel, dim3((B + 63) / 64), dim3(64), 0, st, m->pos, B, past + S);
    hipLaunchKernelGGL(fill_int_kernel, dim3(1), dim3(64), 0, st, m->step, 1, 0);
    XFT_CHECK_HIP(hipGetLastError());
    XFT_CHECK_HIP(hipStreamSynchronize(st));
    if (logits_host) XFT_CHECK_HIP(hipMemcpy(logits_host, m->logits, (size_t)B * c.vocab * 4, hipMemcpyDeviceToHost));
    m->cur_B = B;
    m->cur_pos = past + S;
    m->prompt_rows = B * S;
    return 0;
}

int xfthip_model_prefill(xfthip_model_t m, const int *ids_host, int B, int S, float *logits_host, xfthip_stream_t stream) {
    XFT_REQUIRE(m && ids_host, "xfthip_model_prefill: null argument");
    m->prefix_len = 0; // cache row 0 is written from position 0
    return prompt_pass(m, "xfthip_model_prefill", ids_host, B, S, 0, logits_host, (hipStream_t)stream);
}

int xfthip_model_set_prefix(xfthip_model_t m, const int *ids_host, int n, xfthip_stream_t stream) {
    XFT_REQUIRE(m && ids_host && n > 0, "xfthip_model_set_prefix: bad argument");
    if (int rc = prompt_pass(m, "xfthip_model_set_prefix", ids_host, 1, n, 0, nullptr, (hipStream_t)stream)) return rc;
    m->prefix_len = n;
    return 0;
}

int xfthip_model_prefill_after_prefix(xfthip_model_t m, const int *ids_host, int B, int S, float *logits_host, xfthip_stream_t stream) {
    XFT_REQUIRE(m && ids_host, "xfthip_model_prefill_after_prefix: null argument");
    XFT_REQUIRE(m->prefix_len > 0, "xfthip_model_prefill_after_prefix: no prefix in the cache (xfthip_model_set_prefix, and no plain prompt pass since)");
    const xfthip_model_config &c = m->cfg;
    XFT_REQUIRE(B > 0 && B <= c.max_batch, "xfthip_model_prefill_after_prefix: batch %d exceeds the model's %d cache rows", B, c.max_batch);
    hipStream_t st = (hipStream_t)stream;
    if (B > 1) {
        // KVCacheManager::expandPrefixCache: every sequence's row starts as a copy of the prefix's positions (whole
        // 32-token blocks; what lies behind the prefix in the last block is overwritten by the pass below)
        std::vector<int> dst(B - 1), src(B - 1, 0);
        for (int b = 1; b < B; ++b) dst[b - 1] = b;
        for (int l = 0; l < c.layers; ++l)
            if (int rc = xfthip_kvcache_reorder(m->caches[l], dst.data(), src.data(), B - 1, 0, m->prefix_len, stream)) return rc;
    }
    const int keep = m->prefix_len;
    if (int rc = prompt_pass(m, "xfthip_model_prefill_after_prefix", ids_host, B, S, keep, logits_host, st)) return rc;
    m->prefix_len = keep;
    return 0;
}

int xfthip_model_decode(xfthip_model_t m, int steps, int *ids_out_host, xfthip_stream_t stream) {
    XFT_REQUIRE(m && steps > 0, "xfthip_model_decode: bad argument");
    XFT_REQUIRE(m->cur_B > 0, "xfthip_model_decode: call xfthip_model_prefill first");
    const xfthip_model_config &c = m->cfg;
    XFT_REQUIRE(m->cur_pos + steps <= c.max_seq, "xfthip_model_decode: position %d + %d steps exceeds max_seq %d", m->cur_pos, steps,
            c.max_seq);
    XFT_REQUIRE(steps <= m->idlog_cap, "xfthip_model_decode: too many steps for the id log");
    hipStream_t st = (hipStream_t)stream;
    const int B = m->cur_B;
    m->prompt_rows = 0; // the step overwrites the residual rows of the prompt pass
    hipLaunchKernelGGL(fill_int_kernel, dim3(1), dim3(64), 0, st, m->step, 1, 0);
    // the positions are read from device memory, but the attention split count is fixed at launch
    // (capture) time: it follows an upper bound of the length, rounded up so that the graph is
    // re-captured only every 128 tokens
    m->len_hint = ((m->cur_pos + steps + 127) / 128) * 128;
    const int nsplit = attention_split_count(m->len_hint < c.max_seq ? m->len_hint : c.max_seq, B * c.kv_heads);
    if (!m->use_graph) {
        for (int i = 0; i < steps; ++i)
            if (int rc = decode_step(m, B, st)) return rc;
    } else if (m->graph == nullptr || m->graph_B != B || m->graph_stream != st || m->graph_nsplit != nsplit
            || m->graph_ragged != m->ragged) {
        if (m->graph) {
            (void)hipGraphExecDestroy(m->graph);
            m->graph = nullptr;
        }
        // Capture needs a real stream; every position-dependent value is read from device
        // memory, so the same graph serves every later step.
        hipStream_t cap = st;
        bool own = false;
        if (cap == nullptr) {
            XFT_CHECK_HIP(hipStreamCreate(&cap));
            own = true;
            XFT_CHECK_HIP(hipDeviceSynchronize());
        }
        hipGraph_t g = nullptr;
        // A step at more than 32 rows, or with sparse MLPs, may split K: the parts go to the scratch of the stream the
        // graph will be launched on (not of the capture stream, which may be a temporary one), which has to exist
        // before the capture starts.
        ScratchKeyScope scratch_of_launch_stream(st);
        if (int rc0 = qgemm_split_reserve(st)) return rc0;
        XFT_CHECK_HIP(hipStreamBeginCapture(cap, hipStreamCaptureModeThreadLocal));
        int rc = decode_step(m, B, cap);
        hipError_t e = hipStreamEndCapture(cap, &g);
        if (rc != 0 || e != hipSuccess) {
            if (g) (void)hipGraphDestroy(g);
            if (own) (void)hipStreamDestroy(cap);
            if (rc == 0) set_error("xfthip_model_decode: graph capture failed: %s", hipGetErrorString(e));
            return rc ? rc : 1;
        }
        e = hipGraphInstantiate(&m->graph, g, nullptr, nullptr, 0);
        (void)hipGraphDestroy(g);
        if (own) (void)hipStreamDestroy(cap);
        XFT_CHECK_HIP(e);
        m->graph_B = B;
        m->graph_nsplit = nsplit;
        m->graph_ragged = m->ragged;
        m->graph_stream = st;
    }
    if (m->use_graph)
        for (int i = 0; i < steps; ++i) XFT_CHECK_HIP(hipGraphLaunch(m->graph, st));
    XFT_CHECK_HIP(hipStreamSynchronize(st));
    if (ids_out_host) {
        // the log holds the input id of every step; the outputs are rows 1..steps-1 plus the final ids
        std::vector<int> log((size_t)steps * B);
        XFT_CHECK_HIP(hipMemcpy(log.data(), m->idlog, log.size() * 4, hipMemcpyDeviceToHost));
        for (int i = 0; i + 1 < steps; ++i) memcpy(ids_out_host + (size_t)i * B, log.data() + (size_t)(i + 1) * B, (size_t)B * 4);
        XFT_CHECK_HIP(hipMemcpy(ids_out_host + (size_t)(steps - 1) * B, m->ids, (size_t)B * 4, hipMemcpyDeviceToHost));
    }
    m->cur_pos += steps;
    for (int b = 0; b < B && b < (int)m->row_pos.size(); ++b)
        if (m->row_pos[b] >= 0 && !m->ragged) m->row_pos[b] += steps;
    return 0;
}

// ---- continuous batching: sequences come and go, each in a cache row of its own ------------------
int xfthip_model_seq_prefill(xfthip_model_t m, int row, const int *ids_host, int S, float *logits_host, xfthip_stream_t stream) {
    XFT_REQUIRE(m && ids_host, "xfthip_model_seq_prefill: null argument");
    const xfthip_model_config &c = m->cfg;
    XFT_REQUIRE(m->embedding && m->lm_head, "xfthip_model_seq_prefill: embedding / lm_head not set");
    XFT_REQUIRE(row >= 0 && row < c.max_batch, "xfthip_model_seq_prefill: row %d outside the %d cache rows", row, c.max_batch);
    XFT_REQUIRE(S > 0 && S <= c.max_tokens && S < c.max_seq, "xfthip_model_seq_prefill: %d tokens exceed max_tokens %d / max_seq %d", S,
            c.max_tokens, c.max_seq);
    hipStream_t st = (hipStream_t)stream;
    if (row == 0) m->prefix_len = 0; // the row of a shared prefix is written from position 0
    if ((int)m->row_pos.size() != c.max_batch) m->row_pos.assign(c.max_batch, -1);
    if (!m->active) {
        XFT_CHECK_HIP(hipMalloc((void **)&m->active, (size_t)c.max_batch * 4));
        XFT_CHECK_HIP(hipMemset(m->active, 0, (size_t)c.max_batch * 4));
    }
    if (!m->prompt_ids) XFT_CHECK_HIP(hipMalloc((void **)&m->prompt_ids, (size_t)c.max_tokens * 4));
    if (!m->ragged) {
        // leaving lockstep mode: no row holds a sequence, all sit at position 0 with token 0
        XFT_CHECK_HIP(hipDeviceSynchronize());
        XFT_CHECK_HIP(hipMemset(m->pos, 0, (size_t)c.max_batch * 4));
        XFT_CHECK_HIP(hipMemset(m->ids, 0, (size_t)c.max_batch * 4));
        m->row_pos.assign(c.max_batch, -1);
        m->cur_B = 0;
    }
    m->ragged = true;
    FirstTokenWeights first_token(m);
    XFT_CHECK_HIP(hipMemcpyAsync(m->prompt_ids, ids_host, (size_t)S * 4, hipMemcpyHostToDevice, st));
    hipLaunchKernelGGL(embed_kernel, dim3(S), dim3(256), 0, st, m->embedding, m->prompt_ids, m->x, c.hidden, c.vocab);
    m->row0 = row;
    int rc = 0;
    for (int l = 0; l < c.layers && rc == 0; ++l) rc = layer_forward(m, l, m->x, c.hidden, m->x, c.hidden, 1, S, 0, nullptr, st);
    if (rc == 0) {
        hipLaunchKernelGGL(gather_last_kernel, dim3(1), dim3(256), 0, st, m->x, m->xlast, S, c.hidden);
        rc = head_forward(m, m->xlast, 1, false, st);
    }
    m->row0 = 0;
    if (rc) return rc;
    hipLaunchKernelGGL(fill_int_kernel, dim3(1), dim3(64), 0, st, m->pos + row, 1, S);
    XFT_CHECK_HIP(hipGetLastError());
    XFT_CHECK_HIP(hipStreamSynchronize(st));
    if (logits_host) XFT_CHECK_HIP(hipMemcpy(logits_host, m->logits + (size_t)row * c.vocab, (size_t)c.vocab * 4, hipMemcpyDeviceToHost));
    m->row_pos[row] = S;
    if (row + 1 > m->cur_B) m->cur_B = row + 1;
    m->prompt_rows = S;
    return 0;
}

int xfthip_model_seq_release(xfthip_model_t m, int row) {
    XFT_REQUIRE(m && row >= 0 && row < m->cfg.max_batch, "xfthip_model_seq_release: bad row");
    if ((int)m->row_pos.size() != m->cfg.max_batch) m->row_pos.assign(m->cfg.max_batch, -1);
    m->row_pos[row] = -1;
    // a free row keeps decoding along (at position 0, results dropped) until the rows above it are free too
    XFT_CHECK_HIP(hipDeviceSynchronize());
    int zero = 0;
    if (m->pos) XFT_CHECK_HIP(hipMemcpy(m->pos + row, &zero, 4, hipMemcpyHostToDevice));
    if (m->ids) XFT_CHECK_HIP(hipMemcpy(m->ids + row, &zero, 4, hipMemcpyHostToDevice));
    int top = 0;
    for (int r = 0; r < m->cfg.max_batch; ++r)
        if (m->row_pos[r] >= 0) top = r + 1;
    m->cur_B = top;
    return 0;
}

int xfthip_model_seq_decode(xfthip_model_t m, const int *rows_host, int n, int *ids_out_host, xfthip_stream_t stream) {
    XFT_REQUIRE(m && rows_host && n > 0, "xfthip_model_seq_decode: bad argument");
    const xfthip_model_config &c = m->cfg;
    XFT_REQUIRE(m->ragged && m->active, "xfthip_model_seq_decode: no sequence was started with xfthip_model_seq_prefill");
    std::vector<int> act(c.max_batch, 0);
    int top = 0, deepest = 0;
    for (int i = 0; i < n; ++i) {
        const int r = rows_host[i];
        XFT_REQUIRE(r >= 0 && r < c.max_batch && m->row_pos[r] >= 0, "xfthip_model_seq_decode: row %d holds no sequence", r);
        XFT_REQUIRE(m->row_pos[r] + 1 <= c.max_seq, "xfthip_model_seq_decode: row %d is at position %d of %d", r, m->row_pos[r], c.max_seq);
        XFT_REQUIRE(act[r] == 0, "xfthip_model_seq_decode: row %d listed twice", r);
        act[r] = 1;
    }
    for (int r = 0; r < c.max_batch; ++r)
        if (m->row_pos[r] >= 0) {
            top = r + 1;
            if (m->row_pos[r] > deepest) deepest = m->row_pos[r];
        }
    hipStream_t st = (hipStream_t)stream;
    XFT_CHECK_HIP(hipMemcpyAsync(m->active, act.data(), (size_t)c.max_batch * 4, hipMemcpyHostToDevice, st));
    XFT_CHECK_HIP(hipStreamSynchronize(st));
    // one step over rows 0 .. top - 1; the split count of the attention follows the deepest row
    m->cur_B = top;
    m->cur_pos = deepest;
    if (int rc = xfthip_model_decode(m, 1, nullptr, stream)) return rc;
    for (int i = 0; i < n; ++i) m->row_pos[rows_host[i]] += 1;
    if (ids_out_host) {
        std::vector<int> all(top);
        XFT_CHECK_HIP(hipMemcpy(all.data(), m->ids, (size_t)top * 4, hipMemcpyDeviceToHost));
        for (int i = 0; i < n; ++i) ids_out_host[i] = all[rows_host[i]];
    }
    return 0;
}

// One cache on its own: row dst_rows_host[i] becomes a copy of row src_rows_host[i] over positions
// [pos0, pos1) (whole 32-token blocks); everything is read before anything is written.  The staging
// buffer lives for the call (not a hot path: the model driver keeps its own).
int xfthip_kvcache_reorder(xfthip_kvcache_t cache, const int *dst_rows_host, const int *src_rows_host, int n, int pos0, int pos1,
        xfthip_stream_t stream) {
    XFT_REQUIRE(cache && dst_rows_host && src_rows_host && n > 0, "xfthip_kvcache_reorder: bad argument");
    const KvView &kv = cache->kv;
    XFT_REQUIRE(pos0 >= 0 && pos0 <= pos1 && pos1 <= cache->maxSeq, "xfthip_kvcache_reorder: positions [%d, %d) outside the cache (%d)", pos0, pos1,
            cache->maxSeq);
    std::vector<char> seen(kv.B, 0);
    for (int i = 0; i < n; ++i) {
        const int d = dst_rows_host[i], s = src_rows_host[i];
        XFT_REQUIRE(d >= 0 && d < kv.B && s >= 0 && s < kv.B, "xfthip_kvcache_reorder: row outside the %d cache rows", kv.B);
        XFT_REQUIRE(!seen[d], "xfthip_kvcache_reorder: destination row %d listed twice", d);
        seen[d] = 1;
    }
    if (pos1 == pos0) return 0;
    hipStream_t st = (hipStream_t)stream;
    const int blk0 = pos0 / 32, nblk = (pos1 + 31) / 32 - blk0;
    const int esz = kv.int8 ? 1 : 2;
    const size_t seg = (size_t)nblk * 32 * kv.D * esz;
    const size_t need = (size_t)n * 2 * kv.H * seg + (kv.int8 ? (size_t)n * 2 * kv.H * nblk * 32 * sizeof(float) : 0);
    unsigned char *stage = nullptr;
    int *rows = nullptr;
    XFT_CHECK_HIP(hipMalloc((void **)&stage, need));
    if (hipMalloc((void **)&rows, (size_t)2 * n * 4) != hipSuccess) {
        (void)hipFree(stage);
        XFT_REQUIRE(false, "xfthip_kvcache_reorder: out of device memory");
    }
    bool ok = hipMemcpy(rows, src_rows_host, (size_t)n * 4, hipMemcpyHostToDevice) == hipSuccess
            && hipMemcpy(rows + n, dst_rows_host, (size_t)n * 4, hipMemcpyHostToDevice) == hipSuccess;
    if (ok) {
        float *stage_scales = (float *)(stage + (size_t)n * 2 * kv.H * seg);
        const dim3 grid((unsigned)((seg / 16 + 255) / 256), kv.H, 2 * n), sgrid((nblk * 32 + 255) / 256, kv.H, 2 * n);
        hipLaunchKernelGGL(kv_rows_move_kernel<true>, grid, dim3(256), 0, st, kv, rows, blk0, nblk, stage);
        if (kv.int8) hipLaunchKernelGGL(kv_scales_move_kernel<true>, sgrid, dim3(256), 0, st, kv, rows, blk0, nblk, stage_scales);
        hipLaunchKernelGGL(kv_rows_move_kernel<false>, grid, dim3(256), 0, st, kv, rows + n, blk0, nblk, stage);
        if (kv.int8) hipLaunchKernelGGL(kv_scales_move_kernel<false>, sgrid, dim3(256), 0, st, kv, rows + n, blk0, nblk, stage_scales);
        ok = hipGetLastError() == hipSuccess && hipStreamSynchronize(st) == hipSuccess;
    }
    (void)hipFree(stage);
    (void)hipFree(rows);
    XFT_REQUIRE(ok, "xfthip_kvcache_reorder: device error");
    return 0;
}

int xfthip_model_seq_reorder(xfthip_model_t m, const int *dst_rows_host, const int *src_rows_host, int n, int pos0, int pos1,
        xfthip_stream_t stream) {
    XFT_REQUIRE(m && dst_rows_host && src_rows_host && n > 0, "xfthip_model_seq_reorder: bad argument");
    const xfthip_model_config &c = m->cfg;
    XFT_REQUIRE(m->ragged && n <= c.max_batch, "xfthip_model_seq_reorder: needs sequences started with xfthip_model_seq_prefill, at most %d entries",
            c.max_batch);
    XFT_REQUIRE(pos0 >= 0 && pos0 <= pos1 && pos1 <= c.max_seq, "xfthip_model_seq_reorder: positions [%d, %d) outside the cache (%d)", pos0, pos1,
            c.max_seq);
    std::vector<char> seen(c.max_batch, 0);
    bool identity = true;
    for (int i = 0; i < n; ++i) {
        const int d = dst_rows_host[i], s = src_rows_host[i];
        XFT_REQUIRE(d >= 0 && d < c.max_batch && s >= 0 && s < c.max_batch, "xfthip_model_seq_reorder: row outside the %d cache rows", c.max_batch);
        XFT_REQUIRE(m->row_pos[s] >= 0, "xfthip_model_seq_reorder: source row %d holds no sequence", s);
        XFT_REQUIRE(!seen[d], "xfthip_model_seq_reorder: destination row %d listed twice", d);
        seen[d] = 1;
        identity = identity && d == s;
    }
    hipStream_t st = (hipStream_t)stream;
    // every destination takes over its source's position and next token
    std::vector<int> pos_new(n), ids_all(c.max_batch), ids_new(n);
    for (int i = 0; i < n; ++i) pos_new[i] = m->row_pos[src_rows_host[i]];
    XFT_CHECK_HIP(hipStreamSynchronize(st));
    XFT_CHECK_HIP(hipMemcpy(ids_all.data(), m->ids, (size_t)c.max_batch * 4, hipMemcpyDeviceToHost));
    for (int i = 0; i < n; ++i) ids_new[i] = ids_all[src_rows_host[i]];
    for (int i = 0; i < n; ++i) {
        const int d = dst_rows_host[i];
        m->row_pos[d] = pos_new[i];
        XFT_CHECK_HIP(hipMemcpy(m->pos + d, &pos_new[i], 4, hipMemcpyHostToDevice));
        XFT_CHECK_HIP(hipMemcpy(m->ids + d, &ids_new[i], 4, hipMemcpyHostToDevice));
        if (d + 1 > m->cur_B) m->cur_B = d + 1;
    }
    if (identity || pos1 == pos0) return 0;
    const int blk0 = pos0 / 32, nblk = (pos1 + 31) / 32 - blk0;
    const KvView &k0 = m->caches[0]->kv;
    const int esz = k0.int8 ? 1 : 2;
    const size_t seg = (size_t)nblk * 32 * k0.D * esz;
    const size_t need = (size_t)n * 2 * k0.H * seg + (k0.int8 ? (size_t)n * 2 * k0.H * nblk * 32 * sizeof(float) : 0);
    XFT_REQUIRE((size_t)(blk0 + nblk) * 32 <= (size_t)k0.S, "xfthip_model_seq_reorder: blocks past the cache rows");
    if (need > m->kv_stage_bytes) {
        if (m->kv_stage) (void)hipFree(m->kv_stage);
        m->kv_stage = nullptr, m->kv_stage_bytes = 0;
        XFT_CHECK_HIP(hipMalloc((void **)&m->kv_stage, need));
        m->kv_stage_bytes = need;
    }
    if (!m->reorder_rows) XFT_CHECK_HIP(hipMalloc((void **)&m->reorder_rows, (size_t)2 * c.max_batch * 4));
    XFT_CHECK_HIP(hipMemcpy(m->reorder_rows, src_rows_host, (size_t)n * 4, hipMemcpyHostToDevice));
    XFT_CHECK_HIP(hipMemcpy(m->reorder_rows + c.max_batch, dst_rows_host, (size_t)n * 4, hipMemcpyHostToDevice));
    float *stage_scales = (float *)(m->kv_stage + (size_t)n * 2 * k0.H * seg);
    const dim3 grid((unsigned)((seg / 16 + 255) / 256), k0.H, 2 * n), sgrid((nblk * 32 + 255) / 256, k0.H, 2 * n);
    for (int l = 0; l < c.layers; ++l) {
        const KvView &kv = m->caches[l]->kv;
        hipLaunchKernelGGL(kv_rows_move_kernel<true>, grid, dim3(256), 0, st, kv, m->reorder_rows, blk0, nblk, m->kv_stage);
        if (kv.int8) hipLaunchKernelGGL(kv_scales_move_kernel<true>, sgrid, dim3(256), 0, st, kv, m->reorder_rows, blk0, nblk, stage_scales);
        hipLaunchKernelGGL(kv_rows_move_kernel<false>, grid, dim3(256), 0, st, kv, m->reorder_rows + c.max_batch, blk0, nblk, m->kv_stage);
        if (kv.int8)
            hipLaunchKernelGGL(kv_scales_move_kernel<false>, sgrid, dim3(256), 0, st, kv, m->reorder_rows + c.max_batch, blk0, nblk, stage_scales);
    }
    XFT_CHECK_HIP(hipGetLastError());
    XFT_CHECK_HIP(hipStreamSynchronize(st));
    return 0;
}

int xfthip_model_seq_set_next_id(xfthip_model_t m, int row, int id) {
    XFT_REQUIRE(m && row >= 0 && row < m->cfg.max_batch && m->ids, "xfthip_model_seq_set_next_id: bad row");
    XFT_REQUIRE(id >= 0 && id < m->cfg.vocab, "xfthip_model_seq_set_next_id: id %d outside the vocabulary", id);
    XFT_CHECK_HIP(hipMemcpy(m->ids + row, &id, 4, hipMemcpyHostToDevice));
    return 0;
}

int xfthip_model_seq_logits(xfthip_model_t m, int row, float *logits_host) {
    XFT_REQUIRE(m && logits_host && row >= 0 && row < m->cfg.max_batch && m->logits, "xfthip_model_seq_logits: bad argument");
    XFT_CHECK_HIP(hipMemcpy(logits_host, m->logits + (size_t)row * m->cfg.vocab, (size_t)m->cfg.vocab * 4, hipMemcpyDeviceToHost));
    return 0;
}

int xfthip_model_decode_mode(xfthip_model_t m) {
    if (!m) return -1;
    return m->use_graph ? 1 : 0;
}

int xfthip_model_use_fusion(xfthip_model_t m, int enable) {
    XFT_REQUIRE(m != nullptr, "xfthip_model_use_fusion: null model");
    m->fuse_decode = enable != 0;
    if (m->graph) {
        (void)hipGraphExecDestroy(m->graph);
        m->graph = nullptr;
    }
    return 0;
}

int xfthip_model_use_graph(xfthip_model_t m, int enable) {
    XFT_REQUIRE(m != nullptr, "xfthip_model_use_graph: null model");
    m->use_graph = enable != 0;
    return 0;
}

int xfthip_model_last_ids(xfthip_model_t m, int *ids_host, int *position) {
    XFT_REQUIRE(m && m->cur_B > 0, "xfthip_model_last_ids: nothing generated yet");
    if (ids_host) XFT_CHECK_HIP(hipMemcpy(ids_host, m->ids, (size_t)m->cur_B * 4, hipMemcpyDeviceToHost));
    if (position) *position = m->cur_pos;
    return 0;
}

int xfthip_model_set_next_ids(xfthip_model_t m, const int *ids_host, xfthip_stream_t stream) {
    XFT_REQUIRE(m && ids_host, "xfthip_model_set_next_ids: null argument");
    XFT_REQUIRE(m->cur_B > 0, "xfthip_model_set_next_ids: call xfthip_model_prefill first");
    for (int b = 0; b < m->cur_B; ++b)
        XFT_REQUIRE(ids_host[b] >= 0 && ids_host[b] < m->cfg.vocab, "xfthip_model_set_next_ids: id %d of sequence %d outside the vocabulary",
                ids_host[b], b);
    XFT_CHECK_HIP(hipMemcpyAsync(m->ids, ids_host, (size_t)m->cur_B * 4, hipMemcpyHostToDevice, (hipStream_t)stream));
    XFT_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int xfthip_model_prompt_logits(xfthip_model_t m, int first_row, int rows, float *logits_host, xfthip_stream_t stream) {
    XFT_REQUIRE(m && logits_host && m->lm_head && m->final_norm, "xfthip_model_prompt_logits: bad argument or no head");
    XFT_REQUIRE(first_row >= 0 && rows > 0 && first_row + rows <= m->prompt_rows,
            "xfthip_model_prompt_logits: rows [%d, %d) outside the %d rows of the last prompt pass (a decode step discards them)", first_row,
            first_row + rows, m->prompt_rows);
    const xfthip_model_config &c = m->cfg;
    hipStream_t st = (hipStream_t)stream;
    // final norm + lm_head over the prompt's residual rows, a chunk at a time through a buffer that lives for the
    // call (not a hot path: the reference's logitsAll = true serves scoring, not generation)
    const int chunk = rows < 256 ? rows : 256;
    float *tmp = nullptr;
    XFT_CHECK_HIP(hipMalloc((void **)&tmp, (size_t)chunk * c.vocab * 4));
    int rc = 0;
    for (int r = 0; r < rows && rc == 0; r += chunk) {
        const int n = rows - r < chunk ? rows - r : chunk;
        const float *x = m->x + (size_t)(first_row + r) * c.hidden;
        rc = xfthip_rmsnorm(m->xn, XFTHIP_BF16, x, XFTHIP_F32, m->final_norm, n, c.hidden, c.hidden, c.hidden, c.rms_eps, st);
        if (rc == 0)
            rc = xfthip_gemm(m->lm_head, n, m->xn, c.hidden, tmp, c.vocab, XFTHIP_F32, XFTHIP_EPI_NONE, nullptr, nullptr, 0, XFTHIP_F32, 1.0f, st);
        if (rc == 0 && hipMemcpyAsync(logits_host + (size_t)r * c.vocab, tmp, (size_t)n * c.vocab * 4, hipMemcpyDeviceToHost, st) != hipSuccess) {
            set_error("xfthip_model_prompt_logits: copy to the host failed");
            rc = 1;
        }
        if (rc == 0 && hipStreamSynchronize(st) != hipSuccess) {
            set_error("xfthip_model_prompt_logits: the stream failed");
            rc = 1;
        }
    }
    (void)hipFree(tmp);
    return rc;
}

int xfthip_model_logits(xfthip_model_t m, const float **logits_dev) {
    XFT_REQUIRE(m && logits_dev && m->logits, "xfthip_model_logits: no logits");
    *logits_dev = m->logits;
    return 0;
}

} // extern "C"
