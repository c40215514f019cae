// Attention over a block-paged BF16 KV cache, the data path of xft::invokeAttention
// (reference src/kernels/attention_kernels.cpp:24-157, include/layers_attention.h:22-59).
//
// Cache layout (the caller's, part of that interface): [block_num][block_size][kv_heads][head_size]
// bf16; token t of a sequence lives in block block_table[t / block_size] at row t % block_size; a
// "slot" is block * block_size + row.
//
// Decode (one new token per sequence), as crossAttention does per (sequence, head): the new key and
// value rows go to their slots first, then scores = q . K^T in fp32 over context + 1 tokens,
// softmax(scale * scores) in fp32, out = P . V in fp32, narrowed to bf16.  HBM-bound with one query
// row, so the products run on the vector ALUs: 16 lanes share a token (8 dims each, one 128-bit
// load per lane), a wave covers 4 tokens per load, (max, sum, out) run as an online softmax per
// lane group and are merged through LDS; long contexts are split over workgroups whose partials a
// second kernel merges in a fixed order.
// Where this build departs from the reference's text: sequence b uses query / key / value row b
// (the reference reads row 0 for every sequence: no batch offset at attention_kernels.cpp:51,61,
// right only for batch_size = 1) and query head i uses KV head i / (q_heads / kv_heads) (the
// reference indexes the KV head with the query head, right only without grouped heads).
//
// Prefill: causal self-attention of every sequence over its own new tokens (the reference's
// selfAttention call), through this library's FP16-cache attention kernel on a scratch cache, and
// every token's key / value row stored to its slot (slot_mapping holds one entry per token; the
// reference's closures, marked "TODO: debug and fix", pass only slot_mapping[b]).
#include <map>
#include <mutex>

#include "common.h"

namespace xfthip {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct PagedParams {
    uint16_t *out; // bf16 [batch, o_stride]
    const uint16_t *q; // bf16 [batch, q_stride]
    const uint16_t *kc, *vc; // paged caches
    const int *tables; // [batch, table_stride]
    const int *ctx; // tokens already cached per sequence (the new one excluded)
    float *part; // [batch, q_heads, nsplit, 130]: max, sum, out[128]
    int q_heads, kv_heads, q_stride, o_stride, table_stride, block_size, block_num, nsplit;
    float scale;
};

// rows of the new tokens -> their slots (keys and values), one workgroup per token
__global__ __launch_bounds__(256) void paged_store_kernel(uint16_t *kc, uint16_t *vc, const uint16_t *k, const uint16_t *v,
        const int *slots, int kv_stride, int row_elems, int slot_num) {
    const int tok = blockIdx.x;
    const int slot = slots[tok];
    if (slot < 0 || slot >= slot_num) return; // a slot outside the cache is dropped, never written
    const size_t dst = (size_t)slot * row_elems;
    const uint16_t *ks = k + (size_t)tok * kv_stride, *vs = v + (size_t)tok * kv_stride;
    for (int i = threadIdx.x * 8; i < row_elems; i += blockDim.x * 8) {
        *(u32x4 *)(kc + dst + i) = *(const u32x4 *)(ks + i);
        *(u32x4 *)(vc + dst + i) = *(const u32x4 *)(vs + i);
    }
}

__device__ inline void unpack8(const u32x4 &w, float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = __uint_as_float(w[i] << 16);
        f[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
    }
}

// grid (nsplit, q_heads, batch), 256 threads.  head_size = 128.
__global__ __launch_bounds__(256) void paged_decode_kernel(PagedParams p) {
    constexpr int D = 128, U = 4;
    __shared__ float s_m[16], s_l[16], s_o[16][D];
    const int split = blockIdx.x, hq = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int grp = lane >> 4, sub = lane & 15; // token phase, dims 8 sub .. 8 sub + 7
    const int kvh = hq / (p.q_heads / p.kv_heads);
    // tokens to attend to, the new one included (never more than the table describes)
    const int n = min(max(p.ctx[b], 0) + 1, p.table_stride * p.block_size);
    // tokens of this split: whole 16-token rounds
    const int rounds = (n + 15) / 16;
    const int r0 = (int)((long)rounds * split / p.nsplit), r1 = (int)((long)rounds * (split + 1) / p.nsplit);
    const int *table = p.tables + (size_t)b * p.table_stride;
    const size_t row = (size_t)p.kv_heads * D;

    float q[8];
    unpack8(*(const u32x4 *)(p.q + (size_t)b * p.q_stride + hq * D + sub * 8), q);
    float m = -INFINITY, l = 0.0f, o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int r = r0; r < r1; r += U) {
        u32x4 kk[U], vv[U];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int t = (r + u) * 16 + wave * 4 + grp;
            ok[u] = r + u < r1 && t < n;
            const int tc = ok[u] ? t : 0; // masked lanes read token 0 (always present) and drop it
            const int blk = min(max(table[tc / p.block_size], 0), p.block_num - 1); // a bad table entry reads a valid block
            const size_t at = ((size_t)blk * p.block_size + tc % p.block_size) * row + kvh * D + sub * 8;
            kk[u] = *(const u32x4 *)(p.kc + at);
            vv[u] = *(const u32x4 *)(p.vc + at);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float kf[8], vf[8];
            unpack8(kk[u], kf);
            float s = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) s = fmaf(q[i], kf[i], s);
            s += __shfl_xor(s, 1, 64);
            s += __shfl_xor(s, 2, 64);
            s += __shfl_xor(s, 4, 64);
            s += __shfl_xor(s, 8, 64);
            if (!ok[u]) continue; // uniform over the 16 lanes of a token
            s *= p.scale;
            const float mn = fmaxf(m, s);
            const float c = __expf(m - mn), e = __expf(s - mn); // exp(-inf) = 0 on the first token
            unpack8(vv[u], vf);
            l = l * c + e;
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] = fmaf(e, vf[i], o[i] * c);
            m = mn;
        }
    }
    // merge the 16 (wave, phase) partials of the workgroup
    const int slot = wave * 4 + grp;
    if (sub == 0) s_m[slot] = m, s_l[slot] = l;
#pragma unroll
    for (int i = 0; i < 8; ++i) s_o[slot][sub * 8 + i] = o[i];
    __syncthreads();
    if (threadIdx.x < D) {
        float mm = -INFINITY;
        for (int s = 0; s < 16; ++s) mm = fmaxf(mm, s_m[s]);
        float ll = 0.0f, acc = 0.0f;
        for (int s = 0; s < 16; ++s) {
            const float f = s_m[s] == -INFINITY ? 0.0f : __expf(s_m[s] - mm);
            ll = fmaf(s_l[s], f, ll);
            acc = fmaf(s_o[s][threadIdx.x], f, acc);
        }
        float *dst = p.part + (((size_t)b * p.q_heads + hq) * p.nsplit + split) * (D + 2);
        if (threadIdx.x == 0) dst[0] = mm, dst[1] = ll;
        dst[2 + threadIdx.x] = acc;
    }
}

// grid (q_heads, batch), 128 threads: fixed-order merge of the splits, normalisation, bf16 output
__global__ __launch_bounds__(128) void paged_merge_kernel(PagedParams p) {
    constexpr int D = 128;
    const int hq = blockIdx.x, b = blockIdx.y;
    const float *src = p.part + ((size_t)b * p.q_heads + hq) * p.nsplit * (D + 2);
    float mm = -INFINITY;
    for (int s = 0; s < p.nsplit; ++s) mm = fmaxf(mm, src[(size_t)s * (D + 2)]);
    float ll = 0.0f, acc = 0.0f;
    for (int s = 0; s < p.nsplit; ++s) {
        const float ms = src[(size_t)s * (D + 2)];
        const float f = ms == -INFINITY ? 0.0f : __expf(ms - mm);
        ll = fmaf(src[(size_t)s * (D + 2) + 1], f, ll);
        acc = fmaf(src[(size_t)s * (D + 2) + 2 + threadIdx.x], f, acc);
    }
    p.out[(size_t)b * p.o_stride + hq * D + threadIdx.x] = f32_to_bf16_ref(acc / ll);
}

// q | k | v rows of one sequence -> one fused [tokens, (qH + 2 kvH) * D] bf16 buffer
__global__ __launch_bounds__(256) void paged_fuse_qkv_kernel(uint16_t *qkv, const uint16_t *q, const uint16_t *k, const uint16_t *v,
        int q_stride, int kv_stride, int q_elems, int kv_elems) {
    const int tok = blockIdx.x;
    uint16_t *dst = qkv + (size_t)tok * (q_elems + 2 * kv_elems);
    for (int i = threadIdx.x * 8; i < q_elems; i += blockDim.x * 8) *(u32x4 *)(dst + i) = *(const u32x4 *)(q + (size_t)tok * q_stride + i);
    for (int i = threadIdx.x * 8; i < kv_elems; i += blockDim.x * 8) {
        *(u32x4 *)(dst + q_elems + i) = *(const u32x4 *)(k + (size_t)tok * kv_stride + i);
        *(u32x4 *)(dst + q_elems + kv_elems + i) = *(const u32x4 *)(v + (size_t)tok * kv_stride + i);
    }
}

// Scratch of the paged entry points, grow-only, one set per stream: the context splits and the fused q|k|v rows come
// from stream_scratch, the FP16 scratch cache of the prefill from the table below.
struct PrefillCache {
    xfthip_kvcache_t cache = nullptr;
    int heads = 0, seq = 0;
};
std::mutex g_mu;
std::map<hipStream_t, PrefillCache> g_prefill_cache;

int check_common(const void *out, const void *q, const void *k, const void *v, int q_heads, int kv_heads, int head_size, int q_stride,
        int kv_stride, int o_stride, const void *kc, const void *vc, int block_size) {
    XFT_REQUIRE(out && q && k && v && kc && vc, "xfthip_paged_attention: null argument");
    XFT_REQUIRE(head_size == 128, "xfthip_paged_attention: head size %d unsupported (128 only)", head_size);
    XFT_REQUIRE(q_heads > 0 && kv_heads > 0 && q_heads % kv_heads == 0, "xfthip_paged_attention: bad head counts %d / %d", q_heads, kv_heads);
    XFT_REQUIRE(block_size > 0, "xfthip_paged_attention: bad block size");
    XFT_REQUIRE(q_stride >= q_heads * 128 && kv_stride >= kv_heads * 128 && o_stride >= q_heads * 128, "xfthip_paged_attention: stride too small");
    XFT_REQUIRE(q_stride % 8 == 0 && kv_stride % 8 == 0, "xfthip_paged_attention: strides must be multiples of 8 elements");
    XFT_REQUIRE((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)kc | (uintptr_t)vc) & 15) == 0,
            "xfthip_paged_attention: q, k, v and the caches must be 16-byte aligned");
    return 0;
}

} // namespace
} // namespace xfthip

using namespace xfthip;

extern "C" int xfthip_paged_attention_decode(void *out, const void *q, const void *k, const void *v, int q_heads, int kv_heads,
        int head_size, int q_stride, int kv_stride, int o_stride, float scale, int batch, void *kcache, void *vcache, int block_num,
        int block_size, const int *block_tables, int table_stride, const int *context_lens, const int *slot_mapping,
        int max_context, xfthip_stream_t stream) {
    if (int rc = check_common(out, q, k, v, q_heads, kv_heads, head_size, q_stride, kv_stride, o_stride, kcache, vcache, block_size)) return rc;
    XFT_REQUIRE(batch > 0 && block_tables && context_lens && slot_mapping && table_stride > 0, "xfthip_paged_attention_decode: bad argument");
    XFT_REQUIRE(max_context >= 0 && (long)(max_context / block_size + 1) <= (long)table_stride,
            "xfthip_paged_attention_decode: a context of %d + 1 tokens needs %d table entries a sequence, the table has %d", max_context,
            max_context / block_size + 1, table_stride);
    XFT_REQUIRE(block_num > 0, "xfthip_paged_attention_decode: bad block count");
    hipStream_t st = (hipStream_t)stream;
    // enough workgroups to fill the device, at least 64 tokens a split
    int nsplit = (4 * device_cu_count() + batch * q_heads - 1) / (batch * q_heads);
    const int cap = (max_context + 1 + 63) / 64;
    if (nsplit > cap) nsplit = cap;
    if (nsplit > 64) nsplit = 64;
    if (nsplit < 1) nsplit = 1;
    const size_t need = (size_t)batch * q_heads * nsplit * 130;
    void *part = nullptr;
    if (int rc = stream_scratch(kScratchPagedParts, st, need * sizeof(float), false, &part)) return rc;
    PagedParams p = {};
    p.out = (uint16_t *)out, p.q = (const uint16_t *)q, p.kc = (const uint16_t *)kcache, p.vc = (const uint16_t *)vcache;
    p.tables = block_tables, p.ctx = context_lens, p.part = (float *)part;
    p.q_heads = q_heads, p.kv_heads = kv_heads, p.q_stride = q_stride, p.o_stride = o_stride, p.table_stride = table_stride;
    p.block_size = block_size, p.block_num = block_num, p.nsplit = nsplit, p.scale = scale;
    hipLaunchKernelGGL(paged_store_kernel, dim3(batch), dim3(256), 0, st, (uint16_t *)kcache, (uint16_t *)vcache, (const uint16_t *)k,
            (const uint16_t *)v, slot_mapping, kv_stride, kv_heads * 128, block_num * block_size);
    hipLaunchKernelGGL(paged_decode_kernel, dim3(nsplit, q_heads, batch), dim3(256), 0, st, p);
    hipLaunchKernelGGL(paged_merge_kernel, dim3(q_heads, batch), dim3(128), 0, st, p);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

extern "C" int xfthip_paged_attention_prefill(void *out, const void *q, const void *k, const void *v, int q_heads, int kv_heads,
        int head_size, int q_stride, int kv_stride, int o_stride, float scale, int batch, const int *token_lens_host, void *kcache,
        void *vcache, int block_num, int block_size, const int *slot_mapping, xfthip_stream_t stream) {
    if (int rc = check_common(out, q, k, v, q_heads, kv_heads, head_size, q_stride, kv_stride, o_stride, kcache, vcache, block_size)) return rc;
    XFT_REQUIRE(batch > 0 && token_lens_host && slot_mapping && block_num > 0, "xfthip_paged_attention_prefill: bad argument");
    XFT_REQUIRE(o_stride % 8 == 0, "xfthip_paged_attention_prefill: o_stride must be a multiple of 8 elements");
    hipStream_t st = (hipStream_t)stream;
    int total = 0, longest = 0;
    for (int b = 0; b < batch; ++b) {
        XFT_REQUIRE(token_lens_host[b] > 0, "xfthip_paged_attention_prefill: sequence %d has %d tokens", b, token_lens_host[b]);
        total += token_lens_host[b];
        if (token_lens_host[b] > longest) longest = token_lens_host[b];
    }
    const int q_elems = q_heads * 128, kv_elems = kv_heads * 128, fused = q_elems + 2 * kv_elems;
    void *fused_rows = nullptr;
    if (int rc = stream_scratch(kScratchPagedQkv, st, (size_t)total * fused * 2, false, &fused_rows)) return rc;
    uint16_t *g_qkv = (uint16_t *)fused_rows;
    xfthip_kvcache_t g_cache = nullptr;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        PrefillCache &pc = g_prefill_cache[st];
        if (pc.cache == nullptr || pc.heads != kv_heads || pc.seq < longest) {
            if (pc.cache) {
                XFT_CHECK_HIP(hipDeviceSynchronize());
                (void)xfthip_kvcache_destroy(pc.cache);
                pc.cache = nullptr;
            }
            const int seq = ((longest + 255) / 256) * 256;
            if (int rc = xfthip_kvcache_create(XFTHIP_FP16, 1, kv_heads, seq, 128, &pc.cache)) return rc;
            pc.heads = kv_heads, pc.seq = seq;
        }
        g_cache = pc.cache;
    }
    hipLaunchKernelGGL(paged_store_kernel, dim3(total), dim3(256), 0, st, (uint16_t *)kcache, (uint16_t *)vcache, (const uint16_t *)k,
            (const uint16_t *)v, slot_mapping, kv_stride, kv_elems, block_num * block_size);
    hipLaunchKernelGGL(paged_fuse_qkv_kernel, dim3(total), dim3(256), 0, st, g_qkv, (const uint16_t *)q, (const uint16_t *)k,
            (const uint16_t *)v, q_stride, kv_stride, q_elems, kv_elems);
    XFT_CHECK_HIP(hipGetLastError());
    int first = 0;
    for (int b = 0; b < batch; ++b) {
        const int S = token_lens_host[b];
        uint16_t *rows = g_qkv + (size_t)first * fused;
        if (int rc = xfthip_rope_kvstore(g_cache, rows, XFTHIP_BF16, fused, 1, S, q_heads, nullptr, nullptr, 0, nullptr, stream)) return rc;
        if (int rc = attention_launch(g_cache, rows, fused, (uint16_t *)out + (size_t)first * o_stride, o_stride, XFTHIP_BF16, 1, S, q_heads,
                    scale, 0, nullptr, 0, st, nullptr, false))
            return rc;
        first += S;
    }
    return 0;
}
