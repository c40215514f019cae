// Device-side body of the attention kernels.  See attention.hip for the algorithm.
#pragma once
#include "kvcache.h"

namespace xfthip {

// the cache is device memory even when its pointers reach the kernel through a table in memory
#define ATTN_GLOBAL __attribute__((address_space(1)))

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

union HFrag {
    f16x8 v;
    uint32_t u[4];
    u32x4 q;
    h2 h[4];
};

constexpr float kNegBig = -1.0e30f;
constexpr int kWsSlots = 4096; // partial-result slots of the shared workspace
constexpr int kSlotFloats = 16 * 128 + 32;

struct AttnParams {
    KvView kv;
    const uint16_t *q; // bf16
    int qStride;
    void *out;
    int oStride, out_dtype;
    int B, S, G;
    float scale;
    int past;
    const int *past_dev;
    int nsplit, CG;
    float *ws;
    unsigned int *tickets; // one per (batch, kv head, column group), zero between launches; null: the parts are merged by a launch of their own
};

// 4 int8 -> 2 x (2 fp16), exact: (q ^ 0x80) | 0x6400 is 1152 + q, then subtract 1152
__device__ inline void widen_i8x4(uint32_t w, h2 &lo, h2 &hi) {
    const uint32_t x = w ^ 0x80808080u;
    const uint32_t a = __builtin_amdgcn_perm(0x64646464u, x, 0x04010400u);
    const uint32_t b = __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u);
    const h2 off = {(_Float16)1152.0f, (_Float16)1152.0f};
    lo = __builtin_bit_cast(h2, a) - off;
    hi = __builtin_bit_cast(h2, b) - off;
}

__device__ inline uint32_t pack_f16(float a, float b) {
    h2 v = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, v);
}

// LDS the unit needs: AttnLds<NW> (about 8.5 KB per wave).  Every thread of the NW-wave block calls it.
template <int NW>
struct AttnLds {
    float s_m[NW][16], s_l[NW][16];
    float s_o[NW][16][128 + 1];
    unsigned int s_ticket;
};

// wg_sync: a barrier over the block.
// q, the split partials and a bf16 output go through device-coherent accesses (ld_dev / st_dev),
// and the ticket hand-over between the workgroups of a split needs no cache maintenance: the
// alternative, a device-scope fence by every thread, writes back and invalidates the whole L2 of
// the XCD and costs several microseconds per launch.  It also lets the unit run inside a kernel
// whose other workgroups produced q and will consume the output in the same launch (the cache
// rows appended in that launch must then have been written with st_dev as well).
// PIPE: request the next block behind the current block's arithmetic (pays once a wave walks several blocks; with
// one block a wave the plain order is the shorter program)
template <bool INT8, int NW, bool PIPE, typename Sync>
__device__ inline void attn_unit(const AttnParams &p, const int split, const int kvh, const int cg, const int b, AttnLds<NW> &L,
        const Sync &wg_sync) {
    constexpr int D = 128;
    auto &s_m = L.s_m;
    auto &s_l = L.s_l;
    auto &s_o = L.s_o;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, cl = lane & 15;
    int past = p.past;
    if (p.past_dev) {
        // a position read from device memory is held inside the cache whatever it contains
        past = p.past_dev[b];
        past = past < 0 ? 0 : (past > p.kv.S - p.S ? p.kv.S - p.S : past);
    }

    // this lane's column
    const int ncols = p.S * p.G;
    const int c = cg * 16 + cl;
    const bool cvalid = c < ncols;
    const int cs = cvalid ? c / p.G : 0, cj = cvalid ? c % p.G : 0;
    const int limit = cvalid ? past + cs + 1 : 0; // tokens [0, limit) are visible
    int last_col = cg * 16 + 15;
    last_col = last_col < ncols ? last_col : ncols - 1;
    const int lmax = past + last_col / p.G + 1;

    // token-block range of this wave
    const int nblk = (lmax + 31) >> 5;
    const int per = (nblk + p.nsplit - 1) / p.nsplit;
    int wg_begin = split * per, wg_end = wg_begin + per;
    wg_end = wg_end < nblk ? wg_end : nblk;
    wg_begin = wg_begin < wg_end ? wg_begin : wg_end;
    const int wn = wg_end - wg_begin;
    const int wbase = wn / NW, wrem = wn % NW;
    // (the same for every lane of a wave: scalar values, so that the loop and its load branches are uniform)
    const int blk_begin = __builtin_amdgcn_readfirstlane(wg_begin + wave * wbase + (wave < wrem ? wave : wrem));
    const int blk_end = __builtin_amdgcn_readfirstlane(blk_begin + wbase + (wave < wrem ? 1 : 0));
    // A wave walks its blocks from a starting point of its own and wraps around (the online softmax does not care
    // about the order).  With a cache whose rows per head are a power of two long, the waves of all heads and parts
    // would otherwise be at the same offset modulo the memory channels' stripe at every step, on a fraction of the
    // channels (16 sequences x 8 KV heads x 4096 tokens in a cache of 16384: 67.5 us in step, 54 us staggered; INT8
    // 41.6 / 35.7).  The pipelined INT8 form sits at its register limit and spills with the two scalars more that
    // this takes (33 -> 37 us on the same shape in a cache of 4096): it keeps the plain order.
    constexpr bool STAGGER = !(INT8 && PIPE);
    const int wblk = blk_end - blk_begin;
    const int rot = STAGGER
            ? __builtin_amdgcn_readfirstlane(wblk > 1 ? (int)((unsigned)((b * p.kv.H + kvh) * 5 + split * 3 + wave) % (unsigned)wblk) : 0)
            : 0;

    const size_t bh = (size_t)b * p.kv.H + kvh;
    const ATTN_GLOBAL char *kbase = (const ATTN_GLOBAL char *)p.kv.k + bh * p.kv.S * D * (INT8 ? 1 : 2);
    const ATTN_GLOBAL char *vbase = (const ATTN_GLOBAL char *)p.kv.v + bh * p.kv.S * D * (INT8 ? 1 : 2);
    const ATTN_GLOBAL float *ksc = INT8 ? (const ATTN_GLOBAL float *)p.kv.kscale + bh * p.kv.S : nullptr;
    const ATTN_GLOBAL float *vsc = INT8 ? (const ATTN_GLOBAL float *)p.kv.vscale + bh * p.kv.S : nullptr;

    // K (2 token tiles x 4 steps), V (8 dim tiles) and the scales of one block of 32 tokens
    // An INT8 block stays in registers as codes (32 registers instead of 64) and is widened operand by operand
    // right in front of its MFMA: the kernel then fits three workgroups a CU instead of two.
    HFrag kf[INT8 ? 1 : 2][INT8 ? 1 : 4], vf[INT8 ? 1 : 8];
    u32x4 kraw[INT8 ? 2 : 1][INT8 ? 2 : 1];
    u32x2 vraw[INT8 ? 8 : 1];
    f32x4 ks[2], vs[2];
    // The keys of block blk + 1 are requested as soon as the scores of block blk are scaled (the key registers and
    // key scales are free then) and its values once the P.V products of block blk are issued: the next block
    // travels while this one goes through the softmax and the value products, in the same registers.
    auto load_keys = [&](const int blk) {
        const int t0 = blk << 5;
        if constexpr (INT8) {
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                const ATTN_GLOBAL char *row = kbase + (size_t)(t0 + 16 * a + cl) * D + 16 * g;
#pragma unroll
                for (int j = 0; j < 2; ++j) kraw[a][j] = *(const ATTN_GLOBAL u32x4 *)(row + 64 * j);
                ks[a] = *(const ATTN_GLOBAL f32x4 *)(ksc + t0 + 16 * a + 4 * g);
            }
        } else {
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                const ATTN_GLOBAL char *row = kbase + ((size_t)(t0 + 16 * a + cl) * D + 8 * g) * 2;
#pragma unroll
                for (int s = 0; s < 4; ++s) kf[a][s].q = *(const ATTN_GLOBAL u32x4 *)(row + 64 * s);
            }
        }
    };
    auto load_values = [&](const int blk) {
        const int t0 = blk << 5;
        if constexpr (INT8) {
#pragma unroll
            for (int a = 0; a < 2; ++a) vs[a] = *(const ATTN_GLOBAL f32x4 *)(vsc + t0 + 16 * a + 4 * g);
#pragma unroll
            for (int dt = 0; dt < 8; ++dt) vraw[dt] = *(const ATTN_GLOBAL u32x2 *)(vbase + ((size_t)blk * D + 16 * dt + cl) * 32 + 8 * g);
        } else {
#pragma unroll
            for (int dt = 0; dt < 8; ++dt) {
                const ATTN_GLOBAL char *src = vbase + (((size_t)blk * D + 16 * dt + cl) * 32 + 8 * g) * 2;
                vf[dt].q = *(const ATTN_GLOBAL u32x4 *)src;
            }
        }
    };

    // Q fragments (B operand): lane (col, g) holds 8 dims per MFMA step.  The raw loads go out
    // first, then the first block's K / V loads, and only then is q converted, so that the two
    // round trips overlap.
    HFrag qf[4];
    uint32_t qraw[4][4];
    {
        const uint16_t *qrow = p.q + ((size_t)b * p.S + cs) * p.qStride + (size_t)(kvh * p.G + cj) * D;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int d0 = INT8 ? 64 * (s >> 1) + 16 * g + 8 * (s & 1) : 32 * s + 8 * g;
            qraw[s][0] = qraw[s][1] = qraw[s][2] = qraw[s][3] = 0u;
            if (cvalid) {
                ld_dev16(qrow + d0, qraw[s]);
            }
        }
    }
    if (blk_begin < blk_end) {
        load_keys(blk_begin + rot);
        load_values(blk_begin + rot);
    }
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float lo = u2f(qraw[s][i] << 16), hi = u2f(qraw[s][i] & 0xFFFF0000u);
            qf[s].u[i] = pack_f16(lo, hi);
        }

    float m_run = kNegBig, l_run = 0.0f;
    f32x4 o[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = f32x4 {0.f, 0.f, 0.f, 0.f};

    // (one loop for both orders; in the plain order `bi` is dead and the conditions are those of a loop over blk)
    for (int bi = 0, blk = blk_begin + rot; STAGGER ? bi < wblk : blk < blk_end; ++bi) {
        const auto more = [&] { return STAGGER ? bi + 1 < wblk : blk + 1 < blk_end; };
        const auto next = [&] { return (STAGGER && blk + 1 == blk_end) ? blk_begin : blk + 1; };
        const int t0 = blk << 5;
        if constexpr (!PIPE) {
            if (STAGGER ? bi != 0 : blk != blk_begin) {
                load_keys(blk);
                load_values(blk);
            }
        }

        // ---- scores S^T[token = t0 + 16a + 4g + r][col] ----
        f32x4 sc[2];
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            sc[a] = f32x4 {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                if constexpr (INT8) {
                    HFrag k1;
                    widen_i8x4(kraw[a][s >> 1][2 * (s & 1)], k1.h[0], k1.h[1]);
                    widen_i8x4(kraw[a][s >> 1][2 * (s & 1) + 1], k1.h[2], k1.h[3]);
                    sc[a] = __builtin_amdgcn_mfma_f32_16x16x32_f16(k1.v, qf[s].v, sc[a], 0, 0, 0);
                } else {
                    sc[a] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[a][s].v, qf[s].v, sc[a], 0, 0, 0);
                }
            }
        }
        float bmax = kNegBig;
        bool vis[2][4];
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int t = t0 + 16 * a + 4 * g + r;
                vis[a][r] = t < limit;
                float x = sc[a][r];
                if constexpr (INT8) x *= ks[a][r];
                x *= p.scale;
                sc[a][r] = x;
                bmax = fmaxf(bmax, vis[a][r] ? x : kNegBig);
            }
        if constexpr (PIPE) {
            __builtin_amdgcn_sched_barrier(0);
            if (more()) load_keys(next());
            __builtin_amdgcn_sched_barrier(0);
        }
        // column max across the 4 lane groups
        bmax = fmaxf(bmax, __shfl_xor(bmax, 16, 64));
        bmax = fmaxf(bmax, __shfl_xor(bmax, 32, 64));
        const float m_new = fmaxf(m_run, bmax);
        const float alpha = fast_exp(m_run - m_new);
        m_run = m_new;
        float psum = 0.0f;
        float pr[2][4];
        // INT8 values: the per-token scale is folded into the probability, normalised by the
        // block's largest scale so that the fp16 operand stays in [0, 1]
        // (over the tokens this column sees: what lies behind them in the block may be left from an earlier sequence)
        float vmax = 0.0f;
        if constexpr (INT8) {
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int r = 0; r < 4; ++r) vmax = fmaxf(vmax, vis[a][r] ? vs[a][r] : 0.0f);
            vmax = fmaxf(vmax, __shfl_xor(vmax, 16, 64));
            vmax = fmaxf(vmax, __shfl_xor(vmax, 32, 64));
        }
        const float vinv = (INT8 && vmax > 0.0f) ? 1.0f / vmax : 1.0f;
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float e = vis[a][r] ? fast_exp(sc[a][r] - m_new) : 0.0f;
                psum += e;
                pr[a][r] = INT8 ? e * (vs[a][r] * vinv) : e;
            }
        l_run = l_run * alpha + psum;
        HFrag pf;
        pf.u[0] = pack_f16(pr[0][0], pr[0][1]);
        pf.u[1] = pack_f16(pr[0][2], pr[0][3]);
        pf.u[2] = pack_f16(pr[1][0], pr[1][1]);
        pf.u[3] = pack_f16(pr[1][2], pr[1][3]);
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) {
            if constexpr (INT8) {
                HFrag v1;
                widen_i8x4(vraw[dt][0], v1.h[0], v1.h[1]);
                widen_i8x4(vraw[dt][1], v1.h[2], v1.h[3]);
                f32x4 tmp = {0.f, 0.f, 0.f, 0.f};
                tmp = __builtin_amdgcn_mfma_f32_16x16x32_f16(v1.v, pf.v, tmp, 0, 0, 0);
                o[dt] = o[dt] * alpha + tmp * vmax;
            } else {
                o[dt] = o[dt] * alpha;
                o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf[dt].v, pf.v, o[dt], 0, 0, 0);
            }
        }
        if constexpr (PIPE) {
            __builtin_amdgcn_sched_barrier(0);
            if (more()) load_values(next());
            __builtin_amdgcn_sched_barrier(0);
        }
        blk = next();
    }

    // ---- merge the 4 waves in LDS ----
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (g == 0) {
        s_m[wave][cl] = m_run;
        s_l[wave][cl] = l_run;
    }
#pragma unroll
    for (int dt = 0; dt < 8; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) s_o[wave][cl][16 * dt + 4 * g + r] = o[dt][r];
    wg_sync();

    const size_t group = (size_t)(b * p.kv.H + kvh) * p.CG + cg;
    float *slot = p.ws + (group * p.nsplit + split) * kSlotFloats;
    for (int v = threadIdx.x; v < 16 * D; v += 64 * NW) {
        const int col = v / D, d = v % D;
        const int cc = cg * 16 + col;
        if (cc >= ncols) continue;
        float m = s_m[0][col];
#pragma unroll
        for (int w = 1; w < NW; ++w) m = fmaxf(m, s_m[w][col]);
        float l = 0.0f, acc = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const float f = fast_exp(s_m[w][col] - m);
            l += s_l[w][col] * f;
            acc += s_o[w][col][d] * f;
        }
        if (p.nsplit == 1) {
            const int s_tok = cc / p.G, j = cc % p.G;
            const size_t idx = ((size_t)b * p.S + s_tok) * p.oStride + (size_t)(kvh * p.G + j) * D + d;
            if (p.out_dtype == XFTHIP_BF16)
                st_dev((uint16_t *)p.out + idx, f32_to_bf16_ref(acc / l));
            else
                store_from_f32(p.out, p.out_dtype, idx, acc / l);
        } else {
            st_dev(&slot[32 + col * D + d], acc);
            if (d == 0) {
                st_dev(&slot[col], m);
                st_dev(&slot[16 + col], l);
            }
        }
    }
    if (p.nsplit == 1 || p.tickets == nullptr) return; // no tickets: a launch of attn_merge_unit follows

    // ---- the workgroup that finishes last merges the splits of its column group ----
    // (no waiting: every workgroup publishes its partial, takes a ticket and leaves; the one
    // holding the last ticket sees all partials and resets the counter for the next launch)
    unsigned int &s_ticket = L.s_ticket;
    dev_drain();
    wg_sync();
    if (threadIdx.x == 0) s_ticket = atomicAdd(&p.tickets[group], 1u);
    wg_sync();
    if (s_ticket != (unsigned int)(p.nsplit - 1)) return;
    if (threadIdx.x == 0) st_dev(&p.tickets[group], 0u);
    auto ws_ld = [](const float *q) { return ld_dev(q); };
    // factors first (one thread per column, then per (split, column)), so that the wide pass over
    // the partial outputs is a plain weighted sum with independent loads
    const float *base = p.ws + group * p.nsplit * kSlotFloats;
    float *s_f = &s_o[0][0][0]; // [nsplit][16] factors, reusing the output staging area
    float *s_linv = s_f + 64 * 16;
    float *s_pm = s_linv + 16, *s_pl = s_pm + 64 * 16; // [nsplit][16] partial maxima and sums
    // one load per thread (independent round trips), then the per-column arithmetic from LDS
    // (up to 8 a thread at 64 splits: all sent before the first is used)
    // (at up to 8 parts this thread's first output is requested in the same round trip: with one query
    // row a KV head, the decode step of a single sequence, that is the whole merge)
    constexpr int EARLY = 8;
    const bool early = p.nsplit <= EARLY && (int)threadIdx.x < 16 * D && cg * 16 + (int)threadIdx.x / D < ncols;
    float t_early[EARLY];
    {
        constexpr int PER = 64 * 32 / (64 * NW) > 0 ? 64 * 32 / (64 * NW) : 1;
        float x[PER];
        if (early) {
#pragma unroll
            for (int u = 0; u < EARLY; ++u)
                t_early[u] = u < p.nsplit ? ws_ld(&base[(size_t)u * kSlotFloats + 32 + threadIdx.x]) : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int v = threadIdx.x + i * 64 * NW;
            x[i] = v < p.nsplit * 32 ? ws_ld(&base[(size_t)(v >> 5) * kSlotFloats + (v & 31)]) : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int v = threadIdx.x + i * 64 * NW;
            if (v < p.nsplit * 32) {
                const int s = v >> 5, e = v & 31;
                if (e < 16)
                    s_pm[s * 16 + e] = x[i];
                else
                    s_pl[s * 16 + e - 16] = x[i];
            }
        }
    }
    wg_sync();
    if (threadIdx.x < 16) {
        const int col = threadIdx.x;
        float m = kNegBig;
        for (int s = 0; s < p.nsplit; ++s) m = fmaxf(m, s_pm[s * 16 + col]);
        float l = 0.0f;
        for (int s = 0; s < p.nsplit; ++s) {
            const float f = fast_exp(s_pm[s * 16 + col] - m);
            s_f[s * 16 + col] = f;
            l += s_pl[s * 16 + col] * f;
        }
        s_linv[col] = 1.0f / l;
    }
    wg_sync();
    for (int v = threadIdx.x; v < 16 * D; v += 64 * NW) {
        const int col = v / D, d = v % D;
        const int cc = cg * 16 + col;
        if (cc >= ncols) continue;
        float acc = 0.0f;
        if (early && v == (int)threadIdx.x) {
#pragma unroll
            for (int u = 0; u < EARLY; ++u)
                if (u < p.nsplit) acc = fmaf(t_early[u], s_f[u * 16 + col], acc);
        } else
        // 32 partials in flight a thread (4 made the merge of 64 splits a chain of 16 round trips per output)
        for (int s0 = 0; s0 < p.nsplit; s0 += 32) {
            float t[32];
#pragma unroll
            for (int u = 0; u < 32; ++u) t[u] = s0 + u < p.nsplit ? ws_ld(&base[(size_t)(s0 + u) * kSlotFloats + 32 + col * D + d]) : 0.0f;
#pragma unroll
            for (int u = 0; u < 32; ++u)
                if (s0 + u < p.nsplit) acc = fmaf(t[u], s_f[(s0 + u) * 16 + col], acc);
        }
        const int s_tok = cc / p.G, j = cc % p.G;
        const size_t idx = ((size_t)b * p.S + s_tok) * p.oStride + (size_t)(kvh * p.G + j) * D + d;
        if (p.out_dtype == XFTHIP_BF16)
            st_dev((uint16_t *)p.out + idx, f32_to_bf16_ref(acc * s_linv[col]));
        else
            store_from_f32(p.out, p.out_dtype, idx, acc * s_linv[col]);
    }
}



// Merge of the parts of one column as a launch of its own (more than 16 parts: the last workgroup of a column
// group merging them alone would take longer than the finer split saves).  One 128-thread workgroup a column,
// one thread a dim; same arithmetic and order over the parts as the in-kernel merge above.
__device__ inline void attn_merge_unit(const AttnParams &p, const int group, const int col, float *s_pm, float *s_f) {
    constexpr int D = 128;
    const int cg = group % p.CG, kvh = (group / p.CG) % p.kv.H, b = group / (p.CG * p.kv.H);
    const int cc = cg * 16 + col, d = threadIdx.x;
    if (cc >= p.S * p.G) return; // uniform over the workgroup
    const float *base = p.ws + (size_t)group * p.nsplit * kSlotFloats;
    float pm = kNegBig, pl = 0.0f;
    if (d < p.nsplit) {
        pm = ld_dev(&base[(size_t)d * kSlotFloats + col]);
        pl = ld_dev(&base[(size_t)d * kSlotFloats + 16 + col]);
    }
    float acc = 0.0f;
    for (int s0 = 0; s0 < p.nsplit; s0 += 32) {
        float t[32];
#pragma unroll
        for (int u = 0; u < 32; ++u) t[u] = s0 + u < p.nsplit ? ld_dev(&base[(size_t)(s0 + u) * kSlotFloats + 32 + col * D + d]) : 0.0f;
        if (s0 == 0) {
            // factors of all parts (the loads above are in flight meanwhile)
            s_pm[d] = pm;
            __syncthreads();
            float m = kNegBig;
            for (int s = 0; s < p.nsplit; ++s) m = fmaxf(m, s_pm[s]);
            __syncthreads();
            s_f[d] = fast_exp(pm - m);
            s_pm[d] = pl;
            __syncthreads();
        }
#pragma unroll
        for (int u = 0; u < 32; ++u)
            if (s0 + u < p.nsplit) acc = fmaf(t[u], s_f[s0 + u], acc);
    }
    float l = 0.0f;
    for (int s = 0; s < p.nsplit; ++s) l += s_pm[s] * s_f[s];
    const float r = acc * (1.0f / l);
    const int s_tok = cc / p.G, j = cc % p.G;
    const size_t idx = ((size_t)b * p.S + s_tok) * p.oStride + (size_t)(kvh * p.G + j) * D + d;
    if (p.out_dtype == XFTHIP_BF16)
        st_dev((uint16_t *)p.out + idx, f32_to_bf16_ref(r));
    else
        store_from_f32(p.out, p.out_dtype, idx, r);
}

// Exchange with the lanes 16 / 32 away (the other lane groups holding the same column) through the gfx950
// lane-swap instructions: unlike __shfl_xor (ds_bpermute) they do not go through the LDS pipeline, whose
// completion counter would make the caller wait for every LDS read in flight.
__device__ inline float swap16(float x) { // value of lane ^ 16
    const unsigned u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    // rows 0, 2 keep theirs in r[0] and get the neighbour's in r[1]; rows 1, 3 the other way round
    const bool odd = (threadIdx.x & 16) != 0;
    return __uint_as_float(odd ? r[0] : r[1]);
}
__device__ inline float swap32(float x) { // value of lane ^ 32
    const unsigned u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const bool hi = (threadIdx.x & 32) != 0;
    return __uint_as_float(hi ? r[0] : r[1]);
}


// ---- prefill: many columns per (sequence, KV head), K / V blocks shared through LDS (attention_prefill.h) -----
// Layout of a 32-token block in LDS: keys 32 rows of 256 B at a pitch of 272 B, values 128 dim rows of 64 B (token
// slots as in the cache) at a pitch of 80 B, so that the lanes one 128-bit LDS read serves together touch
// different banks.
constexpr int kPfKPitch = 272, kPfVPitch = 80;
constexpr int kPfBufBytes = 32 * kPfKPitch + 128 * kPfVPitch; // 18,944 B per buffer

} // namespace xfthip
