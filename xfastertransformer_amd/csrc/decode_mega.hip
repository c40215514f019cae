// Persistent whole-step decode kernel: one launch runs embedding, all decoder layers, the final
// norm, lm_head and greedy argmax for a batch of up to 4 sequences (INT8 weight-only layers,
// FP16 KV cache, head size 128).  The same arithmetic as the per-kernel path (qgemm_skinny,
// rmsnorm, rope_kv, attention) with the launches replaced by device-wide barriers, because at
// batch 1 a layer's ten kernels cost more in launch gaps (about 2.6 us each) than in HBM time.
//
// Grid: one 512-thread workgroup per compute unit, all co-resident.  A layer is five phases:
//   P1  RMSNorm (every workgroup normalises the M rows into its LDS) + QKV GEMV; the epilogue
//       applies RoPE (column tiles are processed in (d, d+64) pairs) and appends K / V to the cache
//   P2  split-KV attention (attn_unit)
//   P3  out-projection GEMV + residual
//   P4  RMSNorm + gate/up GEMV + SwiGLU
//   P5  down GEMV + residual
// Work items of a phase (a column tile or a pair of them) are dealt round-robin to the
// workgroups; the 8 waves of a workgroup split K.  Activations always sit in LDS (normalised or
// copied there after the barrier), weights stream straight from the packed tiles into registers.
//
// The weight stream never waits for a barrier: a wave's loads form "chunks" of 8 tiles (8 KiB),
// two chunks are in flight, and chunks 0 and 1 of the NEXT phase are issued inside the barrier
// that ends the current one (weights do not depend on other workgroups).
//
// All GEMV phases run through ONE copy of the staging / streaming / epilogue code, driven by a
// phase descriptor: an earlier version with one specialised copy per phase was 91 KB of code,
// more than the 64 KB instruction cache, and lost more to instruction fetch than it won.
//
// The barrier is a two-level atomic counter (per blockIdx % 8, then global; zeroed by a tiny
// kernel before each launch) with a bounded spin: when the bound is hit the abort flag is raised
// and every workgroup leaves at its next barrier, so the grid always drains.  Activations, new
// cache rows, attention partials and logits cross between workgroups through device-coherent
// accesses (ld_dev / st_dev), so no barrier flushes or invalidates an L2.
#include "attention_dev.h"
#include "decode_mega.h"

namespace xfthip {

typedef uint32_t mu32x4 __attribute__((ext_vector_type(4)));
// Pointers read out of the per-layer table are generic to the compiler; everything they point at
// is device memory, and saying so keeps the loads on the global path (vmcnt only).
#define XFT_GLOBAL __attribute__((address_space(1)))
#define XFT_LDS __attribute__((address_space(3)))
template <class T>
__device__ inline XFT_GLOBAL T *gptr(T *p) {
    return (XFT_GLOBAL T *)p;
}
__device__ inline float mg_round_bf16(float f) {
    return bf16_to_f32(f32_to_bf16_ref(f));
}
union MgFrag {
    bf16x8 v;
    uint32_t u[4];
    mu32x4 q;
};

__device__ inline uint32_t mg_pack_hi16(float lo, float hi) {
    return __builtin_amdgcn_perm(f2u(hi), f2u(lo), 0x07060302u);
}

// threadIdx.x behind an optimisation barrier: address arithmetic derived from it stays inside
// the phase that uses it instead of being hoisted out of the layer loop, where dozens of
// per-phase addresses would be live at once
__device__ inline int opaque_tid() {
    int t = threadIdx.x;
    asm volatile("" : "+v"(t));
    return t;
}

__device__ inline float mg_silu(float x) {
    return x / (1.0f + fast_exp(-x));
}

// ---- LDS map (dynamic allocation) ---------------------------------------------------------
//   [0, 128)    part[4][8]  per-row, per-wave sums of squares
//   [128, 132)  flag        barrier outcome
//   [256, ...)  either AttnLds<8> (attention phase) or
//               act[M][pitch] bf16 activations followed by red[8][4][48] fp32 K-slice partials
constexpr int kLdsHeader = 256;
constexpr int kRedCols = 48;
struct MegaLds {
    XFT_LDS float *part;
    XFT_LDS int *flag;
    XFT_LDS uint16_t *act;
    XFT_LDS float *red;
};

size_t mega_lds_bytes(int M, int act_pitch) {
    size_t g = (((size_t)M * act_pitch * 2 + 15) & ~(size_t)15) + (size_t)8 * 4 * kRedCols * 4;
    if (g < sizeof(AttnLds<8>)) g = sizeof(AttnLds<8>);
    return kLdsHeader + g;
}

// ---- phase descriptor ------------------------------------------------------------------------
// An item is a pair of "streams" of 1 KiB weight tiles that share the item's activations:
//   kb == 4: two column tiles over the same k range (RoPE pair, V pair, gate/up pair)
//   kb == 8: one column tile, its k range interleaved over the two streams (their sums are added)
// A chunk is 4 steps x 2 streams = 8 loads per wave and covers kb k-tiles; an item's chunks are
// dealt to the 8 waves in contiguous runs.  Every wave walks the same number of chunk slots per
// item (nslot) so that the block barriers at the item ends line up.
enum { PH_QKV = 0, PH_O = 1, PH_GU = 2, PH_DOWN = 3, PH_HEAD = 4 };
struct PhaseDesc {
    int kind, layer;
    const XFT_GLOBAL uint8_t *w; // packed tiles
    int KT, K, kb;
    int nitems; // items of this workgroup
    int nslot, ch_begin, ch_n; // chunk slots per item; this wave's run of chunks
};

__device__ inline PhaseDesc setup_phase(const MegaParams &p, int step) {
    PhaseDesc d;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wg = blockIdx.x, G = gridDim.x;
    int total;
    if (step >= 4 * p.nlayers) {
        d.kind = PH_HEAD, d.layer = 0;
        d.w = gptr(p.lm_head), d.KT = p.kt_lm, d.K = p.hidden, d.kb = 8, total = (p.vocab + 15) / 16;
    } else {
        d.kind = step & 3, d.layer = step >> 2;
        const MegaLayer &ly = p.layers[d.layer];
        if (d.kind == PH_QKV) {
            d.w = gptr(ly.wqkv), d.KT = ly.kt_qkv, d.K = p.hidden, d.kb = 4, total = (p.qH + 2 * p.kvH) * 4;
        } else if (d.kind == PH_O) {
            d.w = gptr(ly.wo), d.KT = ly.kt_o, d.K = p.qH * 128, d.kb = 8, total = p.hidden / 16;
        } else if (d.kind == PH_GU) {
            d.w = gptr(ly.wgu), d.KT = ly.kt_gu, d.K = p.hidden, d.kb = 4, total = p.inter / 16;
        } else {
            d.w = gptr(ly.wdown), d.KT = ly.kt_down, d.K = p.inter, d.kb = 8, total = p.hidden / 16;
        }
    }
    d.nitems = wg < total ? (total - wg + G - 1) / G : 0;
    const int nchunk = (d.KT + d.kb - 1) / d.kb;
    const int base = nchunk >> 3, rem = nchunk & 7;
    d.ch_begin = wave * base + (wave < rem ? wave : rem);
    d.ch_n = base + (wave < rem ? 1 : 0);
    d.nslot = base + (rem ? 1 : 0);
    return d;
}

// column tiles of the two streams of item `it`
__device__ inline void item_tiles(const MegaParams &p, const PhaseDesc &d, int it, int &t0, int &t1) {
    if (d.kind == PH_QKV) {
        const int RP = (p.qH + p.kvH) * 4;
        if (it < RP) {
            t0 = (it >> 2) * 8 + (it & 3), t1 = t0 + 4; // dims d and d + 64 of one head: a rotation pair
        } else {
            t0 = (p.qH + p.kvH) * 8 + 2 * (it - RP), t1 = t0 + 1;
        }
    } else if (d.kind == PH_GU) {
        t0 = 2 * it, t1 = t0 + 1; // gate and up tiles are interleaved in the packed layout
    } else {
        t0 = t1 = it;
    }
}

// k-tile of (step u, stream s) within a chunk that starts at k-tile kt0
__device__ inline int chunk_kt(const PhaseDesc &d, int kt0, int u, int s) {
    return d.kb == 4 ? kt0 + u : kt0 + 2 * u + s;
}

// issues chunk slot c (8 loads) into buf; returns false when this wave has nothing there
__device__ inline bool issue_chunk(const MegaParams &p, const PhaseDesc &d, mu32x4 (&buf)[8], int c) {
    const int r = c / d.nslot, j = c - r * d.nslot;
    if (r >= d.nitems || j >= d.ch_n) return false;
    const int tid = opaque_tid();
    const unsigned int lane16 = (tid & 63u) * 16u;
    int t0, t1;
    item_tiles(p, d, blockIdx.x + r * gridDim.x, t0, t1);
    const int kt0 = (d.ch_begin + j) * d.kb;
    const XFT_GLOBAL uint8_t *base0 = d.w + (size_t)t0 * d.KT * 1024, *base1 = d.w + (size_t)t1 * d.KT * 1024;
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            int kt = chunk_kt(d, kt0, u, s2);
            kt = kt < d.KT ? kt : d.KT - 1;
            buf[2 * u + s2] = __builtin_nontemporal_load((const XFT_GLOBAL mu32x4 *)((s2 ? base1 : base0) + (size_t)kt * 1024 + lane16));
        }
    return true;
}

// BF16W: the tiles hold bf16 values (32 k per tile) instead of INT8 codes (64 k per tile)
template <bool BF16W>
__device__ inline void compute_chunk(const PhaseDesc &d, const mu32x4 (&buf)[8], int j, f32x4 (&acc)[2], const XFT_LDS uint16_t *arow) {
    constexpr int KTILE = BF16W ? 32 : 64, KL = BF16W ? 8 : 16, MPT = BF16W ? 1 : 2;
    if (j >= d.ch_n) return;
    const int tid = opaque_tid();
    const int g = (tid & 63) >> 4;
    const int kt0 = (d.ch_begin + j) * d.kb;
    const bool full = (kt0 + d.kb) * KTILE <= d.K; // only an item's last chunk can reach past K
    const XFT_LDS uint16_t *abase = arow + g * KL;
    // activation fragments of one (step, stream) slot, fetched one slot ahead of their use
    auto fetch = [&](int slot, MgFrag(&dst)[MPT]) {
        const int kt = chunk_kt(d, kt0, slot >> 1, slot & 1);
#pragma unroll
        for (int i = 0; i < MPT; ++i) {
            const int koff = kt * KTILE + 8 * i;
            const bool valid = full || (kt < d.KT && koff + g * KL + 8 <= d.K);
            dst[i].q = *(const XFT_LDS mu32x4 *)(abase + (valid ? koff : 0));
            if (!full) dst[i].q = valid ? dst[i].q : mu32x4 {0u, 0u, 0u, 0u};
        }
    };
    MgFrag an[MPT];
    fetch(0, an);
#pragma unroll
    for (int slot = 0; slot < 8; ++slot) {
        MgFrag ac[MPT];
#pragma unroll
        for (int i = 0; i < MPT; ++i) ac[i] = an[i];
        if (slot + 1 < 8) fetch(slot + 1, an);
        MgFrag src;
        src.q = buf[slot];
#pragma unroll
        for (int i = 0; i < MPT; ++i) {
            MgFrag w;
            if constexpr (BF16W) {
                w.q = src.q;
            } else {
                const uint32_t c0 = src.u[2 * i], c1 = src.u[2 * i + 1];
                w.u[0] = mg_pack_hi16((float)(int)(int8_t)(c0), (float)(int)(int8_t)(c0 >> 8));
                w.u[1] = mg_pack_hi16((float)(int)(int8_t)(c0 >> 16), (float)((int)c0 >> 24));
                w.u[2] = mg_pack_hi16((float)(int)(int8_t)(c1), (float)(int)(int8_t)(c1 >> 8));
                w.u[3] = mg_pack_hi16((float)(int)(int8_t)(c1 >> 16), (float)((int)c1 >> 24));
            }
            if (slot & 1)
                acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w.v, ac[i].v, acc[1], 0, 0, 0);
            else
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w.v, ac[i].v, acc[0], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0); // keeps the LDS reads of later slots from piling up in registers
    }
}

// ---- device-wide barrier -----------------------------------------------------------------
// When `next` is given, the first two weight chunks of that phase are issued here so that HBM
// keeps streaming while the workgroup waits.  They come AFTER this wave's stores in program order,
// and the wave then waits until at most those 8 loads are outstanding: memory operations retire
// in order, so the stores have been acknowledged and the loads are still in flight.  The wave
// that runs the barrier protocol (wave 0) must not have them in flight (waiting for an atomic's
// result would wait for its older loads as well): it issues its share after the barrier, behind
// the activation loads of the staging step.
__device__ inline bool grid_barrier(const MegaParams &p, unsigned int &phase, const MegaLds &L, const PhaseDesc *next, mu32x4 (&wb)[2][8]) {
    const bool sync_wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) == 0;
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    bool issued = false;
    if (next && !sync_wave) issued = issue_chunk(p, *next, wb[0], 0);
    __builtin_amdgcn_sched_barrier(0);
    if (issued)
        __builtin_amdgcn_s_waitcnt(0x0F78); // vmcnt(8)
    else
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
    if (next && !sync_wave) issue_chunk(p, *next, wb[1], 1);
    __syncthreads();
    ++phase;
    if (threadIdx.x == 0) {
        int ok = 1;
        const unsigned int grp = blockIdx.x & 7u;
        const unsigned int members = (gridDim.x - grp + 7u) >> 3; // workgroups with this blockIdx % 8
        const unsigned int groups = gridDim.x < 8u ? gridDim.x : 8u;
        const unsigned int old = atomicAdd(&p.counter[64 * (1 + grp)], 1u);
        if (old == phase * members - 1u) atomicAdd(&p.counter[0], 1u);
        const unsigned int target = phase * groups;
        unsigned int spins = 0;
        while (__hip_atomic_load(&p.counter[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
            __builtin_amdgcn_s_sleep(1);
            if (++spins > p.spin_limit || __hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
                __hip_atomic_store(p.abort_flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                ok = 0;
                break;
            }
        }
        *L.flag = ok;
        if (p.trace && blockIdx.x == 0 && phase < (unsigned int)p.trace_cap) p.trace[phase] = wall_clock64();
    }
    __syncthreads();
    return *L.flag != 0;
}

// four residual-stream values written by other workgroups
__device__ inline f32x4 ld_x4(const float *p) {
    uint32_t r[4];
    ld_dev16(p, r);
    return f32x4 {u2f(r[0]), u2f(r[1]), u2f(r[2]), u2f(r[3])};
}

// the sync wave's share of the first two chunks, issued behind the staging loads
__device__ inline void late_chunks(const MegaParams &p, const PhaseDesc &d, mu32x4 (&wb)[2][8]) {
    if (__builtin_amdgcn_readfirstlane(threadIdx.x >> 6) == 0) {
        issue_chunk(p, d, wb[0], 0);
        issue_chunk(p, d, wb[1], 1);
    }
}

// ---- RMSNorm of the M rows of x into LDS (bf16); hidden <= 8192 -------------------------------
__device__ inline void stage_norm(const MegaParams &p, const PhaseDesc &d, const float *weight, float eps, const MegaLds &L,
        mu32x4 (&wb)[2][8]) {
    typedef uint32_t mu32x2 __attribute__((ext_vector_type(2)));
    const int tid = opaque_tid();
    const int H = p.hidden;
    const int lane = tid & 63, wave = tid >> 6;
    f32x4 lnw[4]; // this thread's slice of the weight, issued with the first row's loads: one round trip for both
    for (int m = 0; m < p.M; ++m) {
        f32x4 v[4];
        float sq = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = (tid + 512 * i) * 4;
            v[i] = f32x4 {0.f, 0.f, 0.f, 0.f};
            if (c < H) v[i] = ld_x4(p.x + (size_t)m * H + c);
        }
        if (m == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int c = (tid + 512 * i) * 4;
                lnw[i] = f32x4 {0.f, 0.f, 0.f, 0.f};
                if (c < H) lnw[i] = *(const XFT_GLOBAL f32x4 *)gptr(weight + c);
            }
            late_chunks(p, d, wb);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) sq = fmaf(v[i][0], v[i][0], fmaf(v[i][1], v[i][1], fmaf(v[i][2], v[i][2], fmaf(v[i][3], v[i][3], sq))));
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sq += __shfl_xor(sq, off, 64);
        if (lane == 0) L.part[(m & 1) * 8 + wave] = sq;
        __syncthreads();
        float tot = 0.0f;
#pragma unroll
        for (int w = 0; w < 8; ++w) tot += L.part[(m & 1) * 8 + w];
        const float var = 1.0f / sqrtf(tot / (float)H + eps);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = (tid + 512 * i) * 4;
            if (c < H) {
                const f32x4 w = lnw[i];
                const uint32_t lo = f32_to_bf16_ref((v[i][0] * var) * w[0]) | ((uint32_t)f32_to_bf16_ref((v[i][1] * var) * w[1]) << 16);
                const uint32_t hi = f32_to_bf16_ref((v[i][2] * var) * w[2]) | ((uint32_t)f32_to_bf16_ref((v[i][3] * var) * w[3]) << 16);
                *(XFT_LDS mu32x2 *)(L.act + (size_t)m * p.act_pitch + c) = mu32x2 {lo, hi};
            }
        }
    }
    __syncthreads();
}

// ---- copy M rows of K bf16 values written by other workgroups into LDS ------------------------
__device__ inline void stage_copy(const MegaParams &p, const PhaseDesc &d, const uint16_t *src, const MegaLds &L, mu32x4 (&wb)[2][8]) {
    const int tid = opaque_tid();
    const int K = d.K;
    const int per_row = K >> 3, total = p.M * per_row; // 16-byte pieces
    for (int base = 0; base < total; base += 512 * 4) { // uniform trip count: the late issue runs with all lanes
        const int i0 = base + tid;
        uint32_t r[4][4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = i0 + 512 * u;
            if (i < total) {
                const int m = i / per_row, c = (i - m * per_row) << 3;
                ld_dev16(src + (size_t)m * K + c, r[u]);
            }
        }
        if (base == 0) late_chunks(p, d, wb);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = i0 + 512 * u;
            if (i < total) {
                const int m = i / per_row, c = (i - m * per_row) << 3;
                *(XFT_LDS mu32x4 *)(L.act + (size_t)m * p.act_pitch + c) = mu32x4 {r[u][0], r[u][1], r[u][2], r[u][3]};
            }
        }
    }
    if (total == 0) late_chunks(p, d, wb);
    __syncthreads();
}

__device__ inline float sum_red(const MegaLds &L, int m, int c) {
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < 8; ++w) s += L.red[(w * 4 + m) * kRedCols + c];
    return s;
}

// ---- epilogues ----------------------------------------------------------------------------------
// Operands of an item's epilogue (scales, rotation, position, old residual) are fetched when the
// item starts, so that they have arrived by the time its K-slice sums are ready.
struct EpiRegs {
    float s0, s1, cs, sn, xold;
    int pos;
};

__device__ inline void item_begin(const MegaParams &p, const PhaseDesc &d, int it, EpiRegs &e) {
    const int tid = opaque_tid();
    const int M = p.M, c = tid & 15;
    if (d.kind == PH_HEAD) return;
    const MegaLayer &ly = p.layers[d.layer];
    if (d.kind == PH_QKV) {
        const int RP = (p.qH + p.kvH) * 4;
        if (it < RP) {
            if (tid < M * 16) {
                const int t0 = (it >> 2) * 8 + (it & 3), i = (it & 3) * 16 + c;
                e.pos = p.pos[tid >> 4];
                e.s0 = gptr(ly.sqkv)[t0 * 16 + c];
                e.s1 = gptr(ly.sqkv)[(t0 + 4) * 16 + c];
                e.cs = p.cosT[(size_t)e.pos * 64 + i];
                e.sn = p.sinT[(size_t)e.pos * 64 + i];
            }
        } else if (tid < M * 32) {
            e.pos = p.pos[tid >> 5];
            e.s0 = gptr(ly.sqkv)[((p.qH + p.kvH) * 8 + 2 * (it - RP)) * 16 + (tid & 31)];
        }
    } else if (d.kind == PH_GU) {
        if (tid < M * 16) {
            e.s0 = gptr(ly.sgu)[(2 * it) * 16 + c];
            e.s1 = gptr(ly.sgu)[(2 * it + 1) * 16 + c];
        }
    } else if (tid < M * 16) {
        e.xold = ld_dev(p.x + (size_t)(tid >> 4) * p.hidden + it * 16 + c);
        e.s0 = gptr(d.kind == PH_O ? ly.so : ly.sdown)[it * 16 + c];
    }
}

__device__ inline void item_end(const MegaParams &p, const PhaseDesc &d, int it, const EpiRegs &e, const MegaLds &L) {
    const int tid = opaque_tid();
    const int M = p.M, c = tid & 15, m = tid >> 4;
    if (d.kind == PH_HEAD) {
        const int n = it * 16 + c;
        if (tid < M * 16 && n < p.vocab) st_dev(&p.logits[(size_t)m * p.vocab + n], sum_red(L, m, c) + sum_red(L, m, 16 + c));
        return;
    }
    const MegaLayer &ly = p.layers[d.layer];
    if (d.kind == PH_QKV) {
        const int RP = (p.qH + p.kvH) * 4, qcols = p.qH * 128;
        if (it < RP) {
            const int hh = it >> 2, jj = it & 3;
            if (tid < M * 16) {
                // the QKV GEMM output is bf16 in the reference, RoPE works on those values
                const float lo = mg_round_bf16(sum_red(L, m, c) * e.s0);
                const float hi = mg_round_bf16(sum_red(L, m, 16 + c) * e.s1);
                const int i = jj * 16 + c, pos = e.pos;
                const float nlo = fmaf(lo, e.cs, -(hi * e.sn)), nhi = fmaf(hi, e.cs, lo * e.sn);
                if (hh < p.qH) {
                    uint16_t *dst = p.q + (size_t)m * qcols + hh * 128;
                    st_dev(dst + i, f32_to_bf16_ref(nlo));
                    st_dev(dst + i + 64, f32_to_bf16_ref(nhi));
                } else if (pos < ly.kv.S) {
                    const size_t bh = (size_t)m * ly.kv.H + (hh - p.qH);
                    uint16_t *dst = (uint16_t *)ly.kv.k + (bh * ly.kv.S + pos) * 128;
                    st_dev(dst + i, f32_to_fp16_bits(nlo));
                    st_dev(dst + i + 64, f32_to_fp16_bits(nhi));
                }
            }
        } else if (tid < M * 32) {
            const int mv = tid >> 5, cc = tid & 31;
            const int vt = 2 * (it - RP) + (cc >> 4);
            const float val = mg_round_bf16(sum_red(L, mv, cc) * e.s0);
            const int pos = e.pos;
            if (pos < ly.kv.S) {
                const size_t bh = (size_t)mv * ly.kv.H + (vt >> 3);
                const int dd = (vt & 7) * 16 + (cc & 15);
                uint16_t *dst = (uint16_t *)ly.kv.v + (bh * (ly.kv.S / 32) + (pos >> 5)) * (size_t)128 * 32 + (size_t)dd * 32 + v_slot(pos & 31);
                st_dev(dst, f32_to_fp16_bits(val));
            }
        }
    } else if (d.kind == PH_GU) {
        if (tid < M * 16) {
            const float gate = sum_red(L, m, c) * e.s0;
            const float up = sum_red(L, m, 16 + c) * e.s1;
            st_dev(&p.h[(size_t)m * p.inter + it * 16 + c], f32_to_bf16_ref(up * mg_silu(gate)));
        }
    } else if (tid < M * 16) {
        const int n = it * 16 + c;
        st_dev(p.x + (size_t)m * p.hidden + n, e.xold + (sum_red(L, m, c) + sum_red(L, m, 16 + c)) * e.s0);
    }
}

// Runs this workgroup's items of one phase.  On entry chunks 0 and 1 of the phase are already in
// wb[0] / wb[1] (issued by the barrier before it, or by the staging step for the sync wave).
template <bool BF16W>
__device__ inline void run_phase(const MegaParams &p, const PhaseDesc &d, mu32x4 (&wb)[2][8], const MegaLds &L) {
    const int tid = opaque_tid();
    const int lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 4, ml = lane & 15;
    const int row = ml < p.M ? ml : p.M - 1;
    const XFT_LDS uint16_t *arow = L.act + (size_t)row * p.act_pitch;
    const int total = d.nitems * d.nslot;
    f32x4 acc[2];
    EpiRegs e = {};
    int r = 0, j = 0;
    auto step = [&](mu32x4(&buf)[8], int c) {
        const int it = blockIdx.x + r * gridDim.x;
        if (j == 0) {
            acc[0] = acc[1] = f32x4 {0.f, 0.f, 0.f, 0.f};
            item_begin(p, d, it, e);
        }
        compute_chunk<BF16W>(d, buf, j, acc, arow);
        __builtin_amdgcn_sched_barrier(0);
        if (c + 2 < total) issue_chunk(p, d, buf, c + 2);
        __builtin_amdgcn_sched_barrier(0);
        if (++j == d.nslot) {
            if (ml < p.M) {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int q = 0; q < 4; ++q) L.red[(wave * 4 + ml) * kRedCols + t * 16 + 4 * g + q] = acc[t][q];
            }
            __syncthreads();
            item_end(p, d, it, e, L);
            __syncthreads();
            j = 0;
            ++r;
        }
    };
    for (int c = 0; c < total; c += 2) {
        step(wb[0], c);
        if (c + 1 < total) step(wb[1], c + 1);
    }
}

__device__ inline void attention_phase(const MegaParams &p, int layer, AttnLds<8> &lds) {
    const MegaLayer &ly = p.layers[layer];
    AttnParams ap = {};
    ap.kv = ly.kv;
    ap.q = p.q;
    ap.qStride = p.qH * 128;
    ap.out = p.att;
    ap.oStride = p.qH * 128;
    ap.out_dtype = XFTHIP_BF16;
    ap.B = p.M;
    ap.S = 1;
    ap.G = p.qH / p.kvH;
    ap.scale = p.scale;
    ap.past = 0;
    ap.past_dev = p.pos;
    ap.nsplit = p.nsplit;
    ap.CG = 1;
    ap.ws = p.ws;
    ap.tickets = p.tickets;
    const int units = p.M * p.kvH * p.nsplit;
    for (int it = blockIdx.x; it < units; it += gridDim.x) {
        const int split = it % p.nsplit, kvh = (it / p.nsplit) % p.kvH, b = it / (p.nsplit * p.kvH);
        attn_unit<false, 8, false>(ap, split, kvh, 0, b, lds, [] { __syncthreads(); });
        __syncthreads();
    }
}

__global__ void mega_reset_kernel(unsigned int *sync) {
    for (int i = threadIdx.x; i < 640; i += blockDim.x)
        if (i != 16) sync[i] = 0u; // [16] is the abort flag, which the host owns
}

__global__ __launch_bounds__(512) void decode_mega_kernel(MegaParams p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char mega_smem[];
    MegaLds L;
    L.part = (XFT_LDS float *)mega_smem;
    L.flag = (XFT_LDS int *)(mega_smem + 128);
    L.act = (XFT_LDS uint16_t *)(mega_smem + kLdsHeader);
    L.red = (XFT_LDS float *)(mega_smem + kLdsHeader + p.red_off);
    AttnLds<8> &attn_lds = *reinterpret_cast<AttnLds<8> *>(mega_smem + kLdsHeader);
    const int G = gridDim.x, wg = blockIdx.x;
    const int H = p.hidden, M = p.M;
    unsigned int phase = 0;
    if (p.trace && wg == 0 && threadIdx.x == 0) p.trace[0] = wall_clock64();

    mu32x4 wb[2][8];

    // ---- record the input ids, embed them; the first weights go out inside the barrier ----
    PhaseDesc d = setup_phase(p, 0);
    if (wg == 0 && threadIdx.x < M) p.idlog[(size_t)p.step[0] * M + threadIdx.x] = p.ids[threadIdx.x];
    for (int i = wg * 512 + threadIdx.x; i < M * H; i += G * 512) {
        const int m = i / H, c = i % H;
        int id = p.ids[m];
        id = id < 0 ? 0 : (id >= p.vocab ? p.vocab - 1 : id);
        st_dev(&p.x[i], fp16_bits_to_f32(p.embedding[(size_t)id * H + c]));
    }
    if (!grid_barrier(p, phase, L, &d, wb)) return;

    // ---- the GEMV phases: 4 per layer (qkv [+ attention], out-projection, gate/up, down), then lm_head ----
    const int nsteps = 4 * p.nlayers + 1;
    for (int step = 0; step < nsteps; ++step) {
        if (d.kind == PH_O || d.kind == PH_DOWN) {
            stage_copy(p, d, d.kind == PH_O ? p.att : p.h, L, wb);
        } else {
            const float *weight = d.kind == PH_HEAD ? p.final_norm : (d.kind == PH_QKV ? p.layers[d.layer].ln1 : p.layers[d.layer].ln2);
            // epsilon 1e-6 is hard-coded on the MLP side of the reference (src/layers/mlp_llama.h:212)
            stage_norm(p, d, weight, d.kind == PH_GU ? 1e-6f : p.rms_eps, L, wb);
        }
        if (d.kind == PH_HEAD)
            run_phase<true>(p, d, wb, L);
        else
            run_phase<false>(p, d, wb, L);
        if (d.kind == PH_QKV) {
            if (!grid_barrier(p, phase, L, nullptr, wb)) return;
            attention_phase(p, d.layer, attn_lds);
        }
        if (step + 1 < nsteps) {
            d = setup_phase(p, step + 1);
            if (!grid_barrier(p, phase, L, &d, wb)) return;
        }
    }
    if (!grid_barrier(p, phase, L, nullptr, wb)) return;

    // ================= greedy argmax (first maximum wins), position advance =================
    if (wg < M) {
        XFT_LDS float *sv = L.red;
        XFT_LDS int *si = (XFT_LDS int *)(L.red + 512);
        const float *row = p.logits + (size_t)wg * p.vocab;
        float bv = -INFINITY;
        int bi = 0x7FFFFFFF;
        for (int j = threadIdx.x; j < p.vocab; j += 512) {
            const float v = ld_dev(&row[j]);
            if (v > bv || bi == 0x7FFFFFFF) {
                bv = v;
                bi = j;
            }
        }
        sv[threadIdx.x] = bv;
        si[threadIdx.x] = bi;
        __syncthreads();
        for (int s = 256; s > 0; s >>= 1) {
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
            p.ids[wg] = si[0];
            p.pos[wg] += 1;
            if (wg == 0) p.step[0] += 1;
        }
    }
}

} // namespace xfthip

using namespace xfthip;

namespace xfthip {

int mega_decode_max_blocks(int *blocks_per_cu, size_t lds_bytes) {
    int n = 0;
    XFT_CHECK_HIP(hipFuncSetAttribute((const void *)decode_mega_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
    XFT_CHECK_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, decode_mega_kernel, 512, lds_bytes));
    *blocks_per_cu = n;
    return 0;
}

int mega_decode_launch(const MegaParams &p, int grid, size_t lds_bytes, hipStream_t stream) {
    hipLaunchKernelGGL(mega_reset_kernel, dim3(1), dim3(64), 0, stream, p.counter);
    hipLaunchKernelGGL(decode_mega_kernel, dim3(grid), dim3(512), lds_bytes, stream, p);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

} // namespace xfthip
