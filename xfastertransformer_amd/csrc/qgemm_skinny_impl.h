// Kernel template of the dequant-fused weight-only GEMM for few activation rows (M <= 32), the
// decode-time shape.  Included by one translation unit per weight kind (qgemm_skinny_*.hip) so
// that the instantiations compile in parallel.
// Replaces MMHelper::compute* (reference src/utils/matmul_helper.h:565-1705) for
// INT8 / UINT4 / NF4 / BF16 weights against bf16 activations.
//
// HBM-bound: every weight byte is read exactly once with 128-bit loads.  One wavefront
// owns NT column tiles (16 output columns each) and a slice of K; the weight tile is the
// MFMA "A" operand (rows = output columns), the activation rows are the "B" operand
// (columns = tokens, padded to 16), so D[n][m] accumulates in 4 VGPRs per tile.  The
// integer codes are widened to bf16 in registers (exact: |code| < 256 fits 8 significant
// bits), per-column scale / zero-point are applied once in the epilogue.  The K slices of
// one column block are summed through LDS in a fixed order (deterministic).
#pragma once
#include "qgemm.h"

namespace xfthip {
namespace {


// LDS of the RMSNorm prologue: M rows of K + 8 bf16 values
static inline size_t skinny_norm_lds_bytes(int M, int K) {
    return (size_t)M * (K + 8) * 2;
}

template <int KIND>
struct KindTraits;
template <>
struct KindTraits<XFTHIP_W_INT8> {
    static constexpr int MPT = 2, KL = 16, KTILE = 64;
};
template <>
struct KindTraits<XFTHIP_W_UINT4> {
    static constexpr int MPT = 4, KL = 32, KTILE = 128;
};
template <>
struct KindTraits<XFTHIP_W_NF4> {
    static constexpr int MPT = 4, KL = 32, KTILE = 128;
};
template <>
struct KindTraits<XFTHIP_W_BF16> {
    static constexpr int MPT = 1, KL = 8, KTILE = 32;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

union Frag {
    bf16x8 v;
    uint32_t u[4];
    u32x4 q;
};

// two fp32 -> packed bf16 pair by truncation (exact for small integers)
__device__ inline uint32_t pack_hi16(float lo, float hi) {
    return __builtin_amdgcn_perm(f2u(hi), f2u(lo), 0x07060302u);
}

// Widen the codes of MFMA step `i` of a lane's 16-byte chunk to 8 bf16 values.
template <int KIND>
__device__ inline bf16x8 widen(const u32x4 &w, int i, const uint32_t *lut) {
    Frag f;
    Frag src;
    src.q = w;
    const uint32_t *wd = src.u;
    if constexpr (KIND == XFTHIP_W_INT8) {
        uint32_t a = wd[2 * i], b = wd[2 * i + 1];
        f.u[0] = pack_hi16((float)(int)(int8_t)(a), (float)(int)(int8_t)(a >> 8));
        f.u[1] = pack_hi16((float)(int)(int8_t)(a >> 16), (float)((int)a >> 24));
        f.u[2] = pack_hi16((float)(int)(int8_t)(b), (float)(int)(int8_t)(b >> 8));
        f.u[3] = pack_hi16((float)(int)(int8_t)(b >> 16), (float)((int)b >> 24));
    } else if constexpr (KIND == XFTHIP_W_UINT4) {
        // 0x4300 | u is the bf16 value 128 + u; the 128 is removed in the epilogue
        uint32_t a = wd[i];
        f.u[0] = (a & 0x000F000Fu) | 0x43004300u;
        f.u[1] = ((a >> 4) & 0x000F000Fu) | 0x43004300u;
        f.u[2] = ((a >> 8) & 0x000F000Fu) | 0x43004300u;
        f.u[3] = ((a >> 12) & 0x000F000Fu) | 0x43004300u;
    } else if constexpr (KIND == XFTHIP_W_NF4) {
        (void)lut; // NF4 goes through widen_nf4
    } else {
        f.q = w;
    }
    return f.v;
}

// NF4: a code value is not a bf16 number, so it is split into hi + lo bf16 parts (16
// significant bits, relative error 2^-17) and multiplied with two MFMAs.  The table maps a
// byte (two codes) to {hi pair, lo pair}.
__device__ inline void widen_nf4(const u32x4 &w, int i, const uint2 *lut, bf16x8 &hi, bf16x8 &lo) {
    Frag src, h, l;
    src.q = w;
    const uint32_t a = src.u[i];
    const uint2 e0 = lut[a & 0xFF], e1 = lut[(a >> 8) & 0xFF], e2 = lut[(a >> 16) & 0xFF], e3 = lut[a >> 24];
    h.u[0] = e0.x; h.u[1] = e1.x; h.u[2] = e2.x; h.u[3] = e3.x;
    l.u[0] = e0.y; l.u[1] = e1.y; l.u[2] = e2.y; l.u[3] = e3.y;
    hi = h.v;
    lo = l.v;
}

__device__ inline float silu_f(float x) {
    return x / (1.0f + fast_exp(-x));
}

// NF4 code values (QLoRA appendix E), split into bf16 hi + lo parts for the MFMA
__constant__ float c_nf4_gemm[16] = XFTHIP_NF4_CODE_VALUES;

// KIND: weight kind; NT: column tiles per wave; MT: 16-row activation tiles (1 or 2);
// U: k tiles per load batch (the packed K extent is padded to whole batches);
// NEED_SUM: also accumulate the row sums of A (zero-point term); KTAIL: K is not a whole
// number of tiles, activation loads past K are masked.  NORM: activations come from the fused
// RMSNorm prologue in LDS (M <= 4, MT == 1, no K tail).  blockDim.x = 64 * (K slices).
// ROPE: the RoPE + cache-append epilogue of the QKV projection with its paired column tiles
// (a template flag, so that the plain kernels keep their affine tile addressing).
// 8 waves (K slices) a workgroup; 16 for the one-tile blocks at 17 .. 32 rows, whose time is the chain of load
// round trips over a wave's K slice
// STAGE: activation rows are loaded as whole 128-byte runs (8 or 16 adjacent lanes along a row) and turned into
// MFMA fragments through a wave-private LDS patch.  Loaded straight in fragment order a wave-load is 16 rows x
// four 16-byte pieces, which the memory pipeline serves at a third of the rate of contiguous runs (37 against
// 125 GB/s a CU from L2, measured): with more than a few rows those loads, not the weights, set the time.
// GROUP: several weights of one shape behind one launch (SkinnyParams::group, one grid row a weight); a form of its
// own: with the weight pointers possibly read from memory the plain kernels lost 6 % of the decode step.
template <int KIND, int NT, int MT, int U, bool NEED_SUM, bool KTAIL, bool NORM, bool ROPE, bool STAGE = false, bool GROUP = false>
__global__ __launch_bounds__(512, (STAGE && MT == 1 && NT == 1) ? 4 : 1) void qgemm_skinny_kernel(SkinnyParams p) {
    // (the one-tile staged form is held to 128 registers, two workgroups a CU like its unstaged twin)
    static_assert(!NORM || (MT == 1 && !KTAIL), "the norm prologue covers M <= 4 without a K tail");
    static_assert(!ROPE || (NT % 2 == 0 && !KTAIL), "the RoPE epilogue works on tile pairs");
    static_assert(!STAGE || (!NORM && !ROPE), "staged activation loads belong to the plain kernels");
    static_assert(!GROUP || (!NORM && !ROPE && !KTAIL), "grouped launches: plain kernels, whole k tiles");
    using T = KindTraits<KIND>;
    constexpr int MPT = T::MPT, KL = T::KL, KTILE = T::KTILE;
    extern __shared__ float smem[];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    const int g = lane >> 4, ml = lane & 15;
    constexpr bool need_sum = NEED_SUM;
    if (p.rows_dev) {
        // row count (and, for a group of weights of one shape, the weight: blockIdx.y) from device memory
        const int *rec = p.rows_dev;
        if constexpr (GROUP) {
            rec += blockIdx.y * p.rows_stride;
            p.packed = p.group[blockIdx.y].packed;
            p.scale = p.group[blockIdx.y].scale;
            p.zero = p.group[blockIdx.y].zero;
        }
        if (rec[0] <= 0) return; // uniform: the whole workgroup leaves
        p.M = rec[0] < p.M ? rec[0] : p.M;
        p.A += (size_t)rec[1] * p.lda;
        p.C = (char *)p.C + (size_t)rec[2] * p.ldc * (p.c_dtype == XFTHIP_F32 ? 4 : 2);
    }

    uint2 *lut = nullptr;
    if constexpr (KIND == XFTHIP_W_NF4) {
        // 256-entry table: byte -> {bf16 hi parts of (low, high) nibble, bf16 lo parts}
        lut = (uint2 *)smem;
        for (int i = threadIdx.x; i < 256; i += blockDim.x) {
            const float c0 = c_nf4_gemm[i & 15], c1 = c_nf4_gemm[i >> 4];
            const uint32_t h0 = f32_to_bf16_ref(c0), h1 = f32_to_bf16_ref(c1);
            const uint32_t l0 = f32_to_bf16_ref(c0 - bf16_to_f32((uint16_t)h0));
            const uint32_t l1 = f32_to_bf16_ref(c1 - bf16_to_f32((uint16_t)h1));
            lut[i] = make_uint2(h0 | (h1 << 16), l0 | (l1 << 16));
        }
        __syncthreads();
    }
    float *red = smem + (KIND == XFTHIP_W_NF4 ? 512 : 0);
    // STAGE: this wave's patch, [U][16 MT rows][KTILE bf16 + 16 bytes] (the pad keeps the fragment reads off each
    // other's banks); it shares its LDS with the reduction area, which is used only after the K loop
    constexpr int LPR = KTILE / 8, RPI = 64 / LPR; // lanes along a row, rows a wave-load
    constexpr int SPITCH = KTILE * 2 + 16, STILE = 16 * MT * SPITCH;
    unsigned char *stage = (unsigned char *)red + (size_t)wave * (U * STILE);
    const int s_row = lane / LPR, s_kc = lane % LPR;

    // K slice of this wave: balanced split of the KT / U load batches
    const int nbatch = p.KT / U;
    const int base = nbatch / nwaves, rem = nbatch % nwaves;
    const int b_begin = wave * base + (wave < rem ? wave : rem);
    const int nb = base + (wave < rem ? 1 : 0);
    // With the norm prologue the grid is one workgroup per compute unit and each walks over
    // several column blocks, so that the prologue is paid once per workgroup rather than once per
    // column block; the plain kernel is launched with one workgroup per column block.
    bool first = true;
    uint16_t *xn = nullptr; // NORM: [M][K + 8] bf16 behind the reduction area
    int xn_row = 0;
    // column tile t of column block `it`; the RoPE epilogue pairs dims (d, d + 64) of a head, then V tiles
    const int rope_pairs = ROPE ? (p.qH + p.kvH) * 4 : 0;
    // (a block holds NT / 2 such pairs; the pair count of the rotated heads is even, so no block straddles the
    // border between rotated and value tiles when NT = 4)
    auto tile_index = [&](int it, int t) {
        if constexpr (ROPE) {
            const int pi = it * (NT / 2) + (t >> 1), tt = t & 1;
            return pi < rope_pairs ? (pi >> 2) * 8 + (pi & 3) + 4 * tt : (p.qH + p.kvH) * 8 + 2 * (pi - rope_pairs) + tt;
        }
        return it * NT + t;
    };
    // Every weight load is unconditional: out-of-range column tiles are clamped to the last valid
    // one (their results are never stored).
    const uint8_t *wbase[NT];
    auto set_wbase = [&](int it) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            int nt = tile_index(it, t);
            nt = nt < p.NTILES ? nt : p.NTILES - 1;
            wbase[t] = p.packed + (size_t)nt * p.KT * 1024 + lane * 16;
        }
    };
    u32x4 wbuf[2][U][NT];
    bool pre_issued = false; // NORM: the first batch of this block went out before the previous block's epilogue
    auto run_block = [&](const int blk) {
        const int nt0 = blk * NT;
        auto tile_of = [&](int t) { return tile_index(blk, t); };

        f32x4 acc[NT][MT];
        f32x4 accS[MT];
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int m = 0; m < MT; ++m) acc[t][m] = f32x4 {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int m = 0; m < MT; ++m) accS[m] = f32x4 {0.f, 0.f, 0.f, 0.f};

        Frag ones;
        ones.u[0] = ones.u[1] = ones.u[2] = ones.u[3] = 0x3F803F80u;

        // Activation loads are unconditional too (rows clamped to the last valid one), so the loop
        // body is straight-line code and the loads of the next batch stay in flight during the MFMAs.
        if (!pre_issued) set_wbase(blk);
        const uint16_t *abase[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            int row = m * 16 + ml;
            row = row < p.M ? row : p.M - 1;
            abase[m] = p.A + (size_t)row * p.lda + g * KL;
        }

        // STAGE: element offset of wave-load j of a k tile (row j * RPI + s_row, clamped) without the k part
        uint32_t s_off[MT * MPT];
#pragma unroll
        for (int j = 0; j < MT * MPT; ++j) {
            int row = j * RPI + s_row;
            row = row < p.M ? row : p.M - 1;
            s_off[j] = (uint32_t)row * (uint32_t)p.lda;
        }

        const u32x4 zero4 = {0u, 0u, 0u, 0u};
        u32x4 abuf[2][U][MT][MPT];

        auto issue = [&](int buf, int batch) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int kt = batch * U + u;
#pragma unroll
                for (int t = 0; t < NT; ++t)
                    wbuf[buf][u][t] = __builtin_nontemporal_load((const u32x4 *)(wbase[t] + (size_t)kt * 1024));
                if constexpr (NORM) continue; // activations are read from LDS in compute()
                if constexpr (STAGE) {
#pragma unroll
                    for (int j = 0; j < MT * MPT; ++j) {
                        const int koff = kt * KTILE + s_kc * 8;
                        if constexpr (KTAIL) {
                            const bool v = koff + 8 <= p.K;
                            const u32x4 a = *(const u32x4 *)(p.A + s_off[j] + (v ? koff : 0));
                            abuf[buf][u][j / MPT][j % MPT] = v ? a : zero4;
                        } else {
                            abuf[buf][u][j / MPT][j % MPT] = *(const u32x4 *)(p.A + s_off[j] + koff);
                        }
                    }
                    continue;
                }
#pragma unroll
                for (int m = 0; m < MT; ++m) {
#pragma unroll
                    for (int i = 0; i < MPT; ++i) {
                        int koff = kt * KTILE + 8 * i;
                        if constexpr (KTAIL) {
                            // chunk is inside the row iff koff + 8 <= K - g*KL; otherwise read the row
                            // start (always valid) and discard it
                            const bool v = koff + 8 <= p.K - g * KL;
                            const u32x4 a = *(const u32x4 *)(abase[m] + (v ? koff : -g * KL));
                            abuf[buf][u][m][i] = v ? a : zero4;
                        } else {
                            abuf[buf][u][m][i] = *(const u32x4 *)(abase[m] + koff);
                        }
                    }
                }
            }
        };
        auto compute = [&](int buf, int batch) {
            (void)batch;
            if constexpr (STAGE) {
                // rows as loaded into the patch; the fragments are read back below (same wave, in order)
#pragma unroll
                for (int u = 0; u < U; ++u)
#pragma unroll
                    for (int j = 0; j < MT * MPT; ++j)
                        *(u32x4 *)(stage + u * STILE + (j * RPI + s_row) * SPITCH + s_kc * 16) = abuf[buf][u][j / MPT][j % MPT];
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
                for (int i = 0; i < MPT; ++i) {
                    Frag a[MT];
#pragma unroll
                    for (int m = 0; m < MT; ++m) {
                        if constexpr (NORM)
                            a[m].q = *(const u32x4 *)(xn + xn_row + (batch * U + u) * KTILE + g * KL + 8 * i);
                        else if constexpr (STAGE)
                            a[m].q = *(const u32x4 *)(stage + u * STILE + (m * 16 + ml) * SPITCH + (g * KL + 8 * i) * 2);
                        else
                            a[m].q = abuf[buf][u][m][i];
                    }
#pragma unroll
                    for (int t = 0; t < NT; ++t) {
                        if constexpr (KIND == XFTHIP_W_NF4) {
                            bf16x8 whi, wlo;
                            widen_nf4(wbuf[buf][u][t], i, lut, whi, wlo);
#pragma unroll
                            for (int m = 0; m < MT; ++m) {
                                acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wlo, a[m].v, acc[t][m], 0, 0, 0);
                                acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(whi, a[m].v, acc[t][m], 0, 0, 0);
                            }
                        } else {
                            bf16x8 wv = widen<KIND>(wbuf[buf][u][t], i, nullptr);
#pragma unroll
                            for (int m = 0; m < MT; ++m)
                                acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv, a[m].v, acc[t][m], 0, 0, 0);
                        }
                    }
                    if constexpr (need_sum) {
#pragma unroll
                        for (int m = 0; m < MT; ++m)
                            accS[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones.v, a[m].v, accS[m], 0, 0, 0);
                    }
                }
            }
        };

        // sched_barrier keeps the compiler from sinking the next batch's loads below the MFMAs of
        // the current one: all loads of a batch are issued back to back, then the math runs.
#define XFT_FENCE() __builtin_amdgcn_sched_barrier(0)
        // ROPE: the position of the first row (the only one of a single sequence) is requested ahead of the weights,
        // into a scalar register, so that the epilogue's chain position -> cos / sin -> store is one round trip
        // shorter (the cos / sin values themselves stay in the epilogue: requested here, the wait for their address
        // would hold up the weight stream)
        int pos_pre = 0;
        if constexpr (ROPE) pos_pre = __builtin_amdgcn_readfirstlane(p.pos_dev ? p.pos_dev[0] : p.pos_host);
        if (nb > 0 && !pre_issued) {
            issue(0, b_begin);
            XFT_FENCE();
        }
        // Per-column scale / zero point of the epilogue, fetched now (behind the first weight
        // batch) instead of after the reduction, where their latency would be exposed.
        float e_scale[NT], e_zero[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            e_scale[t] = 0.0f, e_zero[t] = 0.0f;
            if constexpr (KIND != XFTHIP_W_BF16) {
                int nt = tile_of(t);
                nt = nt < p.NTILES ? nt : p.NTILES - 1;
                e_scale[t] = p.scale[nt * 16 + (lane & 15)];
                if ((KIND == XFTHIP_W_UINT4 || need_sum) && p.zero) e_zero[t] = p.zero[nt * 16 + (lane & 15)];
            }
        }
        if (NORM && first) {
            // RMSNorm of the M rows into LDS while the first weight tiles are on their way; same
            // arithmetic as rmsnorm_vec_kernel: y = bf16((x * rstd) * w)
            float *part = red + (size_t)nwaves * (16 * MT * (16 * NT + 1) + 16 * MT);
            xn = (uint16_t *)(part + 16);
            const int pitch = p.K + 8;
            xn_row = (ml < p.M ? ml : p.M - 1) * pitch;
            // The norm weights are first needed behind the first row's reduction, where a miss to memory would be
            // fully exposed: one value of each of their 128-byte lines is requested now, with the first row (4-bit
            // kinds, whose short weight stream leaves the prologue in the open: UINT4 decode 561 -> 574 tok/s; the
            // INT8 kernels, at their 128 registers, lose 0.7 % to the extra one)
            constexpr bool TOUCH = KIND == XFTHIP_W_UINT4 || KIND == XFTHIP_W_NF4;
            constexpr int NB = TOUCH ? 4 : 2;
            float w_touch = 0.0f;
            if (TOUCH && (int)threadIdx.x * 32 < p.K) w_touch = p.norm_w[threadIdx.x * 32];
            for (int m = 0; m < p.M; ++m) {
                const float *row = p.norm_x + (size_t)m * p.ldx;
                float sq = 0.0f;
                // NB loads in flight a thread (the 4-wave workgroups of the 4-bit kinds walk a 4096-wide row in four
                // steps: one round trip instead of four); the sums keep the order of the plain loop
                for (int c = threadIdx.x * 4; c < p.K; c += blockDim.x * 4 * NB) {
                    float4 v[NB];
#pragma unroll
                    for (int i = 0; i < NB; ++i) {
                        const int ci = c + i * (int)blockDim.x * 4;
                        v[i] = ci < p.K ? *(const float4 *)(row + ci) : make_float4(0.f, 0.f, 0.f, 0.f);
                    }
#pragma unroll
                    for (int i = 0; i < NB; ++i) sq = fmaf(v[i].x, v[i].x, fmaf(v[i].y, v[i].y, fmaf(v[i].z, v[i].z, fmaf(v[i].w, v[i].w, sq))));
                }
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) sq += __shfl_xor(sq, off, 64);
                if (lane == 0) part[(m & 1) * 8 + wave] = sq;
                __syncthreads();
                if constexpr (TOUCH) asm volatile("" ::"v"(w_touch)); // keeps the request above alive; the value is not used
                float tot = 0.0f;
                for (int w = 0; w < nwaves; ++w) tot += part[(m & 1) * 8 + w];
                const float var = 1.0f / sqrtf(tot / (float)p.K + p.norm_eps);
                for (int c = threadIdx.x * 4; c < p.K; c += blockDim.x * 4 * NB) {
                    float4 vv[NB], ww[NB];
#pragma unroll
                    for (int i = 0; i < NB; ++i) {
                        const int ci = c + i * (int)blockDim.x * 4;
                        const int cl = ci < p.K ? ci : c; // past the row: a second read of this step's first chunk, not stored
                        vv[i] = *(const float4 *)(row + cl);
                        ww[i] = *(const float4 *)(p.norm_w + cl);
                    }
#pragma unroll
                    for (int i = 0; i < NB; ++i) {
                        const int ci = c + i * (int)blockDim.x * 4;
                        const float4 v = vv[i], w = ww[i];
                        const uint32_t lo = f32_to_bf16_ref((v.x * var) * w.x) | ((uint32_t)f32_to_bf16_ref((v.y * var) * w.y) << 16);
                        const uint32_t hi = f32_to_bf16_ref((v.z * var) * w.z) | ((uint32_t)f32_to_bf16_ref((v.w * var) * w.w) << 16);
                        if (ci < p.K) *(uint2 *)(xn + (size_t)m * pitch + ci) = make_uint2(lo, hi);
                    }
                }
            }
            __syncthreads();
        }
        if (nb > 0) {
            int b = 1; // next batch to issue; buffer 0 holds batch b - 1
            for (; b + 1 < nb; b += 2) {
                issue(1, b_begin + b);
                XFT_FENCE();
                compute(0, b_begin + b - 1);
                XFT_FENCE();
                issue(0, b_begin + b + 1);
                XFT_FENCE();
                compute(1, b_begin + b);
                XFT_FENCE();
            }
            if (b < nb) {
                issue(1, b_begin + b);
                XFT_FENCE();
                compute(0, b_begin + b - 1);
                XFT_FENCE();
                compute(1, b_begin + b);
            } else {
                compute(0, b_begin + b - 1);
            }
        }
        if constexpr (NORM) {
            // the next column block's first batch goes out before this block's reduction and epilogue
            const int nxt = blk + gridDim.x;
            pre_issued = nxt < p.nblocks;
            if (pre_issued) {
                set_wbase(nxt);
                if (nb > 0) issue(0, b_begin);
                XFT_FENCE();
            }
        }
#undef XFT_FENCE

        // ---- cross-wave reduction through LDS: red[wave][m][n] -------------------------------
        constexpr int ROWS = 16 * MT, COLS = 16 * NT, LD = COLS + 1;
        if constexpr (STAGE) __syncthreads(); // the reduction area lies over the other waves' activation patches
        float *mine = red + (size_t)wave * (ROWS * LD + ROWS);
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int m = 0; m < MT; ++m)
#pragma unroll
                for (int r = 0; r < 4; ++r) mine[(m * 16 + ml) * LD + t * 16 + 4 * g + r] = acc[t][m][r];
        if (g == 0) {
#pragma unroll
            for (int m = 0; m < MT; ++m) mine[ROWS * LD + m * 16 + ml] = accS[m][0];
        }
        __syncthreads();

        const int stride = ROWS * LD + ROWS;
        auto total = [&](int m, int c) {
            float s = 0.0f;
            for (int w = 0; w < nwaves; ++w) s += red[(size_t)w * stride + m * LD + c];
            return s;
        };
        auto total_sum = [&](int m) {
            float s = 0.0f;
            for (int w = 0; w < nwaves; ++w) s += red[(size_t)w * stride + ROWS * LD + m];
            return s;
        };
        // (c & 15 equals threadIdx.x & 15 for every caller, so the scales fetched at the start of
        // the block are the ones this thread needs)
        auto column_value = [&](int m, int c, float sumA) {
            float v = total(m, c);
            if constexpr (KIND == XFTHIP_W_BF16) return v;
            const float s = e_scale[c >> 4];
            if constexpr (KIND == XFTHIP_W_UINT4) {
                return fmaf(s, v - 128.0f * sumA, e_zero[c >> 4] * sumA);
            } else if constexpr (KIND == XFTHIP_W_INT8) {
                v = s * v;
                if constexpr (need_sum) v = fmaf(e_zero[c >> 4], sumA, v);
                return v;
            } else {
                return s * v;
            }
        };

        if constexpr (ROPE) {
            // one new token per sequence: row m is sequence m at position pos
#pragma unroll
            for (int sub = 0; sub < NT / 2; ++sub) {
            const int it = blk * (NT / 2) + sub, cofs = 32 * sub; // pair index, its first column in the block
            if (it < rope_pairs) {
                const int hh = it >> 2, jj = it & 3;
                for (int v = threadIdx.x; v < p.M * 16; v += blockDim.x) {
                    const int m = v >> 4, c = v & 15;
                    int pos = m == 0 ? pos_pre : (p.pos_dev ? p.pos_dev[m] : p.pos_host);
                    pos = pos < 0 ? 0 : (pos >= p.kv.S ? p.kv.S - 1 : pos); // held inside the cache whatever the device value is
                    const int i = jj * 16 + c;
                    // (requested before the sums over the waves' partial results are read, not behind them)
                    const float cs = p.cosT[(size_t)pos * 64 + i], sn = p.sinT[(size_t)pos * 64 + i];
                    const float sumA = need_sum ? total_sum(m) : 0.0f;
                    // the projection's output is bf16 in the reference (the rotation reads it back)
                    const float lo = bf16_to_f32(f32_to_bf16_ref(column_value(m, cofs + c, sumA)));
                    const float hi = bf16_to_f32(f32_to_bf16_ref(column_value(m, cofs + 16 + c, sumA)));
                    // reference: fmsub(q, cos, qHalf*sin) ; fmadd(qHalf, cos, q*sin)
                    const float nlo = fmaf(lo, cs, -(hi * sn)), nhi = fmaf(hi, cs, lo * sn);
                    if (hh < p.qH) {
                        uint16_t *dst = (uint16_t *)p.C + (size_t)m * p.ldc + hh * 128;
                        dst[i] = f32_to_bf16_ref(nlo);
                        dst[i + 64] = f32_to_bf16_ref(nhi);
                    } else if (pos < p.kv.S) {
                        const size_t bh = (size_t)m * p.kv.H + (hh - p.qH);
                        uint16_t *dst = (uint16_t *)p.kv.k + (bh * p.kv.S + pos) * 128;
                        dst[i] = f32_to_fp16_bits(nlo);
                        dst[i + 64] = f32_to_fp16_bits(nhi);
                    }
                }
            } else {
                for (int v = threadIdx.x; v < p.M * 32; v += blockDim.x) {
                    const int m = v >> 5, cc = v & 31;
                    const int vt = 2 * (it - rope_pairs) + (cc >> 4);
                    const float sumA = need_sum ? total_sum(m) : 0.0f;
                    const float val = bf16_to_f32(f32_to_bf16_ref(column_value(m, cofs + cc, sumA)));
                    int pos = m == 0 ? pos_pre : (p.pos_dev ? p.pos_dev[m] : p.pos_host);
                    pos = pos < 0 ? 0 : (pos >= p.kv.S ? p.kv.S - 1 : pos);
                    if (pos < p.kv.S) {
                        const size_t bh = (size_t)m * p.kv.H + (vt >> 3);
                        const int d = (vt & 7) * 16 + (cc & 15);
                        uint16_t *dst = (uint16_t *)p.kv.v + (bh * (p.kv.S / 32) + (pos >> 5)) * (size_t)128 * 32 + (size_t)d * 32 + v_slot(pos & 31);
                        *dst = f32_to_fp16_bits(val);
                    }
                }
            }
            }
        } else if (!p.gateup) {
            // up to two tiles: all lanes along the block's rows at once; more: tile by tile (a static index into
            // the per-tile scales), 16 lanes along a row
            constexpr int PASSES = NT <= 2 ? 1 : NT, PCOLS = NT <= 2 ? COLS : 16;
            auto finish = [&](int t, int v) {
                const int m = v / PCOLS, c = t * 16 + v % PCOLS;
                const int np = nt0 * 16 + c;
                if (m >= p.M || np >= p.N) return;
                // the residual value is requested before the sums over the waves' partial results are read
                float resv = 0.0f;
                if (p.epi == XFTHIP_EPI_RESMUL || p.epi == XFTHIP_EPI_RESIDENTIAL || p.epi == XFTHIP_EPI_RESEXT)
                    resv = load_as_f32(p.res, p.res_dtype, (size_t)m * p.ldres + np);
                const float sumA = need_sum ? total_sum(m) : 0.0f;
                float x = column_value(m, c, sumA);
                switch (p.epi) {
                    case XFTHIP_EPI_BIAS: x += p.bias[np]; break;
                    case XFTHIP_EPI_SILU: x = silu_f(x); break;
                    case XFTHIP_EPI_GELU: {
                        float e = fast_exp(1.702f * x);
                        x = e / (e + 1.0f) * x;
                        break;
                    }
                    case XFTHIP_EPI_RESMUL: x *= resv; break;
                    case XFTHIP_EPI_RESIDENTIAL:
                        if (p.bias) x += p.bias[np];
                        x += resv;
                        break;
                    case XFTHIP_EPI_RESEXT:
                        if (p.bias) x += p.bias[np];
                        x = fmaf(p.gamma, resv, x);
                        break;
                    default: break;
                }
                store_from_f32(p.C, p.c_dtype, (size_t)m * p.ldc + np, x);
            };
            if constexpr (PASSES == 1) {
                for (int v = threadIdx.x; v < ROWS * COLS; v += blockDim.x) finish(0, v);
            } else {
#pragma unroll
                for (int t = 0; t < PASSES; ++t) {
#pragma unroll 1
                    for (int v = threadIdx.x; v < ROWS * 16; v += blockDim.x) finish(t, v);
                }
            }
        } else if constexpr (NT >= 2) {
            // tile pairs (2j, 2j+1) hold gate / up columns [16 j', 16 j' + 16)
            constexpr int PAIRS = NT / 2;
#pragma unroll
            for (int pr = 0; pr < PAIRS; ++pr)
#pragma unroll 1
            for (int v = threadIdx.x; v < ROWS * 16; v += blockDim.x) {
                const int m = v >> 4, c = v & 15;
                const int out_col = (blk * PAIRS + pr) * 16 + c;
                if (m >= p.M || out_col >= p.N / 2) continue;
                const float sumA = need_sum ? total_sum(m) : 0.0f;
                const float gate = column_value(m, pr * 32 + c, sumA);
                const float up = column_value(m, pr * 32 + 16 + c, sumA);
                store_from_f32(p.C, p.c_dtype, (size_t)m * p.ldc + out_col, up * silu_f(gate));
            }
        }
        if constexpr (NORM) {
            first = false;
            __syncthreads(); // the next column block reuses the reduction area
        }
    };
    if constexpr (NORM) {
        for (int blk = blockIdx.x; blk < p.nblocks; blk += gridDim.x) run_block(blk);
    } else {
        run_block(blockIdx.x);
    }
}

// k tiles per load batch, sized so that two batches of weight + activation fragments stay in
// registers (256 VGPRs per lane at 8 waves per block)
template <int KIND, int MT, int NT = 1>
constexpr int batch_tiles() {
    if (MT == 2 && NT >= 4) return 1; // wide column blocks: the weight registers of one k tile are a batch already
    if (KIND == XFTHIP_W_INT8) return MT == 1 ? 4 : 2;
    if (KIND == XFTHIP_W_BF16) return MT == 1 ? 4 : 2;
    return MT == 1 ? 2 : 1;
}

template <int KIND, int NT, int MT, int U, bool NEED_SUM, bool KTAIL, bool NORM, bool ROPE = false, bool STAGE = false, bool GROUP = false>
static int launch(const SkinnyParams &p, int kslices, hipStream_t stream) {
    constexpr int ROWS = 16 * MT, COLS = 16 * NT;
    size_t smem = (size_t)kslices * (ROWS * (COLS + 1) + ROWS) * sizeof(float);
    if (STAGE) {
        const size_t patches = (size_t)kslices * U * ROWS * (KindTraits<KIND>::KTILE * 2 + 16);
        smem = smem > patches ? smem : patches;
    }
    smem += (KIND == XFTHIP_W_NF4 ? 2048 : 0);
    if (NORM) smem += 64 + skinny_norm_lds_bytes(p.M, p.K);
    int blocks = (p.NTILES + NT - 1) / NT;
    if (ROPE) blocks = (p.qH + 2 * p.kvH) * 4 / (NT / 2); // rotation pairs of the query and key heads, then value tile pairs
    SkinnyParams q = p;
    q.nblocks = blocks;
    if (NORM) {
        // one workgroup of 8 waves per CU, or two of 4
        // At most two workgroups (of 8 waves) per CU, all resident at once; beyond that a workgroup
        // walks over several column blocks.  Measured on 256 CUs: the 384 blocks of a 7B-shape QKV
        // projection as 384 workgroups 13.6 us against 14.9 as 256 workgroups looping; the 688 blocks
        // of gate/up as 512 workgroups 20.0 us against 21.3 as 256 and 24.7 as 688 (every workgroup
        // pays the prologue).
        // (workgroups of at most 4 waves, the 4-bit kinds at K = 4096: four a CU, UINT4 decode 550 -> 567 tok/s)
        const int cus = device_cu_count() * (kslices <= 4 ? 4 : 2);
        blocks = blocks < cus ? blocks : cus;
    }
    if (smem > 64 * 1024) {
        // more dynamic LDS than the default limit (wide column blocks at 17 .. 32 rows): raise it once per instantiation
        static const hipError_t attr = hipFuncSetAttribute((const void *)qgemm_skinny_kernel<KIND, NT, MT, U, NEED_SUM, KTAIL, NORM, ROPE, STAGE, GROUP>,
                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        XFT_CHECK_HIP(attr);
    }
    hipLaunchKernelGGL((qgemm_skinny_kernel<KIND, NT, MT, U, NEED_SUM, KTAIL, NORM, ROPE, STAGE, GROUP>), dim3(blocks, GROUP ? p.group_n : 1),
            dim3(64 * kslices), smem, stream, q);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

template <int KIND, int NT, int MT, bool NEED_SUM>
static int dispatch_tail(const SkinnyParams &p, int kslices, hipStream_t stream) {
    constexpr int U = batch_tiles<KIND, MT, NT>();
    if (p.KT * KindTraits<KIND>::KTILE != p.K) {
        if (p.norm_x || p.rope) {
            set_error("qgemm_skinny: the fused prologue / epilogue needs K to be a whole number of weight tiles");
            return 2;
        }
        if (MT == 2 || p.M > 4) return launch<KIND, NT, MT, U, NEED_SUM, true, false, false, true>(p, kslices, stream);
        if constexpr (MT == 1) return launch<KIND, NT, MT, U, NEED_SUM, true, false>(p, kslices, stream);
    }
    if constexpr (MT == 1 && (KIND == XFTHIP_W_UINT4 || KIND == XFTHIP_W_NF4)) {
        // 4-bit codes with the norm prologue: no activation registers are needed, so a batch can
        // hold 4 tiles (512 k) like the INT8 kernel's, which doubles the bytes a wave has in flight
        if (p.norm_x && p.KT % 4 == 0) {
            int ks = (p.KT / 4 + 1) / 2;
            ks = ks < 1 ? 1 : (ks > 8 ? 8 : ks);
            if constexpr (NT == 2) {
                if (p.rope) return launch<KIND, NT, MT, 4, NEED_SUM, false, true, true>(p, ks, stream);
            }
            if (!p.rope) return launch<KIND, NT, MT, 4, NEED_SUM, false, true, false>(p, ks, stream);
        }
    }
    if constexpr (MT == 1 && NT == 2) {
        if (p.rope) {
            if (p.norm_x) return launch<KIND, NT, MT, U, NEED_SUM, false, true, true>(p, kslices, stream);
            return launch<KIND, NT, MT, U, NEED_SUM, false, false, true>(p, kslices, stream);
        }
    }
    if constexpr (MT == 2 && NT == 4) {
        // 17 .. 32 rows: two pairs a block, one round over the CUs for a 7B QKV projection
        if (p.rope && !p.norm_x) return launch<KIND, NT, MT, U, NEED_SUM, false, false, true>(p, kslices, stream);
    }
    if (p.rope) {
        set_error("qgemm_skinny: no RoPE epilogue for this shape");
        return 2;
    }
    if constexpr (MT == 1) {
        if (p.norm_x) return launch<KIND, NT, MT, U, NEED_SUM, false, true>(p, kslices, stream);
    }
    // more than a few rows: activation rows loaded as contiguous runs (see STAGE)
    if (p.group) {
        if (MT == 2 || p.M > 4) return launch<KIND, NT, MT, U, NEED_SUM, false, false, false, true, true>(p, kslices, stream);
        if constexpr (MT == 1) return launch<KIND, NT, MT, U, NEED_SUM, false, false, false, false, true>(p, kslices, stream);
    }
    if (MT == 2 || p.M > 4) return launch<KIND, NT, MT, U, NEED_SUM, false, false, false, true>(p, kslices, stream);
    if constexpr (MT == 1) return launch<KIND, NT, MT, U, NEED_SUM, false, false>(p, kslices, stream);
    return 0;
}

template <int KIND, int NT, int MT>
static int dispatch_sum(const SkinnyParams &p, int kslices, hipStream_t stream) {
    if constexpr (KIND == XFTHIP_W_UINT4) {
        return dispatch_tail<KIND, NT, MT, true>(p, kslices, stream);
    } else if constexpr (KIND == XFTHIP_W_INT8) {
        if (p.zero) return dispatch_tail<KIND, NT, MT, true>(p, kslices, stream);
        return dispatch_tail<KIND, NT, MT, false>(p, kslices, stream);
    } else {
        return dispatch_tail<KIND, NT, MT, false>(p, kslices, stream);
    }
}

template <int KIND>
static int dispatch_shape(const SkinnyParams &p, hipStream_t stream) {
    const int cus = device_cu_count();
    const int mt = (p.M + 15) / 16;
    // column tiles per wave: 2 when that still leaves at least 2 blocks per CU (gate/up needs pairs); with two
    // activation tiles (17 .. 32 rows) already at one block per CU: a wave then loads four activation chunks per
    // two weight chunks instead of per one, and those loads are what the kernel waits for (32 x 4096 x 12288:
    // 27.5 -> 23.0 us)
    const bool wide = p.gateup || p.rope || (p.NTILES / 2 >= (mt == 1 ? 2 : 1) * cus);
    // K slices per block: aim at two load batches per wave, at most 8 waves
    const int u = (mt == 1) ? batch_tiles<KIND, 1>() : batch_tiles<KIND, 2>();
    const int nbatch = p.KT / u;
    int kslices = (nbatch + 1) / 2;
    if (kslices < 1) kslices = 1;
    if (kslices > 8) kslices = 8;
    if (mt == 1) {
        if (wide) return dispatch_sum<KIND, 2, 1>(p, kslices, stream);
        return dispatch_sum<KIND, 1, 1>(p, kslices, stream);
    }
    // 17 .. 32 rows: the kernel holds one workgroup a CU and a column block costs about the same time whether it
    // is 16 or 96 columns wide (a chain of load round trips over the wave's K slice), so the blocks are made wide
    // enough for one round over the CUs where the registers allow it: 3 tiles for the 768 of a 7B QKV projection
    // (384 two-tile blocks took two rounds: 23.2 us), 6 for the 1376 of its gate/up
    const int per_cu = (p.NTILES + cus - 1) / cus;
    if (p.rope) return dispatch_sum<KIND, 4, 2>(p, kslices, stream);
    if (p.gateup) {
        if (per_cu > 4) return dispatch_sum<KIND, 6, 2>(p, kslices, stream);
        if (per_cu > 2) return dispatch_sum<KIND, 4, 2>(p, kslices, stream);
        return dispatch_sum<KIND, 2, 2>(p, kslices, stream);
    }
    if (per_cu > 3) return dispatch_sum<KIND, 4, 2>(p, kslices, stream);
    if (per_cu > 2) return dispatch_sum<KIND, 3, 2>(p, kslices, stream);
    if (wide) return dispatch_sum<KIND, 2, 2>(p, kslices, stream);
    return dispatch_sum<KIND, 1, 2>(p, kslices, stream);
}

} // namespace
} // namespace xfthip
