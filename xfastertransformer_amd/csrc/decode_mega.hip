// Persistent whole-step decode kernel: one launch runs embedding, all decoder layers, the final
// norm, lm_head and greedy argmax for a batch of up to 4 sequences (INT8 weight-only layers,
// FP16 KV cache, head size 128).  The same arithmetic as the per-kernel path (qgemm_skinny,
// rmsnorm, rope_kv, attention) with the launches replaced by device-wide barriers, because at
// batch 1 a layer's ten kernels cost more in launch gaps (about 2.6 us each) than in HBM time.
//
// Grid: one 512-thread workgroup per compute unit, all co-resident.  A layer is five phases:
//   P1  RMSNorm (every workgroup normalises the M rows into its LDS) + QKV GEMV; the epilogue
//       applies RoPE (column tiles are processed in (d, d+64) pairs) and appends K / V to the cache
//   P2  split-KV attention (attn_unit), partials merged by the last-arriving workgroup
//   P3  out-projection GEMV + residual
//   P4  RMSNorm + gate/up GEMV + SwiGLU
//   P5  down GEMV + residual
// Work items of a phase are dealt round-robin to the workgroups.  The barrier is an atomic
// counter (zeroed by a tiny kernel before each launch) with a bounded spin: when the bound is hit
// the abort flag is raised and every workgroup leaves at its next barrier, so the grid always
// drains.  Activations, new cache rows, attention partials and logits cross between workgroups
// through device-coherent accesses (ld_dev / st_dev), so no barrier flushes or invalidates an L2;
// weights are read-only and streamed with non-temporal loads.
#include "attention_dev.h"
#include "decode_mega.h"

namespace xfthip {

typedef uint32_t mu32x4 __attribute__((ext_vector_type(4)));
// Pointers read out of the per-layer table are generic to the compiler; everything they point at
// is device memory, and saying so keeps the loads on the global path (vmcnt only).
#define XFT_GLOBAL __attribute__((address_space(1)))
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

struct MegaLds {
    union {
        AttnLds<8> attn;
        struct {
            uint16_t xn[4][4096 + 8]; // normalised rows (bf16), padded pitch
            float red[8][16 * 33 + 16]; // K-slice partial sums: [wave][m][col]
        } g;
    };
    float part[8];
    int flag;
};

// ---- device-wide barrier -----------------------------------------------------------------
__device__ inline bool grid_barrier(const MegaParams &p, unsigned int &phase, MegaLds &L) {
    // Everything one workgroup hands to another inside the launch is written with st_dev and
    // read with ld_dev, so the barrier needs no L2 write-back or invalidate: every wave waits
    // for its stores to be acknowledged, the block meets, and thread 0 signals and polls.
    dev_drain();
    __syncthreads();
    ++phase;
    if (threadIdx.x == 0) {
        int ok = 1;
        const unsigned int target = phase * gridDim.x;
        atomicAdd(p.counter, 1u);
        unsigned int spins = 0;
        while (__hip_atomic_load(p.counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
            __builtin_amdgcn_s_sleep(1);
            if (++spins > p.spin_limit || __hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
                __hip_atomic_store(p.abort_flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                ok = 0;
                break;
            }
        }
        L.flag = ok;
        if (p.trace && blockIdx.x == 0 && phase < (unsigned int)p.trace_cap) p.trace[phase] = wall_clock64();
    }
    __syncthreads();
    return L.flag != 0;
}

// four residual-stream values written by other workgroups
__device__ inline f32x4 ld_x4(const float *p) {
    uint32_t r[4];
    ld_dev16(p, r);
    return f32x4 {u2f(r[0]), u2f(r[1]), u2f(r[2]), u2f(r[3])};
}

// ---- RMSNorm of the M rows of x into LDS (bf16) ---------------------------------------------
__device__ inline void norm_to_lds(const MegaParams &p, const float *weight, float eps, MegaLds &L) {
    const int H = p.hidden;
    for (int m = 0; m < p.M; ++m) {
        const float *row = p.x + (size_t)m * H;
        float sq = 0.0f;
        for (int c = threadIdx.x * 4; c < H; c += 512 * 4) {
            const f32x4 v = ld_x4(row + c);
            sq = fmaf(v[0], v[0], fmaf(v[1], v[1], fmaf(v[2], v[2], fmaf(v[3], v[3], sq))));
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sq += __shfl_xor(sq, off, 64);
        if ((threadIdx.x & 63) == 0) L.part[threadIdx.x >> 6] = sq;
        __syncthreads();
        float tot = 0.0f;
#pragma unroll
        for (int w = 0; w < 8; ++w) tot += L.part[w];
        const float var = 1.0f / sqrtf(tot / (float)H + eps);
        for (int c = threadIdx.x * 4; c < H; c += 512 * 4) {
            const f32x4 v = ld_x4(row + c);
            const f32x4 w = *(const XFT_GLOBAL f32x4 *)gptr(weight + c);
            const uint32_t lo = f32_to_bf16_ref((v[0] * var) * w[0]) | ((uint32_t)f32_to_bf16_ref((v[1] * var) * w[1]) << 16);
            const uint32_t hi = f32_to_bf16_ref((v[2] * var) * w[2]) | ((uint32_t)f32_to_bf16_ref((v[3] * var) * w[3]) << 16);
            *(uint2 *)(&L.g.xn[m][c]) = make_uint2(lo, hi);
        }
        __syncthreads();
    }
}

// ---- GEMV over NT column tiles, the 8 waves splitting K ---------------------------------------
// BF16W: the weight tiles hold bf16 values (32 k per tile) instead of INT8 codes (64 k per tile).
// A_LDS: activations come from L.g.xn, else from global memory A (bf16, row pitch lda).
// After the call L.g.red[wave][m * 33 + t * 16 + c] holds each wave's partial sums; sum_red()
// adds them.  Rows >= M are clamped duplicates and must be ignored.
template <int NT, bool BF16W, bool A_LDS>
__device__ inline void gemv_tiles(const MegaParams &p, const uint8_t *packed, int KT, const int (&tiles)[NT], const uint16_t *A,
        int lda, int K, MegaLds &L) {
    constexpr int U = 4;
    constexpr int KTILE = BF16W ? 32 : 64, KL = BF16W ? 8 : 16, MPT = BF16W ? 1 : 2;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, ml = lane & 15;
    const int nbatch = KT / U;
    const int base = nbatch / 8, rem = nbatch % 8;
    const int b_begin = wave * base + (wave < rem ? wave : rem);
    const int nb = base + (wave < rem ? 1 : 0);

    f32x4 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = f32x4 {0.f, 0.f, 0.f, 0.f};
    const XFT_GLOBAL uint8_t *wbase[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) wbase[t] = gptr(packed) + (size_t)tiles[t] * KT * 1024 + lane * 16;
    int row = ml < p.M ? ml : p.M - 1;
    const uint16_t *alds = &L.g.xn[row][g * KL];
    const XFT_GLOBAL uint16_t *aglb = gptr(A) + (size_t)row * lda + g * KL;

    const mu32x4 zero4 = {0u, 0u, 0u, 0u};
    mu32x4 wbuf[2][U][NT];
    mu32x4 abuf[2][U][MPT];
    auto issue = [&](int buf, int batch) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int kt = batch * U + u;
#pragma unroll
            for (int t = 0; t < NT; ++t) wbuf[buf][u][t] = __builtin_nontemporal_load((const XFT_GLOBAL mu32x4 *)(wbase[t] + (size_t)kt * 1024));
            if constexpr (!A_LDS) {
#pragma unroll
                for (int i = 0; i < MPT; ++i) {
                    const int koff = kt * KTILE + 8 * i;
                    const bool v = koff + 8 <= K - g * KL;
                    uint32_t r[4];
                    ld_dev16((const uint16_t *)(aglb + (v ? koff : -g * KL)), r);
                    const mu32x4 a = {r[0], r[1], r[2], r[3]};
                    abuf[buf][u][i] = v ? a : zero4;
                }
            }
        }
    };
    auto compute = [&](int buf, int batch) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int kt = batch * U + u;
#pragma unroll
            for (int i = 0; i < MPT; ++i) {
                MgFrag a;
                if constexpr (A_LDS) {
                    const int koff = kt * KTILE + 8 * i;
                    const bool v = koff + 8 <= K - g * KL;
                    a.q = v ? *(const mu32x4 *)(alds + koff) : zero4;
                } else {
                    a.q = abuf[buf][u][i];
                }
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    MgFrag w;
                    MgFrag src;
                    src.q = wbuf[buf][u][t];
                    if constexpr (BF16W) {
                        w.q = src.q;
                    } else {
                        const uint32_t c0 = src.u[2 * i], c1 = src.u[2 * i + 1];
                        w.u[0] = mg_pack_hi16((float)(int)(int8_t)(c0), (float)(int)(int8_t)(c0 >> 8));
                        w.u[1] = mg_pack_hi16((float)(int)(int8_t)(c0 >> 16), (float)((int)c0 >> 24));
                        w.u[2] = mg_pack_hi16((float)(int)(int8_t)(c1), (float)(int)(int8_t)(c1 >> 8));
                        w.u[3] = mg_pack_hi16((float)(int)(int8_t)(c1 >> 16), (float)((int)c1 >> 24));
                    }
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w.v, a.v, acc[t], 0, 0, 0);
                }
            }
        }
    };
#define XFT_FENCE() __builtin_amdgcn_sched_barrier(0)
    if (nb > 0) {
        issue(0, b_begin);
        XFT_FENCE();
        int b = 1;
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
#undef XFT_FENCE
    float *mine = L.g.red[wave];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) mine[ml * 33 + t * 16 + 4 * g + r] = acc[t][r];
}

__device__ inline float sum_red(const MegaLds &L, int m, int c) {
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < 8; ++w) s += L.g.red[w][m * 33 + c];
    return s;
}

__device__ inline float mg_silu(float x) {
    return x / (1.0f + fast_exp(-x));
}

__global__ void mega_reset_kernel(unsigned int *counter) {
    if (threadIdx.x == 0) *counter = 0u;
}

__global__ __launch_bounds__(512) void decode_mega_kernel(MegaParams p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char mega_smem[];
    MegaLds &L = *reinterpret_cast<MegaLds *>(mega_smem);
    const int G = gridDim.x, wg = blockIdx.x;
    const int H = p.hidden, M = p.M;
    unsigned int phase = 0;
    if (p.trace && wg == 0 && threadIdx.x == 0) p.trace[0] = wall_clock64();

    // ---- phase 0: record the input ids, embed them ----
    if (wg == 0 && threadIdx.x < M) p.idlog[(size_t)p.step[0] * M + threadIdx.x] = p.ids[threadIdx.x];
    for (int i = wg * 512 + threadIdx.x; i < M * H; i += G * 512) {
        const int m = i / H, c = i % H;
        int id = p.ids[m];
        id = id < 0 ? 0 : (id >= p.vocab ? p.vocab - 1 : id);
        st_dev(&p.x[i], fp16_bits_to_f32(p.embedding[(size_t)id * H + c]));
    }
    if (!grid_barrier(p, phase, L)) return;

    const int qcols = p.qH * 128;
    for (int l = 0; l < p.nlayers; ++l) {
        const MegaLayer &ly = p.layers[l];
        // ================= P1: norm + QKV GEMV + RoPE + KV append =================
        norm_to_lds(p, ly.ln1, p.rms_eps, L);
        {
            const int RP = (p.qH + p.kvH) * 4, VT = p.kvH * 8;
            for (int it = wg; it < RP + VT; it += G) {
                if (it < RP) {
                    const int hh = it >> 2, j = it & 3;
                    const int tiles[2] = {hh * 8 + j, hh * 8 + j + 4};
                    gemv_tiles<2, false, true>(p, ly.wqkv, ly.kt_qkv, tiles, nullptr, 0, H, L);
                    __syncthreads();
                    for (int v = threadIdx.x; v < M * 16; v += 512) {
                        const int m = v >> 4, c = v & 15;
                        const float lo = mg_round_bf16(sum_red(L, m, c) * gptr(ly.sqkv)[tiles[0] * 16 + c]);
                        const float hi = mg_round_bf16(sum_red(L, m, 16 + c) * gptr(ly.sqkv)[tiles[1] * 16 + c]);
                        const int i = j * 16 + c, pos = p.pos[m];
                        const float cs = p.cosT[(size_t)pos * 64 + i], sn = p.sinT[(size_t)pos * 64 + i];
                        const float nlo = fmaf(lo, cs, -(hi * sn)), nhi = fmaf(hi, cs, lo * sn);
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
                    __syncthreads();
                } else {
                    const int vt = it - RP;
                    const int tiles[1] = {(p.qH + p.kvH) * 8 + vt};
                    gemv_tiles<1, false, true>(p, ly.wqkv, ly.kt_qkv, tiles, nullptr, 0, H, L);
                    __syncthreads();
                    for (int v = threadIdx.x; v < M * 16; v += 512) {
                        const int m = v >> 4, c = v & 15;
                        const float val = mg_round_bf16(sum_red(L, m, c) * gptr(ly.sqkv)[tiles[0] * 16 + c]);
                        const int pos = p.pos[m];
                        if (pos < ly.kv.S) {
                            const size_t bh = (size_t)m * ly.kv.H + (vt >> 3);
                            const int d = (vt & 7) * 16 + c;
                            uint16_t *dst = (uint16_t *)ly.kv.v + (bh * (ly.kv.S / 32) + (pos >> 5)) * (size_t)128 * 32 + (size_t)d * 32 + v_slot(pos & 31);
                            st_dev(dst, f32_to_fp16_bits(val));
                        }
                    }
                    __syncthreads();
                }
            }
        }
        if (!grid_barrier(p, phase, L)) return;

        // ================= P2: attention over the cache =================
        {
            AttnParams ap = {};
            ap.kv = ly.kv;
            ap.q = p.q;
            ap.qStride = qcols;
            ap.out = p.att;
            ap.oStride = qcols;
            ap.out_dtype = XFTHIP_BF16;
            ap.B = M;
            ap.S = 1;
            ap.G = p.qH / p.kvH;
            ap.scale = p.scale;
            ap.past = 0;
            ap.past_dev = p.pos;
            ap.nsplit = p.nsplit;
            ap.CG = 1;
            ap.ws = p.ws;
            ap.tickets = p.tickets;
            const int units = M * p.kvH * p.nsplit;
            for (int it = wg; it < units; it += G) {
                const int split = it % p.nsplit, kvh = (it / p.nsplit) % p.kvH, b = it / (p.nsplit * p.kvH);
                attn_unit<false, 8, true>(ap, split, kvh, 0, b, L.attn, [] { __syncthreads(); });
                __syncthreads();
            }
        }
        if (!grid_barrier(p, phase, L)) return;

        // ================= P3: out-projection + residual =================
        for (int it = wg; it < H / 16; it += G) {
            const int tiles[1] = {it};
            gemv_tiles<1, false, false>(p, ly.wo, ly.kt_o, tiles, p.att, qcols, qcols, L);
            __syncthreads();
            for (int v = threadIdx.x; v < M * 16; v += 512) {
                const int m = v >> 4, c = v & 15, n = it * 16 + c;
                float *xp = p.x + (size_t)m * H + n;
                st_dev(xp, ld_dev(xp) + sum_red(L, m, c) * gptr(ly.so)[n]);
            }
            __syncthreads();
        }
        if (!grid_barrier(p, phase, L)) return;

        // ================= P4: norm + gate/up + SwiGLU =================
        norm_to_lds(p, ly.ln2, 1e-6f, L);
        for (int it = wg; it < p.inter / 16; it += G) {
            const int tiles[2] = {2 * it, 2 * it + 1};
            gemv_tiles<2, false, true>(p, ly.wgu, ly.kt_gu, tiles, nullptr, 0, H, L);
            __syncthreads();
            for (int v = threadIdx.x; v < M * 16; v += 512) {
                const int m = v >> 4, c = v & 15;
                const float gate = sum_red(L, m, c) * gptr(ly.sgu)[tiles[0] * 16 + c];
                const float up = sum_red(L, m, 16 + c) * gptr(ly.sgu)[tiles[1] * 16 + c];
                st_dev(&p.h[(size_t)m * p.inter + it * 16 + c], f32_to_bf16_ref(up * mg_silu(gate)));
            }
            __syncthreads();
        }
        if (!grid_barrier(p, phase, L)) return;

        // ================= P5: down projection + residual =================
        for (int it = wg; it < H / 16; it += G) {
            const int tiles[1] = {it};
            gemv_tiles<1, false, false>(p, ly.wdown, ly.kt_down, tiles, p.h, p.inter, p.inter, L);
            __syncthreads();
            for (int v = threadIdx.x; v < M * 16; v += 512) {
                const int m = v >> 4, c = v & 15, n = it * 16 + c;
                float *xp = p.x + (size_t)m * H + n;
                st_dev(xp, ld_dev(xp) + sum_red(L, m, c) * gptr(ly.sdown)[n]);
            }
            __syncthreads();
        }
        if (!grid_barrier(p, phase, L)) return;
    }

    // ================= head: final norm + lm_head =================
    norm_to_lds(p, p.final_norm, p.rms_eps, L);
    for (int it = wg; it < (p.vocab + 15) / 16; it += G) {
        const int tiles[1] = {it};
        gemv_tiles<1, true, true>(p, p.lm_head, p.kt_lm, tiles, nullptr, 0, H, L);
        __syncthreads();
        for (int v = threadIdx.x; v < M * 16; v += 512) {
            const int m = v >> 4, c = v & 15, n = it * 16 + c;
            if (n < p.vocab) st_dev(&p.logits[(size_t)m * p.vocab + n], sum_red(L, m, c));
        }
        __syncthreads();
    }
    if (!grid_barrier(p, phase, L)) return;

    // ================= greedy argmax (first maximum wins), position advance =================
    if (wg < M) {
        float *sv = &L.g.red[0][0];
        int *si = (int *)&L.g.red[4][0];
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

// Host side: called by the model driver.  Returns 0 and sets *supported = 0 when the
// configuration is outside what the persistent kernel covers.
namespace xfthip {

int mega_decode_max_blocks(int *blocks_per_cu) {
    int n = 0;
    XFT_CHECK_HIP(hipFuncSetAttribute((const void *)decode_mega_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(MegaLds)));
    XFT_CHECK_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, decode_mega_kernel, 512, sizeof(MegaLds)));
    *blocks_per_cu = n;
    return 0;
}

int mega_decode_launch(const MegaParams &p, int grid, hipStream_t stream) {
    hipLaunchKernelGGL(mega_reset_kernel, dim3(1), dim3(64), 0, stream, p.counter);
    hipLaunchKernelGGL(decode_mega_kernel, dim3(grid), dim3(512), sizeof(MegaLds), stream, p);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

} // namespace xfthip
