// RMSNorm, rotary embedding and the KV cache (layout, append with FP16 convert or INT8
// quantisation).  Replaces the reference's rmsnorm_kernels.cpp, rotary_embedding_kernels.cpp,
// KVCacheTensor and xft::quantize.  All HBM-bound elementwise work: one wavefront per row /
// per (token, head), coalesced 128-bit or 32-bit accesses, wave-level reductions.
#include <math.h>

#include <vector>

#include "kvcache.h"

namespace xfthip {

__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// ---- RMSNorm: one 256-thread block per row ------------------------------------------------
// The row is read once with 128-bit loads into registers (up to 8192 columns), squared and
// reduced (wave shuffles + one LDS exchange), then scaled and written from the registers.
// All loads of a thread are issued before the first use, so the kernel costs one memory
// round trip instead of one per element.
template <bool IN_BF16>
__device__ inline void load8(const void *in, size_t idx, float *v) {
    if constexpr (IN_BF16) {
        const uint4 raw = *(const uint4 *)((const uint16_t *)in + idx);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = u2f(w[i] << 16);
            v[2 * i + 1] = u2f(w[i] & 0xFFFF0000u);
        }
    } else {
        const float4 a = *(const float4 *)((const float *)in + idx);
        const float4 b = *(const float4 *)((const float *)in + idx + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
}

template <bool IN_BF16, bool OUT_BF16, int CHUNKS> // CHUNKS x 8 elements per thread
__global__ __launch_bounds__(256) void rmsnorm_vec_kernel(void *__restrict__ out, const void *__restrict__ in,
        const float *__restrict__ weight, int cols, int iStride, int oStride, float eps) {
    __shared__ float part[4];
    const int row = blockIdx.x;
    const size_t ibase = (size_t)row * iStride, obase = (size_t)row * oStride;
    // the norm weights are requested with the row, not behind the reduction's barrier (a second, cold round trip)
    float x[CHUNKS][8], w[CHUNKS][8];
    float sq = 0.0f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int col = (c * 256 + threadIdx.x) * 8;
        if (col < cols) {
            load8<IN_BF16>(in, ibase + col, x[c]);
            load8<false>(weight, col, w[c]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) x[c][i] = 0.0f, w[c][i] = 0.0f;
        }
    }
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
        for (int i = 0; i < 8; ++i) sq = fmaf(x[c][i], x[c][i], sq);
    sq = wave_sum(sq);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = sq;
    __syncthreads();
    const float total = (part[0] + part[1]) + (part[2] + part[3]);
    const float var = 1.0f / sqrtf(total / (float)cols + eps);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int col = (c * 256 + threadIdx.x) * 8;
        if (col < cols) {
            if constexpr (OUT_BF16) {
                uint32_t pk[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t lo = f32_to_bf16_ref((x[c][2 * i] * var) * w[c][2 * i]);
                    const uint32_t hi = f32_to_bf16_ref((x[c][2 * i + 1] * var) * w[c][2 * i + 1]);
                    pk[i] = lo | (hi << 16);
                }
                *(uint4 *)((uint16_t *)out + obase + col) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
            } else {
                float *o = (float *)out + obase + col;
                *(float4 *)o = make_float4((x[c][0] * var) * w[c][0], (x[c][1] * var) * w[c][1], (x[c][2] * var) * w[c][2], (x[c][3] * var) * w[c][3]);
                *(float4 *)(o + 4) = make_float4((x[c][4] * var) * w[c][4], (x[c][5] * var) * w[c][5], (x[c][6] * var) * w[c][6], (x[c][7] * var) * w[c][7]);
            }
        }
    }
}

// generic shape: any column count, stride or alignment
__global__ __launch_bounds__(256) void rmsnorm_kernel(void *__restrict__ out, int out_dtype,
        const void *__restrict__ in, int in_dtype, const float *__restrict__ weight, int cols, int iStride,
        int oStride, float eps) {
    __shared__ float part[4];
    const int row = blockIdx.x;
    const size_t ibase = (size_t)row * iStride, obase = (size_t)row * oStride;
    float sq = 0.0f;
    for (int c = threadIdx.x; c < cols; c += 256) {
        float x = load_as_f32(in, in_dtype, ibase + c);
        sq = fmaf(x, x, sq);
    }
    sq = wave_sum(sq);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = sq;
    __syncthreads();
    const float total = (part[0] + part[1]) + (part[2] + part[3]);
    const float var = 1.0f / sqrtf(total / (float)cols + eps);
    for (int c = threadIdx.x; c < cols; c += 256) {
        float x = load_as_f32(in, in_dtype, ibase + c);
        store_from_f32(out, out_dtype, obase + c, (x * var) * weight[c]);
    }
}

// ---- LayerNorm: one 256-thread block per row -----------------------------------------------
// y = (x - mean) * gamma * (1 / sqrt(E[x^2] - mean^2 + eps)) + beta with the sum and the sum of squares taken in
// one pass and fp32 arithmetic in the reference's order (src/kernels/layernorm_kernels.cpp:27-81).  Not on the
// Llama path's hot loop (its layers use RMSNorm): the generic form only.
__global__ __launch_bounds__(256) void layernorm_kernel(void *__restrict__ out, int out_dtype, const void *__restrict__ in, int in_dtype,
        const float *__restrict__ gamma, const float *__restrict__ beta, int cols, int iStride, int oStride, float eps) {
    __shared__ float part[8];
    const int row = blockIdx.x;
    const size_t ibase = (size_t)row * iStride, obase = (size_t)row * oStride;
    float sum = 0.0f, sq = 0.0f;
    for (int c = threadIdx.x; c < cols; c += 256) {
        const float x = load_as_f32(in, in_dtype, ibase + c);
        sum += x;
        sq = fmaf(x, x, sq);
    }
    sum = wave_sum(sum);
    sq = wave_sum(sq);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = sum, part[4 + (threadIdx.x >> 6)] = sq;
    __syncthreads();
    const float mean = ((part[0] + part[1]) + (part[2] + part[3])) / (float)cols;
    const float var = 1.0f / sqrtf(((part[4] + part[5]) + (part[6] + part[7])) / (float)cols - mean * mean + eps);
    for (int c = threadIdx.x; c < cols; c += 256) {
        const float x = load_as_f32(in, in_dtype, ibase + c);
        store_from_f32(out, out_dtype, obase + c, (x - mean) * gamma[c] * var + beta[c]);
    }
}

// ---- RoPE + KV append ---------------------------------------------------------------------
// One wavefront per (token, head); lane l owns elements l, l+64, ... of the two halves.
// D <= 256, D % 2 == 0.  heads [0, qHeads) are query heads (rotated in place), heads
// [qHeads, qHeads+kvHeads) are key heads (rotated, then appended) and their value heads.
struct RopeKvParams {
    void *qkv;
    int dtype, stride;
    int B, S, qHeads, kvHeads, D;
    const float *cosT, *sinT;
    int past;
    const int *past_dev;
    const int *positions; // optional explicit position per token (standalone rotary call)
    int skip_q; // 1: query heads are left untouched
    int table_full; // 1: tables are [maxPos, D] and the second half reads columns [D/2, D)
    KvView kv; // kv.k == nullptr: no append
    void *key; // standalone rotary: separate key pointer (qkv = query), else nullptr
    int kStride;
};

template <int EPL> // elements per lane in each half: D/2 <= 64*EPL
__global__ __launch_bounds__(64) void rope_kv_kernel(RopeKvParams p) {
    const int lane = threadIdx.x;
    const int head = blockIdx.x;
    const int tok = blockIdx.y;
    const int b = tok / p.S, s = tok % p.S;
    const int half = p.D / 2;
    int past = p.past;
    if (p.past_dev) {
        // a position read from device memory is held inside the cache whatever it contains
        past = p.past_dev[b];
        past = past < 0 ? 0 : past;
        if (p.kv.k && past > p.kv.S - p.S) past = p.kv.S - p.S;
    }
    const int pos = p.positions ? p.positions[tok] : past + s;
    const bool isq = head < p.qHeads;
    if (isq && p.skip_q) return;
    const int kvh = head - p.qHeads;

    char *rowbase;
    size_t col;
    if (isq) {
        rowbase = (char *)p.qkv;
        col = (size_t)tok * p.stride + (size_t)head * p.D;
    } else if (p.key) {
        rowbase = (char *)p.key;
        col = (size_t)tok * p.kStride + (size_t)kvh * p.D;
    } else {
        rowbase = (char *)p.qkv;
        col = (size_t)tok * p.stride + (size_t)(p.qHeads + kvh) * p.D;
    }

    float lo[EPL], hi[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
        const int i = lane + 64 * e;
        if (i < half) {
            float a = load_as_f32(rowbase, p.dtype, col + i);
            float bb = load_as_f32(rowbase, p.dtype, col + i + half);
            if (p.cosT) {
                const size_t trow = (size_t)pos * (p.table_full ? p.D : half);
                const float c = p.cosT[trow + i], sn = p.sinT[trow + i];
                const float c2 = p.table_full ? p.cosT[trow + i + half] : c;
                const float sn2 = p.table_full ? p.sinT[trow + i + half] : sn;
                // reference: fmsub(q, cos, qHalf*sin) ; fmadd(qHalf, cos, q*sin)
                lo[e] = fmaf(a, c, -(bb * sn));
                hi[e] = fmaf(bb, c2, a * sn2);
            } else {
                lo[e] = a;
                hi[e] = bb;
            }
        } else {
            lo[e] = hi[e] = 0.0f;
        }
    }

    if (isq || p.key) {
        // rotated values go back in place (query always; key only in the standalone call)
        if (p.cosT) {
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const int i = lane + 64 * e;
                if (i < half) {
                    store_from_f32(rowbase, p.dtype, col + i, lo[e]);
                    store_from_f32(rowbase, p.dtype, col + i + half, hi[e]);
                }
            }
        }
        if (isq || p.kv.k == nullptr) return;
    }
    if (p.kv.k == nullptr) return;

    // ---- append key row (rotated, from fp32 registers) and value row ----
    const int t = past + s;
    if (t >= p.kv.S) return; // host checks this; never write outside the cache
    const size_t bh = (size_t)b * p.kv.H + kvh;
    // value row: raw from qkv
    const size_t vcol = (size_t)tok * p.stride + (size_t)(p.qHeads + p.kvHeads + kvh) * p.D;
    float vlo[EPL], vhi[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
        const int i = lane + 64 * e;
        vlo[e] = (i < half) ? load_as_f32(p.qkv, p.dtype, vcol + i) : 0.0f;
        vhi[e] = (i < half) ? load_as_f32(p.qkv, p.dtype, vcol + i + half) : 0.0f;
    }
    const size_t vblk = (bh * (p.kv.S / 32) + (t >> 5)) * (size_t)p.D * 32 + v_slot(t & 31);
    if (p.kv.int8) {
        // xft::quantize: max = absmax, factor = max == 0 ? 1 : 127/max, scale = max/127, q = rne(x*factor)
        float km = 0.0f, vm = 0.0f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            km = fmaxf(km, fmaxf(fabsf(lo[e]), fabsf(hi[e])));
            vm = fmaxf(vm, fmaxf(fabsf(vlo[e]), fabsf(vhi[e])));
        }
        km = wave_max(km);
        vm = wave_max(vm);
        const float kf = (km == 0.0f) ? 1.0f : 127.0f / km;
        const float vf = (vm == 0.0f) ? 1.0f : 127.0f / vm;
        if (lane == 0) {
            p.kv.kscale[bh * p.kv.S + t] = km / 127.0f;
            p.kv.vscale[bh * p.kv.S + t] = vm / 127.0f;
        }
        int8_t *kd = (int8_t *)p.kv.k + (bh * p.kv.S + t) * (size_t)p.D;
        int8_t *vd = (int8_t *)p.kv.v + vblk;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            const int i = lane + 64 * e;
            if (i < half) {
                kd[i] = (int8_t)__float2int_rn(lo[e] * kf);
                kd[i + half] = (int8_t)__float2int_rn(hi[e] * kf);
                vd[(size_t)i * 32] = (int8_t)__float2int_rn(vlo[e] * vf);
                vd[(size_t)(i + half) * 32] = (int8_t)__float2int_rn(vhi[e] * vf);
            }
        }
    } else {
        uint16_t *kd = (uint16_t *)p.kv.k + (bh * p.kv.S + t) * (size_t)p.D;
        uint16_t *vd = (uint16_t *)p.kv.v + vblk;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            const int i = lane + 64 * e;
            if (i < half) {
                kd[i] = f32_to_fp16_bits(lo[e]);
                kd[i + half] = f32_to_fp16_bits(hi[e]);
                vd[(size_t)i * 32] = f32_to_fp16_bits(vlo[e]);
                vd[(size_t)(i + half) * 32] = f32_to_fp16_bits(vhi[e]);
            }
        }
    }
}

// ---- RoPE + KV append for many tokens: one workgroup per (head, sequence, 32-token cache block) ------------------
// The per-token kernel above moves 2 bytes a lane and scatters a token's value row over 128 cache rows; with a whole
// prompt to append that is 49152 one-wave workgroups a layer at 512 tokens.  Here thread (token tid / 8, chunk tid % 8)
// moves the 8 + 8 values of a rotation pair's two halves with 16-byte accesses, the key rows leave as 16-byte (FP16) or
// 8-byte (INT8) stores, and the value rows of a block are turned through LDS into the cache's [dim][32 slots] tile and
// leave as 16-byte runs.  Blocks the new tokens only partly fill (the first and the last of an append) fall back to
// element stores for the values: the other slots of the tile belong to tokens already there.  Same arithmetic and the
// same rounding points as the per-token kernel.  D = 128, bf16 rows, [maxPos, 64] tables, fused q | k | v rows.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <bool INT8>
__global__ __launch_bounds__(256) void rope_kv_block_kernel(RopeKvParams p, int nblk) {
    __shared__ __attribute__((aligned(16))) unsigned char tile[128 * 32 * 2];
    const int head = blockIdx.x;
    const int b = blockIdx.y / nblk, wb = blockIdx.y % nblk;
    int past = p.past;
    if (p.past_dev) {
        past = p.past_dev[b];
        past = past < 0 ? 0 : past;
        if (past > p.kv.S - p.S) past = p.kv.S - p.S;
    }
    const int cb = (past >> 5) + wb; // cache block of this workgroup
    const int t_lo = past > 32 * cb ? past : 32 * cb;
    int t_hi = past + p.S < 32 * cb + 32 ? past + p.S : 32 * cb + 32;
    t_hi = t_hi < p.kv.S ? t_hi : p.kv.S; // (the host checks the append fits; never write outside the cache)
    if (t_lo >= t_hi) return; // (the whole workgroup)
    const bool isq = head < p.qHeads;
    if (isq && p.skip_q) return;
    const int kvh = head - p.qHeads;
    const int tl = threadIdx.x >> 3, c = threadIdx.x & 7;
    const int t = 32 * cb + tl;
    const bool live = t >= t_lo && t < t_hi;
    const size_t tok = (size_t)b * p.S + (live ? t - past : t_lo - past);
    const uint16_t *row = (const uint16_t *)p.qkv + tok * p.stride + (size_t)head * 128;
    const u32x4 rlo = *(const u32x4 *)(row + 8 * c), rhi = *(const u32x4 *)(row + 64 + 8 * c);
    const float *ct = p.cosT + (size_t)(live ? t : t_lo) * 64 + 8 * c, *st = p.sinT + (size_t)(live ? t : t_lo) * 64 + 8 * c;
    const f32x4 c0 = *(const f32x4 *)ct, c1 = *(const f32x4 *)(ct + 4), s0 = *(const f32x4 *)st, s1 = *(const f32x4 *)(st + 4);
    float lo[8], hi[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t wl = rlo[e >> 1], wh = rhi[e >> 1];
        const float a = bf16_to_f32((uint16_t)(e & 1 ? wl >> 16 : wl)), bb = bf16_to_f32((uint16_t)(e & 1 ? wh >> 16 : wh));
        const float cs = e < 4 ? c0[e & 3] : c1[e & 3], sn = e < 4 ? s0[e & 3] : s1[e & 3];
        // reference: fmsub(q, cos, qHalf*sin) ; fmadd(qHalf, cos, q*sin)
        lo[e] = fmaf(a, cs, -(bb * sn));
        hi[e] = fmaf(bb, cs, a * sn);
    }
    if (isq) {
        if (live) {
            u32x4 olo, ohi;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                olo[e] = (uint32_t)f32_to_bf16_ref(lo[2 * e]) | ((uint32_t)f32_to_bf16_ref(lo[2 * e + 1]) << 16);
                ohi[e] = (uint32_t)f32_to_bf16_ref(hi[2 * e]) | ((uint32_t)f32_to_bf16_ref(hi[2 * e + 1]) << 16);
            }
            uint16_t *dst = (uint16_t *)p.qkv + tok * p.stride + (size_t)head * 128;
            *(u32x4 *)(dst + 8 * c) = olo;
            *(u32x4 *)(dst + 64 + 8 * c) = ohi;
        }
        return;
    }
    // ---- key row into the cache, value row into the tile ----
    const size_t bh = (size_t)b * p.kv.H + kvh;
    const uint16_t *vrow = (const uint16_t *)p.qkv + tok * p.stride + (size_t)(p.qHeads + p.kvHeads + kvh) * 128;
    const u32x4 vl = *(const u32x4 *)(vrow + 8 * c), vh = *(const u32x4 *)(vrow + 64 + 8 * c);
    float vlo[8], vhi[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t wl = vl[e >> 1], wh = vh[e >> 1];
        vlo[e] = bf16_to_f32((uint16_t)(e & 1 ? wl >> 16 : wl));
        vhi[e] = bf16_to_f32((uint16_t)(e & 1 ? wh >> 16 : wh));
    }
    const int slot = v_slot(tl);
    const bool full = t_lo == 32 * cb && t_hi == 32 * cb + 32; // (the whole workgroup)
    const size_t vblk = (bh * (p.kv.S / 32) + cb) * (size_t)128 * 32; // elements
    if constexpr (INT8) {
        // xft::quantize: max = absmax, factor = max == 0 ? 1 : 127/max, scale = max/127, q = rne(x*factor)
        float km = 0.0f, vm = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            km = fmaxf(km, fmaxf(fabsf(lo[e]), fabsf(hi[e])));
            vm = fmaxf(vm, fmaxf(fabsf(vlo[e]), fabsf(vhi[e])));
        }
#pragma unroll
        for (int off = 1; off < 8; off <<= 1) { // the 8 threads of a token are neighbours
            km = fmaxf(km, __shfl_xor(km, off, 64));
            vm = fmaxf(vm, __shfl_xor(vm, off, 64));
        }
        const float kf = (km == 0.0f) ? 1.0f : 127.0f / km;
        const float vf = (vm == 0.0f) ? 1.0f : 127.0f / vm;
        uint32_t klo[2], khi[2];
        int8_t vql[8], vqh[8];
#pragma unroll
        for (int w = 0; w < 2; ++w) {
            klo[w] = khi[w] = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                klo[w] |= (uint32_t)(uint8_t)(int8_t)__float2int_rn(lo[4 * w + e] * kf) << (8 * e);
                khi[w] |= (uint32_t)(uint8_t)(int8_t)__float2int_rn(hi[4 * w + e] * kf) << (8 * e);
            }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            vql[e] = (int8_t)__float2int_rn(vlo[e] * vf);
            vqh[e] = (int8_t)__float2int_rn(vhi[e] * vf);
        }
        if (live) {
            if (c == 0) {
                p.kv.kscale[bh * p.kv.S + t] = km / 127.0f;
                p.kv.vscale[bh * p.kv.S + t] = vm / 127.0f;
            }
            int8_t *kd = (int8_t *)p.kv.k + (bh * p.kv.S + t) * (size_t)128;
            *(uint2 *)(kd + 8 * c) = make_uint2(klo[0], klo[1]);
            *(uint2 *)(kd + 64 + 8 * c) = make_uint2(khi[0], khi[1]);
        }
        int8_t *vd = (int8_t *)p.kv.v + vblk;
        if (full) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                ((int8_t *)tile)[(8 * c + e) * 32 + slot] = vql[e];
                ((int8_t *)tile)[(64 + 8 * c + e) * 32 + slot] = vqh[e];
            }
            __syncthreads();
            *(u32x4 *)(vd + (size_t)threadIdx.x * 16) = *(const u32x4 *)(tile + threadIdx.x * 16); // 128 rows of 32 bytes
        } else if (live) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                vd[(size_t)(8 * c + e) * 32 + slot] = vql[e];
                vd[(size_t)(64 + 8 * c + e) * 32 + slot] = vqh[e];
            }
        }
    } else {
        if (live) {
            u32x4 klo, khi;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                klo[e] = (uint32_t)f32_to_fp16_bits(lo[2 * e]) | ((uint32_t)f32_to_fp16_bits(lo[2 * e + 1]) << 16);
                khi[e] = (uint32_t)f32_to_fp16_bits(hi[2 * e]) | ((uint32_t)f32_to_fp16_bits(hi[2 * e + 1]) << 16);
            }
            uint16_t *kd = (uint16_t *)p.kv.k + (bh * p.kv.S + t) * (size_t)128;
            *(u32x4 *)(kd + 8 * c) = klo;
            *(u32x4 *)(kd + 64 + 8 * c) = khi;
        }
        uint16_t *vd = (uint16_t *)p.kv.v + vblk;
        if (full) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                ((uint16_t *)tile)[(8 * c + e) * 32 + slot] = f32_to_fp16_bits(vlo[e]);
                ((uint16_t *)tile)[(64 + 8 * c + e) * 32 + slot] = f32_to_fp16_bits(vhi[e]);
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 2; ++i) // 128 rows of 64 bytes
                *(u32x4 *)((char *)vd + (size_t)(threadIdx.x + 256 * i) * 16) = *(const u32x4 *)(tile + (threadIdx.x + 256 * i) * 16);
        } else if (live) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                vd[(size_t)(8 * c + e) * 32 + slot] = f32_to_fp16_bits(vlo[e]);
                vd[(size_t)(64 + 8 * c + e) * 32 + slot] = f32_to_fp16_bits(vhi[e]);
            }
        }
    }
}

// ---- export / import between the private layout and the reference's two layouts -----------------
// sbhd = 0: [B][H][S][D] (ENABLE_KV_TRANS, src/common/kvcache_tensor.h:108-112); 1: [S][B][H][D] (:113-117).  The
// INT8 scales are [B][H][S] in both.
__global__ void kv_convert_kernel(KvView kv, int which, void *data, float *scales, int maxSeq, int to_private, int sbhd) {
    const size_t total = (size_t)kv.B * kv.H * maxSeq * kv.D;
    const int esz = kv.int8 ? 1 : 2;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const int d = (int)(i % kv.D);
        const size_t r = i / kv.D;
        const int t = (int)(r % maxSeq);
        const size_t bh = r / maxSeq;
        size_t poff;
        char *priv;
        if (which == 0) {
            priv = (char *)kv.k;
            poff = (bh * kv.S + t) * (size_t)kv.D + d;
        } else {
            priv = (char *)kv.v;
            poff = (bh * (kv.S / 32) + (t >> 5)) * (size_t)kv.D * 32 + (size_t)d * 32 + v_slot(t & 31);
        }
        const size_t b_of = bh / kv.H, h_of = bh % kv.H;
        const size_t ei = sbhd ? (((size_t)t * kv.B + b_of) * kv.H + h_of) * kv.D + d : i;
        char *ext = (char *)data + ei * esz;
        char *in = priv + poff * esz;
        if (to_private) {
            for (int bte = 0; bte < esz; ++bte) in[bte] = ext[bte];
        } else {
            for (int bte = 0; bte < esz; ++bte) ext[bte] = in[bte];
        }
        if (kv.int8 && scales && d == 0) {
            float *ps = (which == 0 ? kv.kscale : kv.vscale) + bh * kv.S + t;
            if (to_private)
                *ps = scales[bh * maxSeq + t];
            else
                scales[bh * maxSeq + t] = *ps;
        }
    }
}

} // namespace xfthip

using namespace xfthip;

extern "C" {

int xfthip_rmsnorm(void *out, int out_dtype, const void *in, int in_dtype, const float *weight, int rows, int cols,
        int iStride, int oStride, float eps, xfthip_stream_t stream) {
    XFT_REQUIRE(out && in && weight, "xfthip_rmsnorm: null argument");
    XFT_REQUIRE(rows > 0 && cols > 0, "xfthip_rmsnorm: bad shape %d x %d", rows, cols);
    XFT_REQUIRE((out_dtype == XFTHIP_F32 || out_dtype == XFTHIP_BF16) && (in_dtype == XFTHIP_F32 || in_dtype == XFTHIP_BF16),
            "xfthip_rmsnorm: dtypes must be f32 or bf16");
    if (iStride == -1) iStride = cols;
    if (oStride == -1) oStride = cols;
    XFT_REQUIRE(iStride >= cols && oStride >= cols, "xfthip_rmsnorm: stride smaller than cols");
    hipStream_t st = (hipStream_t)stream;
    const bool ib = in_dtype == XFTHIP_BF16, ob = out_dtype == XFTHIP_BF16;
    const bool vec = cols % 8 == 0 && cols <= 8192 && iStride % 8 == 0 && oStride % 8 == 0 && ((uintptr_t)in & 15) == 0
            && ((uintptr_t)out & 15) == 0 && ((uintptr_t)weight & 15) == 0;
    if (vec) {
        const int chunks = (cols + 2047) / 2048; // 1..4
#define XFT_RMS(IB, OB, CH) \
    hipLaunchKernelGGL((rmsnorm_vec_kernel<IB, OB, CH>), dim3(rows), dim3(256), 0, st, out, in, weight, cols, iStride, oStride, eps)
#define XFT_RMS_CH(IB, OB)            \
    switch (chunks) {                 \
        case 1: XFT_RMS(IB, OB, 1); break; \
        case 2: XFT_RMS(IB, OB, 2); break; \
        case 3: XFT_RMS(IB, OB, 3); break; \
        default: XFT_RMS(IB, OB, 4); break; \
    }
        if (ib && ob) {
            XFT_RMS_CH(true, true)
        } else if (ib) {
            XFT_RMS_CH(true, false)
        } else if (ob) {
            XFT_RMS_CH(false, true)
        } else {
            XFT_RMS_CH(false, false)
        }
#undef XFT_RMS_CH
#undef XFT_RMS
    } else {
        hipLaunchKernelGGL(rmsnorm_kernel, dim3(rows), dim3(256), 0, st, out, out_dtype, in, in_dtype, weight, cols, iStride,
                oStride, eps);
    }
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

int xfthip_layernorm(void *out, int out_dtype, const void *in, int in_dtype, const float *gamma, const float *beta, int rows, int cols,
        int iStride, int oStride, float eps, xfthip_stream_t stream) {
    XFT_REQUIRE(out && in && gamma && beta, "xfthip_layernorm: null argument");
    XFT_REQUIRE(rows > 0 && cols > 0, "xfthip_layernorm: bad shape %d x %d", rows, cols);
    XFT_REQUIRE((out_dtype == XFTHIP_F32 || out_dtype == XFTHIP_BF16) && (in_dtype == XFTHIP_F32 || in_dtype == XFTHIP_BF16),
            "xfthip_layernorm: dtypes must be f32 or bf16");
    if (iStride == -1) iStride = cols;
    if (oStride == -1) oStride = cols;
    XFT_REQUIRE(iStride >= cols && oStride >= cols, "xfthip_layernorm: stride smaller than cols");
    hipLaunchKernelGGL(layernorm_kernel, dim3(rows), dim3(256), 0, (hipStream_t)stream, out, out_dtype, in, in_dtype, gamma, beta, cols,
            iStride, oStride, eps);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

int xfthip_rope_tables_create(int dim, int maxPos, int base, float scalingFactor, float **cos_dev, float **sin_dev) {
    XFT_REQUIRE(cos_dev && sin_dev, "xfthip_rope_tables_create: null out pointer");
    XFT_REQUIRE(dim > 0 && maxPos > 0 && base > 0, "xfthip_rope_tables_create: bad argument");
    const int half = (dim + 1) / 2;
    std::vector<float> inv(half), c((size_t)maxPos * half), s((size_t)maxPos * half);
    for (int i = 0; i < half; ++i) {
        inv[i] = (float)(1.0 / pow((double)base, (double)((float)(i * 2) / (float)dim)));
        inv[i] /= scalingFactor;
    }
    for (size_t pz = 0; pz < (size_t)maxPos; ++pz)
        for (int j = 0; j < half; ++j) {
            float t = (float)pz * inv[j];
            c[pz * half + j] = cosf(t);
            s[pz * half + j] = sinf(t);
        }
    *cos_dev = *sin_dev = nullptr;
    XFT_CHECK_HIP(hipMalloc((void **)cos_dev, c.size() * sizeof(float)));
    XFT_CHECK_HIP(hipMalloc((void **)sin_dev, s.size() * sizeof(float)));
    XFT_CHECK_HIP(hipMemcpy(*cos_dev, c.data(), c.size() * sizeof(float), hipMemcpyHostToDevice));
    XFT_CHECK_HIP(hipMemcpy(*sin_dev, s.data(), s.size() * sizeof(float), hipMemcpyHostToDevice));
    return 0;
}

static int launch_rope(const RopeKvParams &p, int tokens, hipStream_t stream) {
    const int half = p.D / 2;
    // many tokens of fused bf16 rows into a cache: the block form (see rope_kv_block_kernel for what it assumes)
    if (p.kv.k && p.S >= 16 && p.D == 128 && p.dtype == XFTHIP_BF16 && p.cosT && !p.table_full && !p.positions && !p.key &&
            p.stride % 8 == 0 && ((uintptr_t)p.qkv & 15) == 0 && ((uintptr_t)p.cosT & 15) == 0 && ((uintptr_t)p.sinT & 15) == 0) {
        const int nblk = (p.S + 31) / 32 + 1; // cache blocks an append of S tokens can touch
        dim3 grid(p.qHeads + p.kvHeads, p.B * nblk);
        if (p.kv.int8) hipLaunchKernelGGL(rope_kv_block_kernel<true>, grid, dim3(256), 0, stream, p, nblk);
        else hipLaunchKernelGGL(rope_kv_block_kernel<false>, grid, dim3(256), 0, stream, p, nblk);
        XFT_CHECK_HIP(hipGetLastError());
        return 0;
    }
    dim3 grid(p.qHeads + p.kvHeads, tokens);
    if (half <= 64)
        hipLaunchKernelGGL(rope_kv_kernel<1>, grid, dim3(64), 0, stream, p);
    else
        hipLaunchKernelGGL(rope_kv_kernel<2>, grid, dim3(64), 0, stream, p);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

static int rotary_impl(int dtype, const int *positions, void *query, void *key, const float *embCos, const float *embSin,
        int dim, int qStride, int kStride, int numTokens, int headNum, int headSize, int numKvHeads, int table_full,
        xfthip_stream_t stream);

int xfthip_rotary_embedding(int dtype, const int *positions, void *query, void *key, const float *embCos,
        const float *embSin, int dim, int qStride, int kStride, int numTokens, int headNum, int headSize,
        int numKvHeads, xfthip_stream_t stream) {
    return rotary_impl(dtype, positions, query, key, embCos, embSin, dim, qStride, kStride, numTokens, headNum, headSize,
            numKvHeads, 0, stream);
}

int xfthip_rotary_embedding_full(int dtype, const int *positions, void *query, void *key, const float *embCos,
        const float *embSin, int dim, int qStride, int kStride, int numTokens, int headNum, int headSize,
        int numKvHeads, xfthip_stream_t stream) {
    return rotary_impl(dtype, positions, query, key, embCos, embSin, dim, qStride, kStride, numTokens, headNum, headSize,
            numKvHeads, 1, stream);
}

static int rotary_impl(int dtype, const int *positions, void *query, void *key, const float *embCos, const float *embSin,
        int dim, int qStride, int kStride, int numTokens, int headNum, int headSize, int numKvHeads, int table_full,
        xfthip_stream_t stream) {
    XFT_REQUIRE(positions && query && key && embCos && embSin, "xfthip_rotary_embedding: null argument");
    XFT_REQUIRE(dtype == XFTHIP_F32 || dtype == XFTHIP_BF16, "xfthip_rotary_embedding: dtype must be f32 or bf16");
    XFT_REQUIRE(dim == headSize, "xfthip_rotary_embedding: rot dim %d must equal head size %d", dim, headSize);
    XFT_REQUIRE(headSize % 2 == 0 && headSize <= 256, "xfthip_rotary_embedding: head size %d unsupported", headSize);
    XFT_REQUIRE(numTokens > 0 && headNum > 0 && numKvHeads > 0, "xfthip_rotary_embedding: bad shape");
    RopeKvParams p = {};
    p.qkv = query;
    p.key = key;
    p.dtype = dtype;
    p.stride = qStride;
    p.kStride = kStride;
    p.B = 1;
    p.S = numTokens;
    p.qHeads = headNum;
    p.kvHeads = numKvHeads;
    p.D = headSize;
    p.cosT = embCos;
    p.sinT = embSin;
    p.positions = positions;
    p.table_full = table_full;
    return launch_rope(p, numTokens, (hipStream_t)stream);
}

int xfthip_kvcache_create(int dtype, int batch, int kvHeads, int maxSeq, int headSize, xfthip_kvcache_t *out) {
    XFT_REQUIRE(out != nullptr, "xfthip_kvcache_create: null out pointer");
    XFT_REQUIRE(dtype == XFTHIP_FP16 || dtype == XFTHIP_INT8, "xfthip_kvcache_create: dtype must be fp16 or int8");
    XFT_REQUIRE(batch > 0 && kvHeads > 0 && maxSeq > 0, "xfthip_kvcache_create: bad shape");
    XFT_REQUIRE(headSize == 128, "xfthip_kvcache_create: head size %d unsupported (attention kernels are built for 128)", headSize);
    xfthip_kvcache *c = new xfthip_kvcache();
    c->maxSeq = maxSeq;
    KvView &kv = c->kv;
    kv.int8 = dtype == XFTHIP_INT8;
    kv.B = batch;
    kv.H = kvHeads;
    kv.D = headSize;
    kv.S = (maxSeq + 31) / 32 * 32;
    const size_t elems = (size_t)batch * kvHeads * kv.S * headSize;
    const size_t bytes = elems * (kv.int8 ? 1 : 2);
    kv.k = kv.v = nullptr;
    kv.kscale = kv.vscale = nullptr;
    if (hipMalloc(&kv.k, bytes) != hipSuccess || hipMalloc(&kv.v, bytes) != hipSuccess) {
        set_error("xfthip_kvcache_create: hipMalloc of 2 x %zu bytes failed", bytes);
        xfthip_kvcache_destroy(c);
        return 1;
    }
    (void)hipMemset(kv.k, 0, bytes);
    (void)hipMemset(kv.v, 0, bytes);
    if (kv.int8) {
        const size_t sb = (size_t)batch * kvHeads * kv.S * sizeof(float);
        if (hipMalloc((void **)&kv.kscale, sb) != hipSuccess || hipMalloc((void **)&kv.vscale, sb) != hipSuccess) {
            set_error("xfthip_kvcache_create: hipMalloc of scales failed");
            xfthip_kvcache_destroy(c);
            return 1;
        }
        (void)hipMemset(kv.kscale, 0, sb);
        (void)hipMemset(kv.vscale, 0, sb);
    }
    XFT_CHECK_HIP(hipDeviceSynchronize());
    *out = c;
    return 0;
}

int xfthip_kvcache_destroy(xfthip_kvcache_t c) {
    if (!c) return 0;
    if (c->kv.k) (void)hipFree(c->kv.k);
    if (c->kv.v) (void)hipFree(c->kv.v);
    if (c->kv.kscale) (void)hipFree(c->kv.kscale);
    if (c->kv.vscale) (void)hipFree(c->kv.vscale);
    delete c;
    return 0;
}

static int kv_convert(xfthip_kvcache_t c, int which, void *data, float *scales, int to_private, hipStream_t stream, int sbhd = 0) {
    XFT_REQUIRE(c && data, "xfthip_kvcache_export/import: null argument");
    XFT_REQUIRE(which == 0 || which == 1, "xfthip_kvcache_export/import: which must be 0 (keys) or 1 (values)");
    const size_t total = (size_t)c->kv.B * c->kv.H * c->maxSeq * c->kv.D;
    int blocks = (int)((total + 255) / 256 > 1048576 ? 1048576 : (total + 255) / 256);
    hipLaunchKernelGGL(kv_convert_kernel, dim3(blocks), dim3(256), 0, stream, c->kv, which, data, scales, c->maxSeq,
            to_private, sbhd);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

int xfthip_kvcache_export(xfthip_kvcache_t c, int which, void *data_dev, float *scales_dev, xfthip_stream_t stream) {
    return kv_convert(c, which, data_dev, scales_dev, 0, (hipStream_t)stream);
}

int xfthip_kvcache_import(xfthip_kvcache_t c, int which, const void *data_dev, const float *scales_dev,
        xfthip_stream_t stream) {
    XFT_REQUIRE(!(c && c->kv.int8) || scales_dev, "xfthip_kvcache_import: INT8 cache needs scales");
    return kv_convert(c, which, (void *)data_dev, (float *)scales_dev, 1, (hipStream_t)stream);
}

int xfthip_kvcache_export_sbhd(xfthip_kvcache_t c, int which, void *data_dev, float *scales_dev, xfthip_stream_t stream) {
    return kv_convert(c, which, data_dev, scales_dev, 0, (hipStream_t)stream, 1);
}

int xfthip_kvcache_import_sbhd(xfthip_kvcache_t c, int which, const void *data_dev, const float *scales_dev,
        xfthip_stream_t stream) {
    XFT_REQUIRE(!(c && c->kv.int8) || scales_dev, "xfthip_kvcache_import_sbhd: INT8 cache needs scales");
    return kv_convert(c, which, (void *)data_dev, (float *)scales_dev, 1, (hipStream_t)stream, 1);
}

int xfthip_rope_kvstore(xfthip_kvcache_t c, void *qkv, int dtype, int stride, int B, int S, int qHeads,
        const float *embCos, const float *embSin, int past, const int *past_dev, xfthip_stream_t stream) {
    return rope_kvstore_impl(c, qkv, dtype, stride, B, S, qHeads, embCos, embSin, past, past_dev, true, (hipStream_t)stream);
}

} // extern "C"

namespace xfthip {

int rope_kvstore_impl(xfthip_kvcache *c, void *qkv, int dtype, int stride, int B, int S, int qHeads, const float *embCos,
        const float *embSin, int past, const int *past_dev, bool rotate_q, hipStream_t stream) {
    XFT_REQUIRE(c && qkv, "xfthip_rope_kvstore: null argument");
    XFT_REQUIRE(dtype == XFTHIP_F32 || dtype == XFTHIP_BF16, "xfthip_rope_kvstore: dtype must be f32 or bf16");
    XFT_REQUIRE((embCos == nullptr) == (embSin == nullptr), "xfthip_rope_kvstore: cos and sin go together");
    XFT_REQUIRE(B > 0 && B <= c->kv.B, "xfthip_rope_kvstore: batch %d exceeds cache batch %d", B, c->kv.B);
    XFT_REQUIRE(S > 0 && qHeads > 0 && qHeads % c->kv.H == 0, "xfthip_rope_kvstore: bad S=%d or qHeads=%d (kvHeads=%d)", S,
            qHeads, c->kv.H);
    XFT_REQUIRE(stride >= (qHeads + 2 * c->kv.H) * c->kv.D, "xfthip_rope_kvstore: stride %d too small", stride);
    XFT_REQUIRE(past_dev != nullptr || (past >= 0 && past + S <= c->maxSeq),
            "xfthip_rope_kvstore: past %d + S %d exceeds the cache length %d", past, S, c->maxSeq);
    RopeKvParams p = {};
    p.qkv = qkv;
    p.dtype = dtype;
    p.stride = stride;
    p.B = B;
    p.S = S;
    p.qHeads = qHeads;
    p.kvHeads = c->kv.H;
    p.D = c->kv.D;
    p.cosT = embCos;
    p.sinT = embSin;
    p.past = past;
    p.past_dev = past_dev;
    p.kv = c->kv;
    p.skip_q = rotate_q ? 0 : 1;
    return launch_rope(p, B * S, stream);
}

} // namespace xfthip
