// W8A8 GEMM: per-row asymmetric INT8 quantisation of the activations, int8 x int8 -> int32 MFMA
// against the packed INT8 weight, dequantisation with the scale / zero / sum correction terms and
// the usual epilogues.  Replaces MMHelper::onednn_amx_gemm_f32s8f32_compute, quantize_s8 and
// dequant (reference src/utils/matmul_helper.h:2762-2965).
//
// The packed INT8 tile (16 columns x 64 rows, 16 K-consecutive codes per lane) is exactly the
// "A" operand of v_mfma_i32_16x16x64_i8, so the weight goes from HBM to the matrix core without
// a single ALU instruction; the quantised activation rows are the "B" operand.
#include <mutex>

#include "qgemm.h"

// The dequantisation formula is evaluated as written (multiply, multiply, add): no contraction
// into fused multiply-adds anywhere in this file (plain operators, not the __fmul_rn family,
// whose bodies live in a header compiled with the default contraction); the one fused operation
// of the reference (the activation quantiser) is an explicit fmaf.
#include <type_traits>
#pragma clang fp contract(off)

namespace xfthip {

typedef int i32x4 __attribute__((ext_vector_type(4)));

// ---- activation quantisation: one 256-thread workgroup per row -------------------------------
// zero = (min+max)/2, scale = max(|max-zero|, |zero-min|)/127, q = rne(fma(x, 1/scale, -zero/scale)),
// sum = (sum q) * scale + K * zero   (matmul_helper.h:2810-2853).  min / max and the integer sum do not
// depend on the order of the reduction, so the result is the one of a sequential pass.  A thread moves
// 8 values at a time (16-byte loads, 8-byte stores) where the row pitches allow it.
__device__ inline void w8a8_load8(const void *A, int a_dtype, size_t at, bool wide, float v[8]) {
    if (wide) {
        if (a_dtype == XFTHIP_F32) {
            const f32x4 a = *(const f32x4 *)((const float *)A + at), b = *(const f32x4 *)((const float *)A + at + 4);
            v[0] = a[0], v[1] = a[1], v[2] = a[2], v[3] = a[3], v[4] = b[0], v[5] = b[1], v[6] = b[2], v[7] = b[3];
        } else {
            const i32x4 a = *(const i32x4 *)((const uint16_t *)A + at);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[2 * e] = bf16_to_f32((uint16_t)((uint32_t)a[e] & 0xFFFFu));
                v[2 * e + 1] = bf16_to_f32((uint16_t)((uint32_t)a[e] >> 16));
            }
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = load_as_f32(A, a_dtype, at + e);
    }
}

__global__ __launch_bounds__(256) void w8a8_quantize_kernel(const void *__restrict__ A, int a_dtype, int K, int lda,
        int8_t *__restrict__ qa, int ldq, float *__restrict__ scale, float *__restrict__ zero, float *__restrict__ sum) {
    __shared__ float s_mx[4], s_mn[4];
    __shared__ int s_sum[4];
    const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const size_t base = (size_t)row * lda;
    const int esz = a_dtype == XFTHIP_F32 ? 4 : 2;
    const bool wide = (((size_t)A | ((size_t)lda * esz)) & 15) == 0;
    const bool qwide = (((size_t)qa | (size_t)ldq) & 7) == 0;
    const int nchunk = K >> 3;
    float mx = -INFINITY, mn = INFINITY;
    for (int c = tid; c < nchunk; c += 256) {
        float v[8];
        w8a8_load8(A, a_dtype, base + 8 * (size_t)c, wide, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) mx = fmaxf(mx, v[e]), mn = fminf(mn, v[e]);
    }
    for (int k = 8 * nchunk + tid; k < K; k += 256) {
        const float x = load_as_f32(A, a_dtype, base + k);
        mx = fmaxf(mx, x), mn = fminf(mn, x);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        mn = fminf(mn, __shfl_xor(mn, off, 64));
    }
    if (lane == 0) s_mx[wave] = mx, s_mn[wave] = mn;
    __syncthreads();
    mx = fmaxf(fmaxf(s_mx[0], s_mx[1]), fmaxf(s_mx[2], s_mx[3]));
    mn = fminf(fminf(s_mn[0], s_mn[1]), fminf(s_mn[2], s_mn[3]));
    const float fzero = (mn + mx) / 2.0f;
    const float fscale = fmaxf(fabsf(mx - fzero), fabsf(fzero - mn)) / 127.0f;
    const float vs = 1.0f / fscale, vz = -fzero / fscale;
    int isum = 0;
    int8_t *qrow = qa + (size_t)row * ldq;
    for (int c = tid; c < nchunk; c += 256) {
        float v[8];
        w8a8_load8(A, a_dtype, base + 8 * (size_t)c, wide, v);
        uint32_t w0 = 0, w1 = 0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int q = __float2int_rn(fmaf(v[e], vs, vz));
            isum += q;
            const uint32_t b = (uint32_t)(uint8_t)(int8_t)q;
            if (e < 4)
                w0 |= b << (8 * e);
            else
                w1 |= b << (8 * (e - 4));
        }
        if (qwide) {
            *(uint2 *)(qrow + 8 * (size_t)c) = make_uint2(w0, w1);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) qrow[8 * (size_t)c + e] = (int8_t)((e < 4 ? w0 >> (8 * e) : w1 >> (8 * (e - 4))) & 0xFFu);
        }
    }
    for (int k = 8 * nchunk + tid; k < K; k += 256) {
        const int q = __float2int_rn(fmaf(load_as_f32(A, a_dtype, base + k), vs, vz));
        isum += q;
        qrow[k] = (int8_t)q;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) isum += __shfl_xor(isum, off, 64);
    if (lane == 0) s_sum[wave] = isum;
    __syncthreads();
    if (tid == 0) {
        isum = (s_sum[0] + s_sum[1]) + (s_sum[2] + s_sum[3]);
        scale[row] = fscale;
        zero[row] = fzero;
        const float qs = (float)isum * fscale, kz = (float)K * fzero;
        sum[row] = qs + kz;
    }
}

struct W8A8Params {
    const uint8_t *packed;
    const float *scaleB, *zeroB, *sumB;
    int KT, NTILES, K, N, M;
    const int8_t *qa;
    int ldq;
    const float *sA, *zA, *sumA;
    void *C;
    int ldc, c_dtype, epi;
    const float *bias;
    const void *res;
    int ldres, res_dtype;
    float gamma;
};

// NT column tiles per wave, MT 16-row activation tiles; U = 4 k tiles (256 k) per load batch;
// blockDim.x = 64 * (K slices)
template <int NT, int MT>
__global__ __launch_bounds__(512) void w8a8_gemm_kernel(W8A8Params p) {
    constexpr int U = 4;
    extern __shared__ int smem_i[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int g = lane >> 4, ml = lane & 15;
    const int nbatch = p.KT / U;
    const int base = nbatch / nwaves, rem = nbatch % nwaves;
    const int b_begin = wave * base + (wave < rem ? wave : rem);
    const int nb = base + (wave < rem ? 1 : 0);
    const int nt0 = blockIdx.x * NT;

    i32x4 acc[NT][MT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[t][m] = i32x4 {0, 0, 0, 0};

    const uint8_t *wbase[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        int nt = nt0 + t;
        nt = nt < p.NTILES ? nt : p.NTILES - 1;
        wbase[t] = p.packed + (size_t)nt * p.KT * 1024 + lane * 16;
    }
    const int8_t *abase[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        int row = m * 16 + ml;
        row = row < p.M ? row : p.M - 1;
        abase[m] = p.qa + (size_t)row * p.ldq + g * 16;
    }
    const i32x4 zero4 = {0, 0, 0, 0};
    i32x4 wbuf[2][U][NT], abuf[2][U][MT];
    auto issue = [&](int buf, int batch) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int kt = batch * U + u;
#pragma unroll
            for (int t = 0; t < NT; ++t) wbuf[buf][u][t] = __builtin_nontemporal_load((const i32x4 *)(wbase[t] + (size_t)kt * 1024));
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                // chunk inside the row iff kt*64 + 16 g + 16 <= K (K % 16 == 0 is required)
                const bool v = kt * 64 + g * 16 + 16 <= p.K;
                const i32x4 a = *(const i32x4 *)(abase[m] + (v ? kt * 64 : -g * 16));
                abuf[buf][u][m] = v ? a : zero4;
            }
        }
    };
    auto compute = [&](int buf) {
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    acc[t][m] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wbuf[buf][u][t], abuf[buf][u][m], acc[t][m], 0, 0, 0);
    };
#define XFT_FENCE() __builtin_amdgcn_sched_barrier(0)
    if (nb > 0) {
        issue(0, b_begin);
        XFT_FENCE();
        int b = 1;
        for (; b + 1 < nb; b += 2) {
            issue(1, b_begin + b);
            XFT_FENCE();
            compute(0);
            XFT_FENCE();
            issue(0, b_begin + b + 1);
            XFT_FENCE();
            compute(1);
            XFT_FENCE();
        }
        if (b < nb) {
            issue(1, b_begin + b);
            XFT_FENCE();
            compute(0);
            XFT_FENCE();
            compute(1);
        } else {
            compute(0);
        }
    }
#undef XFT_FENCE

    // exact integer reduction over the K slices, then dequantise
    constexpr int ROWS = 16 * MT, COLS = 16 * NT, LD = COLS + 1;
    int *mine = smem_i + (size_t)wave * ROWS * LD;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int r = 0; r < 4; ++r) mine[(m * 16 + ml) * LD + t * 16 + 4 * g + r] = acc[t][m][r];
    __syncthreads();
    for (int v = threadIdx.x; v < ROWS * COLS; v += blockDim.x) {
        const int m = v / COLS, c = v % COLS;
        const int np = nt0 * 16 + c;
        if (m >= p.M || np >= p.N) continue;
        int tot = 0;
        for (int w = 0; w < nwaves; ++w) tot += smem_i[(size_t)w * ROWS * LD + m * LD + c];
        // C = s32*sA*sB + sumB*sB*zA + sumA*zB, evaluated left to right without contraction
        const float t0 = ((float)tot * p.sA[m]) * p.scaleB[np];
        const float t1 = (p.sumB[np] * p.scaleB[np]) * p.zA[m];
        const float t2 = p.sumA[m] * (p.zeroB ? p.zeroB[np] : 0.0f);
        float x = (t0 + t1) + t2;
        switch (p.epi) {
            case XFTHIP_EPI_BIAS: x += p.bias[np]; break;
            case XFTHIP_EPI_SILU: x = x / (1.0f + fast_exp(-x)); break;
            case XFTHIP_EPI_GELU: {
                float e = fast_exp(1.702f * x);
                x = e / (e + 1.0f) * x;
                break;
            }
            case XFTHIP_EPI_RESMUL: x *= load_as_f32(p.res, p.res_dtype, (size_t)m * p.ldres + np); break;
            case XFTHIP_EPI_RESIDENTIAL:
                if (p.bias) x += p.bias[np];
                x += load_as_f32(p.res, p.res_dtype, (size_t)m * p.ldres + np);
                break;
            case XFTHIP_EPI_RESEXT:
                if (p.bias) x += p.bias[np];
                x = fmaf(p.gamma, load_as_f32(p.res, p.res_dtype, (size_t)m * p.ldres + np), x);
                break;
            default: break;
        }
        store_from_f32(p.C, p.c_dtype, (size_t)m * p.ldc + np, x);
    }
}

template <int NT, int MT>
static int launch_w8a8(const W8A8Params &p, hipStream_t stream) {
    const int nbatch = p.KT / 4;
    int kslices = (nbatch + 1) / 2;
    if (kslices < 1) kslices = 1;
    if (kslices > 8) kslices = 8;
    const size_t smem = (size_t)kslices * (16 * MT) * (16 * NT + 1) * sizeof(int);
    hipLaunchKernelGGL((w8a8_gemm_kernel<NT, MT>), dim3((p.NTILES + NT - 1) / NT), dim3(64 * kslices), smem, stream, p);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

// ---- many activation rows (M > 32): block-tiled int8 MFMA GEMM ------------------------------------
// A workgroup of 4 waves computes a (4 * WN * 32 columns) x (WM * 32 rows) tile with
// v_mfma_i32_32x32x32_i8.  The quantised activation rows are the "A" operand, shared by the four
// waves through a double-buffered LDS tile (64 k bytes per row and step); the packed INT8 weight is
// the "B" operand: lane (column nl, k half h) of k step s finds its 16 K-consecutive codes at
// lane slot (2 s + h) * 16 + (nl & 15) of the 1-KiB tile of column tile nl >> 4, so weights go from
// HBM to the matrix core with one 128-bit load per lane and no ALU work, and every weight tile is
// read once per block of WM * 32 rows.  Integer accumulation is exact; the dequantisation is the
// same expression, evaluated in the same order, as in the M <= 32 kernel: bit-identical results.
typedef int i32x16 __attribute__((ext_vector_type(16)));

// the epilogue of one output value; x is the dequantised sum
__device__ inline float w8a8_epilogue(int epi, float x, float bias, bool has_bias, float r, float gamma) {
    switch (epi) {
        case XFTHIP_EPI_BIAS: return x + bias;
        case XFTHIP_EPI_SILU: return x / (1.0f + fast_exp(-x));
        case XFTHIP_EPI_GELU: {
            const float e = fast_exp(1.702f * x);
            return e / (e + 1.0f) * x;
        }
        case XFTHIP_EPI_RESMUL: return x * r;
        case XFTHIP_EPI_RESIDENTIAL: return (has_bias ? x + bias : x) + r;
        case XFTHIP_EPI_RESEXT: return fmaf(gamma, r, has_bias ? x + bias : x);
        default: return x;
    }
}

// A workgroup is 4 x WR waves: four side by side over 4 * WN * 32 columns, WR on top of each other over
// WR * WM * 32 rows; a wave owns WN x WM accumulator tiles of 32 x 32.  (WR = 2, eight waves on 256 x 256, was
// measured and is no better than 128 x 128 tiles at three workgroups a CU: every dispatch uses WR = 1.)
//
// DIRECT (the 128 x 256 block, K a multiple of 256): the quantised activation rows go from global memory straight into
// LDS (global_load_lds_dwordx4: a wave instruction fills 1 KiB of consecutive LDS from 64 addresses of its choice), a
// step covers 128 k.  Rows are 128 bytes without padding, the 16-byte chunk c of row r in slot c ^ ((r >> 1) & 7) of
// its row (the lane picks the global chunk that belongs there), which keeps the operand reads free of bank conflicts.
// Four LDS tiles of 16 KB, tile k + 3 requested in step k; the weights of a micro-step (32 k) are loaded two steps
// ahead into the registers its MFMAs have just read; the barrier that ends a step first waits for the wave's requests
// of the step before (s_waitcnt vmcnt: weights and requests retire in order).  Without staging registers and with
// two instead of six weight tiles in registers the block fits two workgroups a CU; every operand read from LDS feeds
// two MFMAs, where the 128 x 128 block (three workgroups a CU) needs one read per MFMA and is bound by the LDS port.
template <int WN, int WM, int WR, bool DIRECT = false>
__global__ __launch_bounds__(256 * WR, DIRECT ? 2 : 1) void w8a8_mfma_kernel(W8A8Params p, int nblocks_n, int nblocks_m) {
    static_assert(!DIRECT || (WR == 1 && WM == 4), "direct-to-LDS form: four waves, 128 rows");
    constexpr int ROWS = 32 * WM, BROWS = ROWS * WR, ROWB = DIRECT ? 128 : 64 + 16; // rows of a wave / of the block, LDS row pitch in bytes
    constexpr int CHUNKS = BROWS * 4; // 16-byte chunks of an activation tile
    constexpr int ALOADS = CHUNKS / (256 * WR);
    static_assert(CHUNKS % (256 * WR) == 0, "an activation tile must split evenly over the workgroup");
    constexpr int OPITCH = 32 * WN * 4 + 32; // row pitch in bytes of a wave's result patch
    constexpr int NTILE_LDS = DIRECT ? 4 : 3;
    constexpr int STAT_OFF = NTILE_LDS * BROWS * ROWB > 4 * WR * 32 * OPITCH ? NTILE_LDS * BROWS * ROWB : 4 * WR * 32 * OPITCH;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_a[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = lane >> 5, nl = lane & 31;
    // block -> (column block, row block): blocks that share a column block sit on the same XCD; row
    // blocks are walked in bands of 8, all column blocks of a band before the next band
    int nb, mb;
    {
        constexpr int BAND = 8;
        const int id = blockIdx.x, xcd = id & 7, slot = id >> 3;
        const int nb8 = (nblocks_n + 7) >> 3;
        if (slot >= nb8 * nblocks_m) return;
        const int band = slot / (nb8 * BAND), rem = slot - band * (nb8 * BAND);
        const int left = nblocks_m - band * BAND, rows_in_band = left < BAND ? left : BAND;
        nb = rem / rows_in_band + xcd * nb8;
        mb = band * BAND + rem % rows_in_band;
        if (nb >= nblocks_n) return;
    }
    const int wave_c = wave & 3, wave_r = wave >> 2;
    const int n32_0 = (nb * 4 + wave_c) * WN;
    const int m0 = mb * BROWS, mw = wave_r * ROWS; // first row of the block, of this wave inside the block

    i32x16 acc[WN][WM];
#pragma unroll
    for (int t = 0; t < WN; ++t)
#pragma unroll
        for (int m = 0; m < WM; ++m)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[t][m][j] = 0;

    const uint8_t *wbase[WN];
#pragma unroll
    for (int t = 0; t < WN; ++t) {
        int nt = (n32_0 + t) * 2 + (nl >> 4);
        nt = nt < p.NTILES ? nt : p.NTILES - 1;
        wbase[t] = p.packed + (size_t)nt * p.KT * 1024 + h * 256 + (nl & 15) * 16;
    }
    // per-row statistics of this row block, kept behind the tiles / result patches for the epilogue
    float *rowstat = (float *)(lds_a + STAT_OFF);
    if (threadIdx.x < BROWS) {
        int row = m0 + threadIdx.x;
        row = row < p.M ? row : p.M - 1;
        rowstat[threadIdx.x] = p.sA[row];
        rowstat[BROWS + threadIdx.x] = p.zA[row];
        rowstat[2 * BROWS + threadIdx.x] = p.sumA[row];
    }
    if constexpr (DIRECT) {
        constexpr int TILEB = BROWS * ROWB, MICRO = 4, REQS_PER_STEP = MICRO * WN + 4;
        const int kt_n = p.K / 128; // (even: the launcher takes this form for K % 256 == 0 only)
        const int wave_u = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        // request i of this wave fills LDS chunks 64 (4 wave + i) ..+ 63 = rows 8 (4 wave + i) ..+ 7 of a tile; this
        // lane's chunk is slot lane & 7 of row lane >> 3 of those and holds global chunk slot ^ swizzle(row)
        uint32_t a_off[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = 8 * (4 * wave_u + i) + (lane >> 3);
            int row = m0 + r;
            row = row < p.M ? row : p.M - 1;
            a_off[i] = (uint32_t)row * (uint32_t)p.ldq + ((lane & 7) ^ ((r >> 1) & 7)) * 16;
        }
        const uint64_t a_bits = (uint64_t)(uintptr_t)p.qa; // the same in every lane; said so, for a scalar register pair
        const int8_t *a_uniform = (const int8_t *)(uintptr_t)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(a_bits >> 32)) << 32) |
                (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a_bits));
        const uint32_t lds_tiles = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds_a + 4096 * (uint32_t)wave_u;
        // (assembly, not the compiler's builtin: after that one every later counted wait becomes a wait for all loads.
        // M0 carries the LDS address of the wave's first lane; one wait state between writing it and the request.)
        auto request_a = [&](int buf, int kt_raw, int i) {
            const int kt = __builtin_amdgcn_readfirstlane(kt_raw < kt_n ? kt_raw : kt_n - 1);
            const uint32_t dst = lds_tiles + buf * TILEB + i * 1024;
            const int8_t *src = a_uniform + (size_t)kt * 128;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(a_off[i]), "s"(src) : "memory");
        };
        // weights of micro-step ms (32 k) of step kt: half ms & 1 of packed tile 2 kt + ms / 2
        i32x4 wreg[2][MICRO][WN];
        auto load_w = [&](int slot, int kt_raw, int ms) {
            const int kt = kt_raw < kt_n ? kt_raw : kt_n - 1;
#pragma unroll
            for (int t = 0; t < WN; ++t) wreg[slot][ms][t] = *(const i32x4 *)(wbase[t] + (size_t)(2 * kt + (ms >> 1)) * 1024 + (ms & 1) * 512);
        };
        // operand of micro-step ms: bytes 32 ms + 16 h ..+ 15 of a row = chunk 2 ms + h
        i32x4 afr[2][WM];
        auto read_frags = [&](int slot, int buf, int ms) {
            const unsigned char *src = lds_a + buf * TILEB + (mw + nl) * ROWB + (((2 * ms + h) ^ ((nl >> 1) & 7)) << 4);
#pragma unroll
            for (int m = 0; m < WM; ++m) afr[slot][m] = *(const i32x4 *)(src + m * 32 * ROWB);
        };
#pragma unroll
        for (int d = 0; d < 3; ++d) {
            if (d < 2) {
#pragma unroll
                for (int ms = 0; ms < MICRO; ++ms) load_w(d, d, ms);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) request_a(d, d, i);
        }
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        read_frags(0, 0, 0);
        int lds_cur = 0;
        auto step = [&](auto slot_tag, int kt) {
            constexpr int SLOT = decltype(slot_tag)::value;
            const int lds_next = (lds_cur + 1) & 3, lds_req = (lds_cur + 3) & 3;
#pragma unroll
            for (int ms = 0; ms < MICRO; ++ms) {
                request_a(lds_req, kt + 3, ms);
                if (ms + 1 < MICRO)
                    read_frags((ms + 1) & 1, lds_cur, ms + 1);
                else
                    read_frags((ms + 1) & 1, lds_next, 0);
#pragma unroll
                for (int t = 0; t < WN; ++t)
#pragma unroll
                    for (int m = 0; m < WM; ++m)
                        acc[t][m] = __builtin_amdgcn_mfma_i32_32x32x32_i8(afr[ms & 1][m], wreg[SLOT][ms][t], acc[t][m], 0, 0, 0);
                load_w(SLOT, kt + 2, ms);
            }
            __builtin_amdgcn_sched_barrier(0);
            // everything but this step's requests is in: the tile the next step reads its last operands from
            // (requested in the step before) is complete, and this wave's reads of the tile freed are done
            asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(REQS_PER_STEP) : "memory");
            lds_cur = lds_next;
        };
        for (int kt = 0; kt < kt_n; kt += 2) {
            step(std::integral_constant<int, 0> {}, kt);
            step(std::integral_constant<int, 1> {}, kt + 1);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the requests past the last tile have landed
    } else {
    const int a_kc = threadIdx.x & 3, a_row0 = threadIdx.x >> 2;
    const int8_t *a_src[ALOADS];
#pragma unroll
    for (int i = 0; i < ALOADS; ++i) {
        int row = m0 + a_row0 + 64 * WR * i;
        row = row < p.M ? row : p.M - 1;
        a_src[i] = p.qa + (size_t)row * p.ldq + a_kc * 16;
    }
    const i32x4 zero4 = {0, 0, 0, 0};
    // Six k tiles in flight in registers, three activation tiles in LDS.  At step T the registers of slot
    // T % 6 hold weight tile T, LDS buffers T % 3 and (T + 1) % 3 hold activation tiles T and T + 1 (published by
    // the barriers that ended steps T - 2 and T - 1), and the first operand half of tile T is already in
    // registers.  The step reads the second half, multiplies the first, reads the first half of tile T + 1,
    // multiplies the second, moves activation tile T + 2 from its registers into buffer (T + 2) % 3 (last read in
    // step T - 1), and sends the loads of tile T + 6 into the slot it has just used: no MFMA waits for an LDS
    // read issued in front of it and every global load is four to six steps old when it is needed.  The tile
    // count is rounded up to whole rounds of six steps; tiles past the last one are all zero on the activation
    // side (their weight loads re-read the last tile).
    constexpr int SLOTS = (WR == 1 && WN == 2) ? 6 : 3, TILEB = BROWS * ROWB; // several waves a SIMD share its registers: fewer tiles in flight each
    i32x4 wreg[SLOTS][2][WN], areg[SLOTS][ALOADS];
    bool aval[SLOTS];
    const int kt_n = (p.K + 63) / 64;
    auto load_w = [&](int slot, int kt_raw) {
        const int kt = kt_raw < kt_n ? kt_raw : kt_n - 1;
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int t = 0; t < WN; ++t) wreg[slot][s][t] = *(const i32x4 *)(wbase[t] + (size_t)kt * 1024 + s * 512);
    };
    auto load_a = [&](int slot, int kt) {
        // chunk inside the row iff kt * 64 + 16 a_kc + 16 <= K (K % 16 == 0); otherwise the row start is read and
        // replaced by zeros on its way to LDS (there, not here: the loaded value is not touched before its step)
        const bool v = kt * 64 + a_kc * 16 + 16 <= p.K;
        aval[slot] = v;
#pragma unroll
        for (int i = 0; i < ALOADS; ++i) areg[slot][i] = *(const i32x4 *)(a_src[i] + (v ? kt * 64 : -a_kc * 16));
    };
    auto store_a = [&](int slot, int buf) {
        unsigned char *dst = lds_a + buf * TILEB;
#pragma unroll
        for (int i = 0; i < ALOADS; ++i) *(i32x4 *)(dst + (a_row0 + 64 * WR * i) * ROWB + a_kc * 16) = aval[slot] ? areg[slot][i] : zero4;
    };
    const unsigned char *opnd = lds_a + (mw + nl) * ROWB + 16 * h;
    i32x4 a0[WM], a1[WM];
    auto read_half = [&](i32x4 (&a)[WM], int buf, int s) {
#pragma unroll
        for (int m = 0; m < WM; ++m) a[m] = *(const i32x4 *)(opnd + buf * TILEB + m * 32 * ROWB + 32 * s);
    };
    auto mul_half = [&](const i32x4 (&a)[WM], int slot, int s) {
#pragma unroll
        for (int t = 0; t < WN; ++t)
#pragma unroll
            for (int m = 0; m < WM; ++m) acc[t][m] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[m], wreg[slot][s][t], acc[t][m], 0, 0, 0);
    };
#pragma unroll
    for (int d = 0; d < SLOTS; ++d) {
        load_w(d, d);
        load_a(d, d);
    }
    store_a(0, 0);
    store_a(1, 1);
    __syncthreads();
    read_half(a0, 0, 0);
#define XFT_FENCE() __builtin_amdgcn_sched_barrier(0)
#define XFT_W8_STEP(S)                                  \
    {                                                   \
        read_half(a1, (S) % 3, 1);                      \
        XFT_FENCE();                                    \
        mul_half(a0, (S), 0);                           \
        XFT_FENCE();                                    \
        read_half(a0, ((S) + 1) % 3, 0);                \
        XFT_FENCE();                                    \
        mul_half(a1, (S), 1);                           \
        XFT_FENCE();                                    \
        store_a(((S) + 2) % SLOTS, ((S) + 2) % 3);      \
        load_w((S), kt + (S) + SLOTS);                  \
        load_a((S), kt + (S) + SLOTS);                  \
        __syncthreads();                                \
        XFT_FENCE();                                    \
    }
    for (int kt = 0; kt < kt_n; kt += SLOTS) {
        XFT_W8_STEP(0)
        XFT_W8_STEP(1)
        XFT_W8_STEP(2)
        if constexpr (SLOTS == 6) {
            XFT_W8_STEP(3)
            XFT_W8_STEP(4)
            XFT_W8_STEP(5)
        }
    }
#undef XFT_W8_STEP
#undef XFT_FENCE
    }

    // ---- epilogue: lane holds C[m0 + 32 m + 8 (j / 4) + 4 h + j % 4][32 (n32_0 + t) + nl] ----------
    // Each wave drops one 32-row block of its int32 sums at a time into an LDS patch of its own (constant
    // offsets, so the accumulators stay in registers), then walks the patch in 8-column chunks, consecutive
    // lanes along a row: dequantisation, the epilogue of the call and 16-byte stores run in that short loop.
    __syncthreads(); // every wave is past its last read of the activation tiles
    unsigned char *obuf = lds_a + wave * (32 * OPITCH);
    const bool c_wide = (((size_t)p.C | ((size_t)p.ldc * (p.c_dtype == XFTHIP_F32 ? 4 : 2))) & 15) == 0;
    const bool res_wide = p.res && (((size_t)p.res | ((size_t)p.ldres * (p.res_dtype == XFTHIP_F32 ? 4 : 2))) & 15) == 0;
    int *put_base = (int *)(obuf + 4 * h * OPITCH) + nl;
    constexpr int CPR = 4 * WN; // 8-column chunks a row
    constexpr int ITERS = 32 * CPR / 64, RSTEP = 64 / CPR;
    // a lane keeps the same 8 columns in every pass over the patch: their constants are fetched once
    const int ch = lane % CPR, r0 = lane / CPR;
    const int c = n32_0 * 32 + 8 * ch;
    const bool full = c + 8 <= p.N;
    float sB[8], zB[8], sumBsB[8], bias[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int np = c + e < p.N ? c + e : (c < p.N ? c : 0);
        sB[e] = p.scaleB[np];
        zB[e] = p.zeroB ? p.zeroB[np] : 0.0f;
        sumBsB[e] = p.sumB[np] * sB[e];
        bias[e] = p.bias ? p.bias[np] : 0.0f;
    }
    const bool has_bias = p.bias != nullptr;
    // the epilogue of the call is a compile-time constant inside the loops (one copy of them per epilogue)
    auto run = [&](auto epi_tag) {
        constexpr int EPI = decltype(epi_tag)::value;
        constexpr bool HAS_RES = EPI == XFTHIP_EPI_RESMUL || EPI == XFTHIP_EPI_RESIDENTIAL || EPI == XFTHIP_EPI_RESEXT;
#pragma unroll
        for (int m = 0; m < WM; ++m) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int t = 0; t < WN; ++t)
#pragma unroll
                for (int j = 0; j < 16; ++j) put_base[(8 * (j >> 2) + (j & 3)) * (OPITCH / 4) + 32 * t] = acc[t][m][j];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll 1
            for (int it = 0; it < ITERS; ++it) {
                const int r = r0 + RSTEP * it;
                const int row = m0 + mw + 32 * m + r;
                if (row >= p.M || c >= p.N) continue;
                const int *src = (const int *)(obuf + r * OPITCH) + 8 * ch;
                const i32x4 lo = *(const i32x4 *)src, hi = *(const i32x4 *)(src + 4);
                const int s32[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                const float sA = rowstat[mw + 32 * m + r], zA = rowstat[BROWS + mw + 32 * m + r], sumA = rowstat[2 * BROWS + mw + 32 * m + r];
                float res[8];
                if constexpr (HAS_RES) {
                    const size_t ri = (size_t)row * p.ldres + c;
                    if (full && res_wide) {
                        if (p.res_dtype == XFTHIP_F32) {
                            const f32x4 a = *(const f32x4 *)((const float *)p.res + ri), b = *(const f32x4 *)((const float *)p.res + ri + 4);
                            res[0] = a[0], res[1] = a[1], res[2] = a[2], res[3] = a[3], res[4] = b[0], res[5] = b[1], res[6] = b[2], res[7] = b[3];
                        } else {
                            const i32x4 a = *(const i32x4 *)((const uint16_t *)p.res + ri);
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const uint16_t b0 = (uint16_t)((uint32_t)a[e] & 0xFFFFu), b1 = (uint16_t)((uint32_t)a[e] >> 16);
                                res[2 * e] = p.res_dtype == XFTHIP_BF16 ? bf16_to_f32(b0) : fp16_bits_to_f32(b0);
                                res[2 * e + 1] = p.res_dtype == XFTHIP_BF16 ? bf16_to_f32(b1) : fp16_bits_to_f32(b1);
                            }
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e) res[e] = c + e < p.N ? load_as_f32(p.res, p.res_dtype, ri + e) : 0.0f;
                    }
                }
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    // C = s32*sA*sB + sumB*sB*zA + sumA*zB, evaluated left to right without contraction
                    const float t0 = ((float)s32[e] * sA) * sB[e];
                    const float t1 = sumBsB[e] * zA;
                    const float t2 = sumA * zB[e];
                    float x = (t0 + t1) + t2;
                    if constexpr (EPI == XFTHIP_EPI_BIAS) x = x + bias[e];
                    if constexpr (EPI == XFTHIP_EPI_SILU) x = x / (1.0f + fast_exp(-x));
                    if constexpr (EPI == XFTHIP_EPI_GELU) {
                        const float ex = fast_exp(1.702f * x);
                        x = ex / (ex + 1.0f) * x;
                    }
                    if constexpr (EPI == XFTHIP_EPI_RESMUL) x = x * res[e];
                    if constexpr (EPI == XFTHIP_EPI_RESIDENTIAL) x = (has_bias ? x + bias[e] : x) + res[e];
                    if constexpr (EPI == XFTHIP_EPI_RESEXT) x = fmaf(p.gamma, res[e], has_bias ? x + bias[e] : x);
                    v[e] = x;
                }
                const size_t ci = (size_t)row * p.ldc + c;
                if (full && c_wide) {
                    if (p.c_dtype == XFTHIP_F32) {
                        const f32x4 o0 = {v[0], v[1], v[2], v[3]}, o1 = {v[4], v[5], v[6], v[7]};
                        *(f32x4 *)((float *)p.C + ci) = o0;
                        *(f32x4 *)((float *)p.C + ci + 4) = o1;
                    } else {
                        i32x4 o;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const uint32_t b0 = p.c_dtype == XFTHIP_BF16 ? f32_bits_to_bf16_sel(f2u(v[2 * e])) : f32_to_fp16_bits(v[2 * e]);
                            const uint32_t b1 = p.c_dtype == XFTHIP_BF16 ? f32_bits_to_bf16_sel(f2u(v[2 * e + 1])) : f32_to_fp16_bits(v[2 * e + 1]);
                            o[e] = (int)(b0 | (b1 << 16));
                        }
                        *(i32x4 *)((uint16_t *)p.C + ci) = o;
                    }
                } else {
                    // ragged or unaligned rows: through the patch again, one value at a time
                    float *back = (float *)(obuf + r * OPITCH) + 8 * ch;
#pragma unroll
                    for (int e = 0; e < 8; ++e) back[e] = v[e];
#pragma unroll 1
                    for (int e = 0; e < 8 && c + e < p.N; ++e) store_from_f32(p.C, p.c_dtype, ci + e, back[e]);
                }
            }
        }
    };
    switch (p.epi) {
        case XFTHIP_EPI_BIAS: run(std::integral_constant<int, XFTHIP_EPI_BIAS> {}); break;
        case XFTHIP_EPI_SILU: run(std::integral_constant<int, XFTHIP_EPI_SILU> {}); break;
        case XFTHIP_EPI_GELU: run(std::integral_constant<int, XFTHIP_EPI_GELU> {}); break;
        case XFTHIP_EPI_RESMUL: run(std::integral_constant<int, XFTHIP_EPI_RESMUL> {}); break;
        case XFTHIP_EPI_RESIDENTIAL: run(std::integral_constant<int, XFTHIP_EPI_RESIDENTIAL> {}); break;
        case XFTHIP_EPI_RESEXT: run(std::integral_constant<int, XFTHIP_EPI_RESEXT> {}); break;
        default: run(std::integral_constant<int, XFTHIP_EPI_NONE> {}); break;
    }
}

template <int WN, int WM, int WR, bool DIRECT = false>
static int launch_w8a8_mfma(const W8A8Params &p, hipStream_t stream) {
    const int n32 = (p.NTILES + 1) / 2;
    const int brows = 32 * WM * WR;
    const int nblocks_n = (n32 + 4 * WN - 1) / (4 * WN);
    const int nblocks_m = (p.M + brows - 1) / brows;
    const int blocks = ((nblocks_n + 7) / 8) * 8 * nblocks_m;
    const size_t tiles = DIRECT ? 4 * (size_t)brows * 128 : 3 * (size_t)brows * (64 + 16), patches = 4 * WR * 32 * (size_t)(32 * WN * 4 + 32);
    // the result patches reuse the activation tiles; the per-row statistics sit behind both
    const size_t smem = (tiles > patches ? tiles : patches) + 3 * (size_t)brows * sizeof(float);
    if (smem > 64 * 1024) {
        static const hipError_t attr = hipFuncSetAttribute((const void *)w8a8_mfma_kernel<WN, WM, WR, DIRECT>,
                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        XFT_CHECK_HIP(attr);
    }
    hipLaunchKernelGGL((w8a8_mfma_kernel<WN, WM, WR, DIRECT>), dim3(blocks), dim3(256 * WR), smem, stream, p, nblocks_n, nblocks_m);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}


} // namespace xfthip

using namespace xfthip;

extern "C" {

int xfthip_w8a8_quantize_rows(const void *A, int a_dtype, int M, int K, int lda, int8_t *qa, int ldq, float *scale,
        float *zero, float *sum, xfthip_stream_t stream) {
    XFT_REQUIRE(A && qa && scale && zero && sum, "xfthip_w8a8_quantize_rows: null argument");
    XFT_REQUIRE(M > 0 && K > 0 && lda >= K && ldq >= K, "xfthip_w8a8_quantize_rows: bad shape");
    XFT_REQUIRE(a_dtype == XFTHIP_F32 || a_dtype == XFTHIP_BF16, "xfthip_w8a8_quantize_rows: dtype must be f32 or bf16");
    hipLaunchKernelGGL(w8a8_quantize_kernel, dim3(M), dim3(256), 0, (hipStream_t)stream, A, a_dtype, K, lda, qa, ldq, scale, zero, sum);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

int xfthip_gemm_w8a8(xfthip_weight_t w, int M, const int8_t *qa, int ldq, const float *scaleA, const float *zeroA,
        const float *sumA, void *C, int ldc, int c_dtype, int epilogue, const float *bias, const void *res, int ldres,
        int res_dtype, float gamma, xfthip_stream_t stream) {
    XFT_REQUIRE(w && qa && scaleA && zeroA && sumA && C, "xfthip_gemm_w8a8: null argument");
    const PackedWeight &pw = w->pw;
    XFT_REQUIRE(pw.kind == XFTHIP_W_W8A8, "xfthip_gemm_w8a8: weight kind is %d, not W8A8", pw.kind);
    XFT_REQUIRE(M > 0 && ldq >= pw.K && (ldq % 16) == 0 && ((uintptr_t)qa & 15) == 0 && (pw.K % 16) == 0,
            "xfthip_gemm_w8a8: qa must be 16-byte aligned with ldq %% 16 == 0 and K %% 16 == 0");
    XFT_REQUIRE(ldc >= pw.N, "xfthip_gemm_w8a8: ldc=%d < N=%d", ldc, pw.N);
    XFT_REQUIRE(c_dtype == XFTHIP_F32 || c_dtype == XFTHIP_BF16, "xfthip_gemm_w8a8: c_dtype must be f32 or bf16");
    XFT_REQUIRE(epilogue >= XFTHIP_EPI_NONE && epilogue <= XFTHIP_EPI_RESEXT, "xfthip_gemm_w8a8: unknown epilogue %d", epilogue);
    XFT_REQUIRE(epilogue != XFTHIP_EPI_BIAS || bias, "xfthip_gemm_w8a8: bias epilogue without bias");
    const bool needs_res = epilogue == XFTHIP_EPI_RESMUL || epilogue == XFTHIP_EPI_RESIDENTIAL || epilogue == XFTHIP_EPI_RESEXT;
    XFT_REQUIRE(!needs_res || (res && ldres >= pw.N), "xfthip_gemm_w8a8: epilogue %d needs res with ldres >= N", epilogue);
    const size_t csz = c_dtype == XFTHIP_F32 ? 4 : 2, rsz = res_dtype == XFTHIP_F32 ? 4 : 2;
    const int cus = device_cu_count();
    if (M > 32) {
        // block-tiled kernel: every weight tile is read once per 128 (or 64) rows
        W8A8Params p = {};
        p.packed = pw.packed, p.scaleB = pw.scale, p.zeroB = pw.zero, p.sumB = pw.colsum;
        p.KT = pw.KT, p.NTILES = pw.NTILES, p.K = pw.K, p.N = pw.N, p.M = M;
        p.qa = qa, p.ldq = ldq, p.sA = scaleA, p.zA = zeroA, p.sumA = sumA;
        p.C = C, p.ldc = ldc, p.c_dtype = c_dtype, p.epi = epilogue, p.bias = bias;
        p.res = res, p.ldres = ldres, p.res_dtype = res_dtype, p.gamma = gamma;
        const int n32 = (pw.NTILES + 1) / 2;
        // Staged through registers (other K): 128 x 128 tiles once they give every CU its three resident workgroups
        // (registers allow three), else 128 x 256 with one (eight-wave 256 x 256 blocks were no better anywhere)
        const long t_large = (long)((n32 + 7) / 8) * ((M + 127) / 128);
        const long t_mid = (long)((n32 + 3) / 4) * ((M + 127) / 128);
        // 128 x 256 blocks with the activation rows straight into LDS, two workgroups a CU, wherever they give every
        // CU a block and K is a whole number of step pairs (the kernel keeps a lane's byte offset into the rows in 32
        // bits).  With the quantisation of the rows, 2048 / 4096 / 8192 rows on 4096x4096 / 11008x4096 / 4096x11008:
        // 58 / 130 / 129, 94 / 251 / 226 and 184 / 488 / 483 us against 64 / 163 / 148, 112 / 309 / 317 and
        // 231 / 583 / 604 us for the forms below.
        if (t_large >= cus && pw.K % 256 == 0 && (size_t)M * (size_t)ldq < ((size_t)1 << 32))
            return launch_w8a8_mfma<2, 4, 1, true>(p, (hipStream_t)stream);
        if (t_mid >= 3 * cus) return launch_w8a8_mfma<1, 4, 1>(p, (hipStream_t)stream);
        if (t_large >= cus) return launch_w8a8_mfma<2, 4, 1>(p, (hipStream_t)stream);
        return launch_w8a8_mfma<1, 2, 1>(p, (hipStream_t)stream);
    }
    for (int m0 = 0; m0 < M; m0 += 32) {
        W8A8Params p = {};
        p.packed = pw.packed;
        p.scaleB = pw.scale;
        p.zeroB = pw.zero;
        p.sumB = pw.colsum;
        p.KT = pw.KT;
        p.NTILES = pw.NTILES;
        p.K = pw.K;
        p.N = pw.N;
        p.M = M - m0 < 32 ? M - m0 : 32;
        p.qa = qa + (size_t)m0 * ldq;
        p.ldq = ldq;
        p.sA = scaleA + m0;
        p.zA = zeroA + m0;
        p.sumA = sumA + m0;
        p.C = (char *)C + (size_t)m0 * ldc * csz;
        p.ldc = ldc;
        p.c_dtype = c_dtype;
        p.epi = epilogue;
        p.bias = bias;
        p.res = res ? (const char *)res + (size_t)m0 * ldres * rsz : nullptr;
        p.ldres = ldres;
        p.res_dtype = res_dtype;
        p.gamma = gamma;
        const bool wide = p.NTILES / 2 >= 2 * cus;
        int rc;
        if (p.M <= 16)
            rc = wide ? launch_w8a8<2, 1>(p, (hipStream_t)stream) : launch_w8a8<1, 1>(p, (hipStream_t)stream);
        else
            rc = wide ? launch_w8a8<2, 2>(p, (hipStream_t)stream) : launch_w8a8<1, 2>(p, (hipStream_t)stream);
        if (rc) return rc;
    }
    return 0;
}

} // extern "C"

namespace xfthip {

// xfthip_gemm on a W8A8 weight: quantise the bf16 activations into the stream's scratch (stream_scratch: one buffer a
// stream, grown on demand, so a first call of a given size is not for use under stream capture), then run the int8
// GEMM.  The model driver keeps a scratch of its own, sized when the weights are attached.
int gemm_w8a8_from_bf16(xfthip_weight_t w, int M, const void *A, int lda, void *C, int ldc, int c_dtype, int epilogue,
        const float *bias, const void *res, int ldres, int res_dtype, float gamma, hipStream_t stream) {
    const int K = w->pw.K;
    const int ldq = (K + 15) / 16 * 16;
    const size_t need = (size_t)M * ldq;
    void *codes = nullptr, *stats = nullptr;
    if (int rc = stream_scratch(kScratchW8a8Codes, stream, need, false, &codes)) return rc;
    if (int rc = stream_scratch(kScratchW8a8Stats, stream, (size_t)M * 3 * sizeof(float), false, &stats)) return rc;
    int8_t *qa = (int8_t *)codes;
    float *sA = (float *)stats, *zA = sA + M, *sumA = sA + 2 * M;
    if (int rc = xfthip_w8a8_quantize_rows(A, XFTHIP_BF16, M, K, lda, qa, ldq, sA, zA, sumA, stream)) return rc;
    return xfthip_gemm_w8a8(w, M, qa, ldq, sA, zA, sumA, C, ldc, c_dtype, epilogue, bias, res, ldres, res_dtype, gamma, stream);
}

} // namespace xfthip
