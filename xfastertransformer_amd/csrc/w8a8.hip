// W8A8 GEMM: per-row asymmetric INT8 quantisation of the activations, int8 x int8 -> int32 MFMA
// against the packed INT8 weight, dequantisation with the scale / zero / sum correction terms and
// the usual epilogues.  Replaces MMHelper::onednn_amx_gemm_f32s8f32_compute, quantize_s8 and
// dequant (reference src/utils/matmul_helper.h:2762-2965).
//
// The packed INT8 tile (16 columns x 64 rows, 16 K-consecutive codes per lane) is exactly the
// "A" operand of v_mfma_i32_16x16x64_i8, so the weight goes from HBM to the matrix core without
// a single ALU instruction; the quantised activation rows are the "B" operand.
#include "qgemm.h"

// The dequantisation formula is evaluated as written (multiply, multiply, add): no contraction
// into fused multiply-adds anywhere in this file (plain operators, not the __fmul_rn family,
// whose bodies live in a header compiled with the default contraction); the one fused operation
// of the reference (the activation quantiser) is an explicit fmaf.
#pragma clang fp contract(off)

namespace xfthip {

typedef int i32x4 __attribute__((ext_vector_type(4)));

// ---- activation quantisation: one wave per row ---------------------------------------------
// zero = (min+max)/2, scale = max(|max-zero|, |zero-min|)/127, q = rne(fma(x, 1/scale, -zero/scale)),
// sum = (sum q) * scale + K * zero   (matmul_helper.h:2810-2853)
__global__ __launch_bounds__(64) void w8a8_quantize_kernel(const void *__restrict__ A, int a_dtype, int K, int lda,
        int8_t *__restrict__ qa, int ldq, float *__restrict__ scale, float *__restrict__ zero, float *__restrict__ sum) {
    const int row = blockIdx.x, lane = threadIdx.x;
    const size_t base = (size_t)row * lda;
    float mx = -INFINITY, mn = INFINITY;
    for (int k = lane; k < K; k += 64) {
        const float x = load_as_f32(A, a_dtype, base + k);
        mx = fmaxf(mx, x);
        mn = fminf(mn, x);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        mn = fminf(mn, __shfl_xor(mn, off, 64));
    }
    const float fzero = (mn + mx) / 2.0f;
    const float fscale = fmaxf(fabsf(mx - fzero), fabsf(fzero - mn)) / 127.0f;
    const float vs = 1.0f / fscale, vz = -fzero / fscale;
    int isum = 0;
    for (int k = lane; k < K; k += 64) {
        const float x = load_as_f32(A, a_dtype, base + k);
        const int q = __float2int_rn(fmaf(x, vs, vz));
        isum += q;
        qa[(size_t)row * ldq + k] = (int8_t)q;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) isum += __shfl_xor(isum, off, 64);
    if (lane == 0) {
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

template <int WN, int WM>
__global__ __launch_bounds__(256) void w8a8_mfma_kernel(W8A8Params p, int nblocks_n, int nblocks_m) {
    constexpr int ROWS = 32 * WM, ROWB = 64 + 16; // padded LDS row pitch in bytes
    constexpr int CHUNKS = ROWS * 4; // 16-byte chunks of an activation tile
    constexpr int ALOADS = (CHUNKS + 255) / 256;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_a[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = lane >> 5, nl = lane & 31;
    // block -> (column block, row block): blocks that share a column block sit on the same XCD
    int nb, mb;
    {
        const int id = blockIdx.x, xcd = id & 7, slot = id >> 3;
        const int nb8 = (nblocks_n + 7) >> 3;
        nb = (slot / nblocks_m) + xcd * nb8;
        mb = slot % nblocks_m;
        if (slot / nblocks_m >= nb8 || nb >= nblocks_n) return;
    }
    const int n32_0 = (nb * 4 + wave) * WN;
    const int m0 = mb * ROWS;

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
    const int a_kc = threadIdx.x & 3, a_row0 = threadIdx.x >> 2;
    const int8_t *a_src[ALOADS];
#pragma unroll
    for (int i = 0; i < ALOADS; ++i) {
        int row = m0 + a_row0 + 64 * i;
        row = row < p.M ? row : p.M - 1;
        a_src[i] = p.qa + (size_t)row * p.ldq + a_kc * 16;
    }
    const i32x4 zero4 = {0, 0, 0, 0};
    i32x4 wreg[2][2][WN], areg[ALOADS];
    auto load_w = [&](int buf, int kt) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int t = 0; t < WN; ++t) wreg[buf][s][t] = *(const i32x4 *)(wbase[t] + (size_t)kt * 1024 + s * 512);
    };
    auto load_a = [&](int kt) {
        // chunk inside the row iff kt * 64 + 16 a_kc + 16 <= K (K % 16 == 0); otherwise the row start is read and dropped
        const bool v = kt * 64 + a_kc * 16 + 16 <= p.K;
#pragma unroll
        for (int i = 0; i < ALOADS; ++i) {
            const i32x4 a = *(const i32x4 *)(a_src[i] + (v ? kt * 64 : -a_kc * 16));
            areg[i] = v ? a : zero4;
        }
    };
    auto store_a = [&](int buf) {
        unsigned char *dst = lds_a + buf * (ROWS * ROWB);
#pragma unroll
        for (int i = 0; i < ALOADS; ++i)
            if (a_row0 + 64 * i < ROWS) *(i32x4 *)(dst + (a_row0 + 64 * i) * ROWB + a_kc * 16) = areg[i];
    };
    auto compute = [&](int wb, int ab) {
        const unsigned char *src = lds_a + ab * (ROWS * ROWB) + nl * ROWB + 16 * h;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            i32x4 a[WM];
#pragma unroll
            for (int m = 0; m < WM; ++m) a[m] = *(const i32x4 *)(src + m * 32 * ROWB + 32 * s);
#pragma unroll
            for (int t = 0; t < WN; ++t)
#pragma unroll
                for (int m = 0; m < WM; ++m) acc[t][m] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[m], wreg[wb][s][t], acc[t][m], 0, 0, 0);
        }
    };
#define XFT_FENCE() __builtin_amdgcn_sched_barrier(0)
    const int kt_n = (p.K + 63) / 64;
    load_w(0, 0);
    load_a(0);
    store_a(0);
    __syncthreads();
    int kt = 0;
    for (; kt + 2 <= kt_n - 1; kt += 2) {
        load_w(1, kt + 1);
        load_a(kt + 1);
        XFT_FENCE();
        compute(0, 0);
        XFT_FENCE();
        store_a(1);
        __syncthreads();
        load_w(0, kt + 2);
        load_a(kt + 2);
        XFT_FENCE();
        compute(1, 1);
        XFT_FENCE();
        store_a(0);
        __syncthreads();
    }
    if (kt + 1 < kt_n) {
        load_w(1, kt + 1);
        load_a(kt + 1);
        XFT_FENCE();
        compute(0, 0);
        XFT_FENCE();
        store_a(1);
        __syncthreads();
        compute(1, 1);
    } else {
        compute(0, 0);
    }
#undef XFT_FENCE

    // ---- epilogue: lane holds C[m0 + 32 m + 8 (j / 4) + 4 h + j % 4][32 (n32_0 + t) + nl] ----------
#pragma unroll
    for (int t = 0; t < WN; ++t) {
        const int np = (n32_0 + t) * 32 + nl;
        if (np >= p.N) continue;
        const float sB = p.scaleB[np], zB = p.zeroB ? p.zeroB[np] : 0.0f, sumB = p.sumB[np];
        const float bias = p.bias ? p.bias[np] : 0.0f;
#pragma unroll
        for (int m = 0; m < WM; ++m) {
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int row = m0 + 32 * m + 8 * (j >> 2) + 4 * h + (j & 3);
                if (row >= p.M) continue;
                // C = s32*sA*sB + sumB*sB*zA + sumA*zB, evaluated left to right without contraction
                const float t0 = ((float)acc[t][m][j] * p.sA[row]) * sB;
                const float t1 = (sumB * sB) * p.zA[row];
                const float t2 = p.sumA[row] * zB;
                float x = (t0 + t1) + t2;
                switch (p.epi) {
                    case XFTHIP_EPI_BIAS: x += bias; break;
                    case XFTHIP_EPI_SILU: x = x / (1.0f + fast_exp(-x)); break;
                    case XFTHIP_EPI_GELU: {
                        float e = fast_exp(1.702f * x);
                        x = e / (e + 1.0f) * x;
                        break;
                    }
                    case XFTHIP_EPI_RESMUL: x *= load_as_f32(p.res, p.res_dtype, (size_t)row * p.ldres + np); break;
                    case XFTHIP_EPI_RESIDENTIAL:
                        if (p.bias) x += bias;
                        x += load_as_f32(p.res, p.res_dtype, (size_t)row * p.ldres + np);
                        break;
                    case XFTHIP_EPI_RESEXT:
                        if (p.bias) x += bias;
                        x = fmaf(p.gamma, load_as_f32(p.res, p.res_dtype, (size_t)row * p.ldres + np), x);
                        break;
                    default: break;
                }
                store_from_f32(p.C, p.c_dtype, (size_t)row * p.ldc + np, x);
            }
        }
    }
}

template <int WN, int WM>
static int launch_w8a8_mfma(const W8A8Params &p, hipStream_t stream) {
    const int n32 = (p.NTILES + 1) / 2;
    const int nblocks_n = (n32 + 4 * WN - 1) / (4 * WN);
    const int nblocks_m = (p.M + 32 * WM - 1) / (32 * WM);
    const int blocks = ((nblocks_n + 7) / 8) * 8 * nblocks_m;
    const size_t smem = 2 * (size_t)(32 * WM) * (64 + 16);
    hipLaunchKernelGGL((w8a8_mfma_kernel<WN, WM>), dim3(blocks), dim3(256), smem, stream, p, nblocks_n, nblocks_m);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

// scratch for the quantised activations of xfthip_gemm on a W8A8 weight (grown on demand)
static int8_t *g_qa = nullptr;
static float *g_qstat = nullptr;
static size_t g_qa_cap = 0, g_qstat_cap = 0;

} // namespace xfthip

using namespace xfthip;

extern "C" {

int xfthip_w8a8_quantize_rows(const void *A, int a_dtype, int M, int K, int lda, int8_t *qa, int ldq, float *scale,
        float *zero, float *sum, xfthip_stream_t stream) {
    XFT_REQUIRE(A && qa && scale && zero && sum, "xfthip_w8a8_quantize_rows: null argument");
    XFT_REQUIRE(M > 0 && K > 0 && lda >= K && ldq >= K, "xfthip_w8a8_quantize_rows: bad shape");
    XFT_REQUIRE(a_dtype == XFTHIP_F32 || a_dtype == XFTHIP_BF16, "xfthip_w8a8_quantize_rows: dtype must be f32 or bf16");
    hipLaunchKernelGGL(w8a8_quantize_kernel, dim3(M), dim3(64), 0, (hipStream_t)stream, A, a_dtype, K, lda, qa, ldq, scale, zero, sum);
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
        const long t_large = (long)((n32 + 7) / 8) * ((M + 127) / 128);
        if (t_large >= cus) return launch_w8a8_mfma<2, 4>(p, (hipStream_t)stream);
        return launch_w8a8_mfma<1, 2>(p, (hipStream_t)stream);
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

// xfthip_gemm on a W8A8 weight: quantise the bf16 activations into a library-owned scratch, then
// run the int8 GEMM.  The scratch grows with hipMalloc: not for use under stream capture.
int gemm_w8a8_from_bf16(xfthip_weight_t w, int M, const void *A, int lda, void *C, int ldc, int c_dtype, int epilogue,
        const float *bias, const void *res, int ldres, int res_dtype, float gamma, hipStream_t stream) {
    const int K = w->pw.K;
    const int ldq = (K + 15) / 16 * 16;
    const size_t need = (size_t)M * ldq;
    if (need > g_qa_cap) {
        XFT_CHECK_HIP(hipStreamSynchronize(stream));
        if (g_qa) (void)hipFree(g_qa);
        g_qa = nullptr;
        XFT_CHECK_HIP(hipMalloc((void **)&g_qa, need));
        g_qa_cap = need;
    }
    if ((size_t)M * 3 > g_qstat_cap) {
        XFT_CHECK_HIP(hipStreamSynchronize(stream));
        if (g_qstat) (void)hipFree(g_qstat);
        g_qstat = nullptr;
        XFT_CHECK_HIP(hipMalloc((void **)&g_qstat, (size_t)M * 3 * sizeof(float)));
        g_qstat_cap = (size_t)M * 3;
    }
    float *sA = g_qstat, *zA = g_qstat + M, *sumA = g_qstat + 2 * M;
    if (int rc = xfthip_w8a8_quantize_rows(A, XFTHIP_BF16, M, K, lda, g_qa, ldq, sA, zA, sumA, stream)) return rc;
    return xfthip_gemm_w8a8(w, M, g_qa, ldq, sA, zA, sumA, C, ldc, c_dtype, epilogue, bias, res, ldres, res_dtype, gamma, stream);
}

} // namespace xfthip
