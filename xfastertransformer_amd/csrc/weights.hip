// Weight handles: upload of the reference's pre-pack layout, re-tiling into the private
// 1-KiB tile layout (device kernels), the inverse, full-matrix dequantisation and the
// build-owned quantizers.  Replaces MMHelper::convertWeight / packWeight
// (reference src/utils/matmul_helper.h:149-534).
#include <math.h>
#include <string.h>

#include <vector>

#include "common.h"

namespace xfthip {

// NormalFloat4 code values (QLoRA, Dettmers et al. 2023, appendix E)
__constant__ float c_nf4[16] = XFTHIP_NF4_CODE_VALUES;
static const float h_nf4[16] = XFTHIP_NF4_CODE_VALUES;

// ---- forward map: logical (k, n) -> position in the packed buffer -------------------------
struct PackPos {
    size_t byte; // byte offset (bf16: offset of the 2-byte element)
    int hi; // 4-bit kinds: 1 = high nibble
};

__host__ __device__ inline PackPos pack_pos(int kind, int KT, int inter, int k, int n) {
    int np = packed_col(n, inter);
    int nt = np >> 4, nl = np & 15;
    PackPos r;
    if (kind == XFTHIP_W_INT8 || kind == XFTHIP_W_W8A8) {
        int kt = k >> 6, kk = k & 63;
        int lane = nl + 16 * (kk >> 4);
        r.byte = ((size_t)nt * KT + kt) * 1024 + lane * 16 + (kk & 15);
        r.hi = 0;
    } else if (kind == XFTHIP_W_BF16) {
        int kt = k >> 5, kk = k & 31;
        int lane = nl + 16 * (kk >> 3);
        r.byte = ((size_t)nt * KT + kt) * 1024 + lane * 16 + (kk & 7) * 2;
        r.hi = 0;
    } else {
        int kt = k >> 7, kk = k & 127;
        int lane = nl + 16 * (kk >> 5);
        int c = kk & 31, d = c >> 3, e = c & 7;
        // UINT4: pair (e=2p, e=2p+1) at nibbles (p, p+4) so one mask extracts it; NF4: natural
        // order, the pair shares a byte and is looked up with one table read
        int ni = (kind == XFTHIP_W_NF4) ? e : ((e & 1) ? 4 + (e >> 1) : (e >> 1));
        r.byte = ((size_t)nt * KT + kt) * 1024 + lane * 16 + d * 4 + (ni >> 1);
        r.hi = ni & 1;
    }
    return r;
}

// ---- inverse map, written independently: packed byte -> logical (k, n) of its code(s) ------
__device__ inline void unpack_pos8(int KT, size_t byte, int *k, int *np) {
    size_t tile = byte >> 10;
    int in = (int)(byte & 1023);
    int lane = in >> 4, j = in & 15;
    int nt = (int)(tile / KT), kt = (int)(tile % KT);
    *k = kt * 64 + (lane >> 4) * 16 + j;
    *np = nt * 16 + (lane & 15);
}
__device__ inline void unpack_pos4(int kind, int KT, size_t byte, int half, int *k, int *np) {
    size_t tile = byte >> 10;
    int in = (int)(byte & 1023);
    int lane = in >> 4, j = in & 15;
    int nt = (int)(tile / KT), kt = (int)(tile % KT);
    int d = j >> 2;
    int ni = (j & 3) * 2 + half;
    int e = (kind == XFTHIP_W_NF4) ? ni : ((ni < 4) ? 2 * ni : 2 * (ni - 4) + 1);
    *k = kt * 128 + (lane >> 4) * 32 + d * 8 + e;
    *np = nt * 16 + (lane & 15);
}
__device__ inline void unpack_pos16(int KT, size_t elem, int *k, int *np) {
    size_t tile = elem >> 9;
    int in = (int)(elem & 511);
    int lane = in >> 3, j = in & 7;
    int nt = (int)(tile / KT), kt = (int)(tile % KT);
    *k = kt * 32 + (lane >> 4) * 8 + j;
    *np = nt * 16 + (lane & 15);
}

// one thread per packed byte (bf16: per packed element)
__global__ void pack_kernel(int kind, int K, int N, int KT, int NTILES, int inter, const uint8_t *__restrict__ raw,
        uint8_t *__restrict__ packed) {
    size_t total = (size_t)NTILES * KT * 1024;
    if (kind == XFTHIP_W_BF16) total >>= 1;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        int k, np;
        if (kind == XFTHIP_W_INT8 || kind == XFTHIP_W_W8A8) {
            unpack_pos8(KT, i, &k, &np);
            int n = (np < N) ? logical_col(np, inter) : N;
            packed[i] = (k < K && n < N) ? raw[(size_t)k * N + n] : 0;
        } else if (kind == XFTHIP_W_BF16) {
            unpack_pos16(KT, i, &k, &np);
            int n = (np < N) ? logical_col(np, inter) : N;
            ((uint16_t *)packed)[i] = (k < K && n < N) ? ((const uint16_t *)raw)[(size_t)k * N + n] : 0;
        } else {
            uint8_t out = 0;
            for (int half = 0; half < 2; ++half) {
                unpack_pos4(kind, KT, i, half, &k, &np);
                int n = (np < N) ? logical_col(np, inter) : N;
                uint8_t code = 0;
                if (k < K && n < N) {
                    uint8_t b = raw[((size_t)k * N + n) >> 1];
                    code = (n & 1) ? (b >> 4) : (b & 15);
                } else if (kind == XFTHIP_W_NF4) {
                    code = 7; // code value 0.0
                }
                out |= half ? (uint8_t)(code << 4) : code;
            }
            packed[i] = out;
        }
    }
}

// one thread per raw byte (bf16: per element) using the forward map
__global__ void unpack_kernel(int kind, int K, int N, int KT, int inter, const uint8_t *__restrict__ packed,
        uint8_t *__restrict__ raw) {
    size_t total = (size_t)K * N;
    if (kind == XFTHIP_W_UINT4 || kind == XFTHIP_W_NF4) total >>= 1;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        if (kind == XFTHIP_W_INT8 || kind == XFTHIP_W_W8A8) {
            int k = (int)(i / N), n = (int)(i % N);
            raw[i] = packed[pack_pos(kind, KT, inter, k, n).byte];
        } else if (kind == XFTHIP_W_BF16) {
            int k = (int)(i / N), n = (int)(i % N);
            ((uint16_t *)raw)[i] = *(const uint16_t *)(packed + pack_pos(kind, KT, inter, k, n).byte);
        } else {
            size_t e0 = i * 2;
            int k = (int)(e0 / N), n = (int)(e0 % N);
            PackPos p0 = pack_pos(kind, KT, inter, k, n), p1 = pack_pos(kind, KT, inter, k, n + 1);
            uint8_t c0 = p0.hi ? packed[p0.byte] >> 4 : packed[p0.byte] & 15;
            uint8_t c1 = p1.hi ? packed[p1.byte] >> 4 : packed[p1.byte] & 15;
            raw[i] = (uint8_t)(c0 | (c1 << 4));
        }
    }
}

// w[k][n] = fmaf(scale, q, zero) (NF4: code * absmax), optionally narrowed to bf16
__global__ void dequant_kernel(int kind, int K, int N, int KT, int inter, const uint8_t *__restrict__ packed,
        const float *__restrict__ scale, const float *__restrict__ zero, void *__restrict__ out, int out_dtype) {
    size_t total = (size_t)K * N;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        int k = (int)(i / N), n = (int)(i % N);
        PackPos p = pack_pos(kind, KT, inter, k, n);
        int np = packed_col(n, inter);
        float v;
        if (kind == XFTHIP_W_INT8 || kind == XFTHIP_W_W8A8) {
            float z = zero ? zero[np] : 0.0f;
            v = fmaf(scale[np], (float)(int8_t)packed[p.byte], z);
        } else if (kind == XFTHIP_W_BF16) {
            v = bf16_to_f32(*(const uint16_t *)(packed + p.byte));
        } else {
            int code = p.hi ? packed[p.byte] >> 4 : packed[p.byte] & 15;
            if (kind == XFTHIP_W_UINT4) {
                float z = zero ? zero[np] : 0.0f;
                v = fmaf(scale[np], (float)code, z);
            } else {
                v = c_nf4[code] * scale[np];
            }
        }
        if (out_dtype == XFTHIP_F32)
            ((float *)out)[i] = v;
        else
            ((uint16_t *)out)[i] = f32_to_bf16_ref(v);
    }
}

// per-column integer sums of an int8 [K,N] matrix, accumulated in float in row order
// (reference matmul_helper.h:362-372)
__global__ void colsum_kernel(int K, int N, int inter, const int8_t *__restrict__ raw, float *__restrict__ colsum) {
    int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= N) return;
    float s = 0.0f;
    for (int k = 0; k < K; ++k) s += (float)raw[(size_t)k * N + n];
    colsum[packed_col(n, inter)] = s;
}

} // namespace xfthip

using namespace xfthip;

static size_t raw_bytes(int kind, int K, int N) {
    size_t e = (size_t)K * N;
    if (kind == XFTHIP_W_UINT4 || kind == XFTHIP_W_NF4) return e / 2;
    if (kind == XFTHIP_W_BF16) return e * 2;
    return e;
}

extern "C" {

int xfthip_weight_create(int kind, int K, int N, const void *q_host, const float *scale_host,
        const float *zero_host, int flags, xfthip_weight_t *out) {
    XFT_REQUIRE(out != nullptr && q_host != nullptr, "xfthip_weight_create: null argument");
    XFT_REQUIRE(kind >= XFTHIP_W_INT8 && kind <= XFTHIP_W_BF16, "xfthip_weight_create: unknown weight kind %d", kind);
    XFT_REQUIRE(K > 0 && N > 0, "xfthip_weight_create: bad shape K=%d N=%d", K, N);
    XFT_REQUIRE(K % 8 == 0, "xfthip_weight_create: K=%d must be a multiple of 8", K);
    XFT_REQUIRE(kind == XFTHIP_W_BF16 || scale_host != nullptr, "xfthip_weight_create: scale is required");
    XFT_REQUIRE(!((kind == XFTHIP_W_UINT4 || kind == XFTHIP_W_NF4) && (N & 1)),
            "xfthip_weight_create: 4-bit weights need an even N (got %d)", N);
    XFT_REQUIRE(!(kind == XFTHIP_W_W8A8 && (N % 16)), "xfthip_weight_create: W8A8 needs N %% 16 == 0 (got %d)", N);
    int inter = 0;
    if (flags & XFTHIP_WF_GATEUP) {
        XFT_REQUIRE(N % 32 == 0, "xfthip_weight_create: gate/up weight needs N/2 %% 16 == 0 (N=%d)", N);
        inter = N / 2;
    }
    xfthip_weight *w = new xfthip_weight();
    PackedWeight &pw = w->pw;
    memset(&pw, 0, sizeof(pw));
    pw.kind = kind;
    pw.K = K;
    pw.N = N;
    pw.ktile = ktile_of(kind);
    pw.KT = (K + pw.ktile - 1) / pw.ktile;
    // the GEMM streams whole load batches of tiles: pad with zero tiles (decode to 0 / code 7)
    const int kbatch = (kind == XFTHIP_W_UINT4 || kind == XFTHIP_W_NF4) ? 2 : 4;
    pw.KT = (pw.KT + kbatch - 1) / kbatch * kbatch;
    pw.NTILES = (N + 15) / 16;
    pw.flags = flags;
    pw.inter = inter;
    pw.packed_bytes = (size_t)pw.NTILES * pw.KT * 1024;

    size_t rb = raw_bytes(kind, K, N);
    uint8_t *raw = nullptr;
    int rc = 0;
    auto fail = [&](int code) {
        if (raw) (void)hipFree(raw);
        xfthip_weight_destroy(w);
        return code;
    };
    if (hipMalloc((void **)&raw, rb) != hipSuccess) {
        set_error("xfthip_weight_create: hipMalloc(%zu) for staging failed", rb);
        return fail(1);
    }
    if (hipMalloc((void **)&pw.packed, pw.packed_bytes) != hipSuccess) {
        set_error("xfthip_weight_create: hipMalloc(%zu) for packed weight failed", pw.packed_bytes);
        return fail(1);
    }
    if (hipMemcpy(raw, q_host, rb, hipMemcpyHostToDevice) != hipSuccess) {
        set_error("xfthip_weight_create: upload failed");
        return fail(1);
    }
    int npad = pw.NTILES * 16;
    if (kind != XFTHIP_W_BF16) {
        std::vector<float> s(npad, 0.0f), z(npad, 0.0f);
        for (int n = 0; n < N; ++n) {
            s[packed_col(n, inter)] = scale_host[n];
            if (zero_host) z[packed_col(n, inter)] = zero_host[n];
        }
        bool has_zero = false;
        if (zero_host && kind != XFTHIP_W_NF4)
            for (int n = 0; n < N; ++n) has_zero |= (zero_host[n] != 0.0f);
        if (hipMalloc((void **)&pw.scale, npad * sizeof(float)) != hipSuccess
                || hipMemcpy(pw.scale, s.data(), npad * sizeof(float), hipMemcpyHostToDevice) != hipSuccess) {
            set_error("xfthip_weight_create: scale upload failed");
            return fail(1);
        }
        if (has_zero || kind == XFTHIP_W_W8A8) {
            if (hipMalloc((void **)&pw.zero, npad * sizeof(float)) != hipSuccess
                    || hipMemcpy(pw.zero, z.data(), npad * sizeof(float), hipMemcpyHostToDevice) != hipSuccess) {
                set_error("xfthip_weight_create: zero upload failed");
                return fail(1);
            }
        }
    }
    size_t work = (kind == XFTHIP_W_BF16) ? pw.packed_bytes / 2 : pw.packed_bytes;
    int blocks = (int)((work + 255) / 256 > 65535 * 16 ? 65535 * 16 : (work + 255) / 256);
    hipLaunchKernelGGL(pack_kernel, dim3(blocks), dim3(256), 0, 0, kind, K, N, pw.KT, pw.NTILES, inter, raw, pw.packed);
    if (kind == XFTHIP_W_W8A8) {
        if (hipMalloc((void **)&pw.colsum, npad * sizeof(float)) != hipSuccess
                || hipMemset(pw.colsum, 0, npad * sizeof(float)) != hipSuccess) {
            set_error("xfthip_weight_create: colsum alloc failed");
            return fail(1);
        }
        hipLaunchKernelGGL(colsum_kernel, dim3((N + 255) / 256), dim3(256), 0, 0, K, N, inter, (const int8_t *)raw,
                pw.colsum);
    }
    if (hipDeviceSynchronize() != hipSuccess || hipGetLastError() != hipSuccess) {
        set_error("xfthip_weight_create: pack kernel failed");
        return fail(1);
    }
    (void)hipFree(raw);
    (void)rc;
    *out = w;
    return 0;
}

int xfthip_weight_destroy(xfthip_weight_t w) {
    if (!w) return 0;
    if (w->pw.packed) (void)hipFree(w->pw.packed);
    if (w->pw.scale) (void)hipFree(w->pw.scale);
    if (w->pw.zero) (void)hipFree(w->pw.zero);
    if (w->pw.colsum) (void)hipFree(w->pw.colsum);
    delete w;
    return 0;
}

int xfthip_weight_shape(xfthip_weight_t w, int *kind, int *K, int *N) {
    XFT_REQUIRE(w != nullptr, "xfthip_weight_shape: null handle");
    if (kind) *kind = w->pw.kind;
    if (K) *K = w->pw.K;
    if (N) *N = w->pw.N;
    return 0;
}

size_t xfthip_weight_bytes(xfthip_weight_t w) {
    if (!w) return 0;
    size_t side = 0;
    if (w->pw.scale) side += (size_t)w->pw.N * 4;
    if (w->pw.zero) side += (size_t)w->pw.N * 4;
    return raw_bytes(w->pw.kind, w->pw.K, w->pw.N) + side;
}

int xfthip_weight_unpack(xfthip_weight_t w, void *q_host_out) {
    XFT_REQUIRE(w != nullptr && q_host_out != nullptr, "xfthip_weight_unpack: null argument");
    const PackedWeight &pw = w->pw;
    size_t rb = raw_bytes(pw.kind, pw.K, pw.N);
    uint8_t *raw = nullptr;
    XFT_CHECK_HIP(hipMalloc((void **)&raw, rb));
    size_t work = (pw.kind == XFTHIP_W_BF16) ? rb / 2 : rb;
    int blocks = (int)((work + 255) / 256 > 65535 * 16 ? 65535 * 16 : (work + 255) / 256);
    hipLaunchKernelGGL(unpack_kernel, dim3(blocks), dim3(256), 0, 0, pw.kind, pw.K, pw.N, pw.KT, pw.inter, pw.packed,
            raw);
    hipError_t e = hipMemcpy(q_host_out, raw, rb, hipMemcpyDeviceToHost);
    (void)hipFree(raw);
    XFT_CHECK_HIP(e);
    return 0;
}

int xfthip_weight_dequant(xfthip_weight_t w, void *out, int out_dtype, xfthip_stream_t stream) {
    XFT_REQUIRE(w != nullptr && out != nullptr, "xfthip_weight_dequant: null argument");
    XFT_REQUIRE(out_dtype == XFTHIP_F32 || out_dtype == XFTHIP_BF16, "xfthip_weight_dequant: out_dtype must be f32 or bf16");
    const PackedWeight &pw = w->pw;
    size_t work = (size_t)pw.K * pw.N;
    int blocks = (int)((work + 255) / 256 > 65535 * 16 ? 65535 * 16 : (work + 255) / 256);
    hipLaunchKernelGGL(dequant_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, pw.kind, pw.K, pw.N, pw.KT,
            pw.inter, pw.packed, pw.scale, pw.zero, out, out_dtype);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

// Build-owned quantizers: one scale (and zero) per output column of W[K,N].
//   INT8 : s = max|w| / 127, q = clamp(rne(w / s), -127, 127), zero = 0
//   UINT4: s = (max - min) / 15, zero = min, q = clamp(rne((w - min) / s), 0, 15)
//   NF4  : absmax per column, q = index of the nearest code to w / absmax (lowest index on ties)
int xfthip_quantize_weight(int kind, int K, int N, const float *W, void *q_out, float *scale_out, float *zero_out) {
    XFT_REQUIRE(W && q_out && scale_out, "xfthip_quantize_weight: null argument");
    XFT_REQUIRE(K > 0 && N > 0, "xfthip_quantize_weight: bad shape");
    if (kind == XFTHIP_W_INT8 || kind == XFTHIP_W_W8A8) {
        int8_t *q = (int8_t *)q_out;
        for (int n = 0; n < N; ++n) {
            float amax = 0.0f;
            for (size_t k = 0; k < (size_t)K; ++k) amax = fmaxf(amax, fabsf(W[k * N + n]));
            float s = amax / 127.0f;
            scale_out[n] = s;
            if (zero_out) zero_out[n] = 0.0f;
            for (size_t k = 0; k < (size_t)K; ++k) {
                float v = (s == 0.0f) ? 0.0f : nearbyintf(W[k * N + n] / s);
                q[k * N + n] = (int8_t)fminf(fmaxf(v, -127.0f), 127.0f);
            }
        }
        return 0;
    }
    XFT_REQUIRE(kind == XFTHIP_W_UINT4 || kind == XFTHIP_W_NF4, "xfthip_quantize_weight: unsupported kind %d", kind);
    XFT_REQUIRE((N & 1) == 0, "xfthip_quantize_weight: 4-bit kinds need an even N");
    XFT_REQUIRE(kind == XFTHIP_W_NF4 || zero_out != nullptr, "xfthip_quantize_weight: UINT4 needs a zero output");
    uint8_t *q = (uint8_t *)q_out;
    memset(q, 0, (size_t)K * N / 2);
    for (int n = 0; n < N; ++n) {
        float mn = W[n], mx = W[n], amax = 0.0f;
        for (size_t k = 0; k < (size_t)K; ++k) {
            float v = W[k * N + n];
            mn = fminf(mn, v);
            mx = fmaxf(mx, v);
            amax = fmaxf(amax, fabsf(v));
        }
        float s = (kind == XFTHIP_W_UINT4) ? (mx - mn) / 15.0f : amax;
        scale_out[n] = s;
        if (kind == XFTHIP_W_UINT4) zero_out[n] = mn;
        for (size_t k = 0; k < (size_t)K; ++k) {
            int code;
            if (kind == XFTHIP_W_UINT4) {
                float v = (s == 0.0f) ? 0.0f : nearbyintf((W[k * N + n] - mn) / s);
                code = (int)fminf(fmaxf(v, 0.0f), 15.0f);
            } else {
                float v = (s == 0.0f) ? 0.0f : W[k * N + n] / s;
                code = 0;
                float bd = fabsf(v - h_nf4[0]);
                for (int c = 1; c < 16; ++c) {
                    float d = fabsf(v - h_nf4[c]);
                    if (d < bd) {
                        bd = d;
                        code = c;
                    }
                }
            }
            q[(k * N + n) >> 1] |= (n & 1) ? (uint8_t)(code << 4) : (uint8_t)code;
        }
    }
    return 0;
}

} // extern "C"
