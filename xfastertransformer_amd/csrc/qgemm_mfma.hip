// Dequant-fused weight-only GEMM for many activation rows (M > 32): the prefill shape.
// Replaces MMHelper::compute* (reference src/utils/matmul_helper.h:565-1705) at large M, where
// the reference switches to AMX (oneDNN) kernels.  The kernel lives in qgemm_mfma_impl.h; this
// file picks the weight kind.
#include <mutex>

#include "qgemm.h"

namespace xfthip {

int qgemm_mfma_int8(const SkinnyParams &p, hipStream_t stream);
int qgemm_mfma_int8z(const SkinnyParams &p, hipStream_t stream);
int qgemm_mfma_uint4(const SkinnyParams &p, hipStream_t stream);
int qgemm_mfma_nf4(const SkinnyParams &p, hipStream_t stream);
int qgemm_mfma_bf16(const SkinnyParams &p, hipStream_t stream);

namespace {

__device__ inline float silu_split(float x) {
    return x / (1.0f + fast_exp(-x));
}

// One thread per VEC neighbouring output values of a row (4 where N allows 16-byte part loads, else 1): the K parts are
// added in order (the same result on every run), then the epilogue of the call.  p.C / p.ldc / p.c_dtype / p.epi are
// the caller's.
template <int VEC>
__global__ __launch_bounds__(256) void qgemm_split_finish_kernel(SkinnyParams p) {
    const int nv = p.N / VEC;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)p.M * nv) return;
    const int m = (int)(idx / nv), n0 = (int)(idx - (size_t)m * nv) * VEC;
    int row_out = m;
    if (p.group) {
        // the parts hold the rows where C holds them; rows past the last weight's were never written
        int total = 0;
        for (int e = 0; e < p.group_n; ++e) total += p.rows_dev[e * p.rows_stride];
        if (m >= total) return;
    } else if (p.rows_dev) {
        if (m >= p.rows_dev[0]) return;
        row_out = m + p.rows_dev[2];
    }
    float x[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) x[v] = 0.0f;
    for (int s = 0; s < p.ksplit; ++s) {
        const float *src = p.split_part + ((size_t)s * p.M + m) * p.N + n0;
        if constexpr (VEC == 4) {
            const float4 t = *(const float4 *)src;
            x[0] += t.x, x[1] += t.y, x[2] += t.z, x[3] += t.w;
        } else {
            x[0] += src[0];
        }
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        const int n = n0 + v;
        float y = x[v];
        switch (p.epi) {
            case XFTHIP_EPI_BIAS: y += p.bias[n]; break;
            case XFTHIP_EPI_SILU: y = silu_split(y); break;
            case XFTHIP_EPI_GELU: {
                const float e = fast_exp(1.702f * y);
                y = e / (e + 1.0f) * y;
                break;
            }
            case XFTHIP_EPI_RESMUL: y *= load_as_f32(p.res, p.res_dtype, (size_t)m * p.ldres + n); break;
            case XFTHIP_EPI_RESIDENTIAL:
                if (p.bias) y += p.bias[n];
                y += load_as_f32(p.res, p.res_dtype, (size_t)m * p.ldres + n);
                break;
            case XFTHIP_EPI_RESEXT:
                if (p.bias) y += p.bias[n];
                y = fmaf(p.gamma, load_as_f32(p.res, p.res_dtype, (size_t)m * p.ldres + n), y);
                break;
            default: break;
        }
        x[v] = y;
    }
    const size_t ci = (size_t)row_out * p.ldc + n0;
    if constexpr (VEC == 4) {
        // whole 16-byte (fp32) or 8-byte (16-bit) stores where the row start allows them
        if (p.c_dtype == XFTHIP_F32 && ((((uintptr_t)p.C) | ((size_t)p.ldc * 4)) & 15) == 0) {
            *(float4 *)((float *)p.C + ci) = make_float4(x[0], x[1], x[2], x[3]);
            return;
        }
        if (p.c_dtype == XFTHIP_BF16 && ((((uintptr_t)p.C) | ((size_t)p.ldc * 2)) & 7) == 0) {
            const uint32_t lo = f32_to_bf16_ref(x[0]) | ((uint32_t)f32_to_bf16_ref(x[1]) << 16);
            const uint32_t hi = f32_to_bf16_ref(x[2]) | ((uint32_t)f32_to_bf16_ref(x[3]) << 16);
            *(uint2 *)((uint16_t *)p.C + ci) = make_uint2(lo, hi);
            return;
        }
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) store_from_f32(p.C, p.c_dtype, ci + v, x[v]);
}

// Partial results of the K split: one buffer per stream and device (stream_scratch), allocated once at its upper
// bound (a split launch has at most CUs / 2 tiles of 32 x 128 results in at most 16 parts: 33.5 MB on 256 CUs), so
// nothing is allocated or freed on a stream once its buffer exists.  Launches on one stream are ordered; launches
// on different streams work in different buffers.
size_t split_bound_floats() { return (size_t)16 * (device_cu_count() / 2 + 1) * 4096; }

} // namespace

int qgemm_split_reserve(hipStream_t stream, float **out) {
    void *p = nullptr;
    if (int rc = stream_scratch(kScratchGemmSplit, stream, split_bound_floats() * sizeof(float), false, &p)) return rc;
    if (out) *out = (float *)p;
    return 0;
}

int qgemm_mfma(const PackedWeight &pw, const SkinnyParams &p0, hipStream_t stream) {
    SkinnyParams p = p0;
    p.packed = pw.packed;
    p.scale = pw.scale;
    p.zero = pw.zero;
    p.KT = pw.KT;
    p.NTILES = pw.NTILES;
    p.K = pw.K;
    p.N = pw.N;
    p.ksplit = 0, p.split_ktiles = 0, p.split_part = nullptr;
    // Few rows against few columns and a deep K (the down projection of an expert, the output projection at a
    // few dozen sequences): the 32-row tiles would not even give every CU a workgroup, so K is split as well.
    const int ktile = ktile_of(pw.kind), kt_n = (pw.K + ktile - 1) / ktile;
    const int cus = device_cu_count(), n32 = (pw.NTILES + 1) / 2;
    const int rows_expected = (p.rows_dev && !p.group && p.m_hint > 0) ? p.m_hint : p.M;
    const long tiles = (long)((n32 + 3) / 4) * ((rows_expected + 31) / 32);
    if (!p.gateup && 2 * tiles <= cus && kt_n >= 16) {
        long want = (2L * cus) / tiles;
        want = want < kt_n / 8 ? want : kt_n / 8;
        want = want < 16 ? want : 16;
        if (want >= 2) {
            p.split_ktiles = (kt_n + (int)want - 1) / (int)want;
            p.ksplit = (kt_n + p.split_ktiles - 1) / p.split_ktiles;
        }
    }
    if (p.group && !p.gateup && kt_n >= 16) {
        // A group's workgroups all run side by side; K is split until there are about 8 of them a CU (measured on
        // 8 weights of 14336 x 4096 with 512 rows in all: 4 parts 497 us a layer against 523 unsplit), as far as
        // the parts fit their buffer
        const long tiles64 = (long)((n32 + 3) / 4) * ((p.M + 63) / 64 + p.group_n);
        long want = (8L * cus + tiles64 - 1) / tiles64;
        want = want < kt_n / 8 ? want : kt_n / 8;
        want = want < 16 ? want : 16;
        const long fit = (long)(split_bound_floats() / ((size_t)p.M * p.N));
        want = want < fit ? want : fit;
        p.ksplit = 0;
        if (want >= 2) {
            p.split_ktiles = (kt_n + (int)want - 1) / (int)want;
            p.ksplit = (kt_n + p.split_ktiles - 1) / p.split_ktiles;
        }
    }
    if (p.ksplit <= 1 && !p.gateup && !p.group && !p.rows_dev && p.M >= 256 && pw.K >= 8192) {
        // A few hundred rows against few columns and a very deep K (the down projection of a 512-token prompt, 4096
        // columns x 11008): 64-row tiles give every CU at most one workgroup with a k loop of 172 steps, 32-row tiles
        // (two a CU) widen every weight for a single row tile.  K is split until the 64-row tiles come two a CU:
        // 65 us with the addition of the parts against 79 (512 x 4096 x 11008).  At K = 4096 the loops are too short
        // for the split to pay (31 us either way).
        const long tiles64 = (long)((n32 + 3) / 4) * ((p.M + 63) / 64);
        if (tiles64 < 2 * cus) {
            long want = (2L * cus + tiles64 - 1) / tiles64;
            const long fit = (long)(split_bound_floats() / ((size_t)p.M * p.N));
            want = want < fit ? want : fit;
            want = want < pw.K / 2048 ? want : pw.K / 2048; // parts at least 2048 deep
            if (want >= 2) {
                p.split_ktiles = (kt_n + (int)want - 1) / (int)want;
                p.ksplit = (kt_n + p.split_ktiles - 1) / p.split_ktiles;
            }
        }
    }
    if (p.ksplit > 1) {
        if ((size_t)p.ksplit * p.M * p.N > split_bound_floats()) p.ksplit = 0; // cannot happen within the bound; stay correct anyway
        else if (int rc = qgemm_split_reserve(stream, &p.split_part)) return rc;
    }
    if (p.ksplit <= 1) p.ksplit = 0;
    int rc;
    switch (pw.kind) {
        case XFTHIP_W_INT8: rc = p.zero ? qgemm_mfma_int8z(p, stream) : qgemm_mfma_int8(p, stream); break;
        case XFTHIP_W_UINT4: rc = qgemm_mfma_uint4(p, stream); break;
        case XFTHIP_W_NF4: rc = qgemm_mfma_nf4(p, stream); break;
        case XFTHIP_W_BF16: rc = qgemm_mfma_bf16(p, stream); break;
        default: set_error("qgemm_mfma: weight kind %d not supported", pw.kind); return 2;
    }
    if (rc || p.ksplit <= 1) return rc;
    const size_t outs = (size_t)p.M * p.N;
    if (p.N % 4 == 0) // the parts are [M][N] fp32 in a 256-byte aligned buffer: 16-byte loads need only N % 4 == 0
        hipLaunchKernelGGL(qgemm_split_finish_kernel<4>, dim3((unsigned)((outs / 4 + 255) / 256)), dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(qgemm_split_finish_kernel<1>, dim3((unsigned)((outs + 255) / 256)), dim3(256), 0, stream, p);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

} // namespace xfthip
