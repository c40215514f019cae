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

// One thread per output value: the K parts are added in order (the same result on every run), then the
// epilogue of the call.  p.C / p.ldc / p.c_dtype / p.epi are the caller's.
__global__ __launch_bounds__(256) void qgemm_split_finish_kernel(SkinnyParams p) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)p.M * p.N) return;
    const int m = (int)(idx / p.N), n = (int)(idx - (size_t)m * p.N);
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
    float x = 0.0f;
    for (int s = 0; s < p.ksplit; ++s) x += p.split_part[((size_t)s * p.M + m) * p.N + n];
    switch (p.epi) {
        case XFTHIP_EPI_BIAS: x += p.bias[n]; break;
        case XFTHIP_EPI_SILU: x = silu_split(x); break;
        case XFTHIP_EPI_GELU: {
            const float e = fast_exp(1.702f * x);
            x = e / (e + 1.0f) * x;
            break;
        }
        case XFTHIP_EPI_RESMUL: x *= load_as_f32(p.res, p.res_dtype, (size_t)m * p.ldres + n); break;
        case XFTHIP_EPI_RESIDENTIAL:
            if (p.bias) x += p.bias[n];
            x += load_as_f32(p.res, p.res_dtype, (size_t)m * p.ldres + n);
            break;
        case XFTHIP_EPI_RESEXT:
            if (p.bias) x += p.bias[n];
            x = fmaf(p.gamma, load_as_f32(p.res, p.res_dtype, (size_t)m * p.ldres + n), x);
            break;
        default: break;
    }
    store_from_f32(p.C, p.c_dtype, (size_t)row_out * p.ldc + n, x);
}

// Partial results of the K split: one buffer per process and device, allocated once at its upper bound (a
// split launch has at most CUs / 2 tiles of 32 x 128 results in at most 16 parts: 33.5 MB on 256 CUs), so
// nothing is allocated or freed once it exists.  Launches on one stream are ordered; split launches that
// overlap on different streams race on it.
std::mutex g_split_mu;
float *g_split_part = nullptr;
size_t g_split_floats = 0;

} // namespace

int qgemm_split_reserve() {
    std::lock_guard<std::mutex> lk(g_split_mu);
    if (g_split_part) return 0;
    const size_t floats = (size_t)16 * (device_cu_count() / 2 + 1) * 4096;
    XFT_CHECK_HIP(hipMalloc((void **)&g_split_part, floats * sizeof(float)));
    g_split_floats = floats;
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
        if (int rc = qgemm_split_reserve()) return rc;
        const long fit = (long)(g_split_floats / ((size_t)p.M * p.N));
        want = want < fit ? want : fit;
        p.ksplit = 0;
        if (want >= 2) {
            p.split_ktiles = (kt_n + (int)want - 1) / (int)want;
            p.ksplit = (kt_n + p.split_ktiles - 1) / p.split_ktiles;
        }
    }
    if (p.ksplit > 1) {
        if (int rc = qgemm_split_reserve()) return rc;
        if ((size_t)p.ksplit * p.M * p.N > g_split_floats) p.ksplit = 0; // cannot happen within the bound; stay correct anyway
        p.split_part = g_split_part;
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
    hipLaunchKernelGGL(qgemm_split_finish_kernel, dim3((unsigned)((outs + 255) / 256)), dim3(256), 0, stream, p);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

} // namespace xfthip
