// C-ABI entry points of the weight-only GEMM: argument checks and kernel selection.
#include "qgemm.h"


using namespace xfthip;

static int check_common(const char *fn, xfthip_weight_t w, int M, const void *A, int lda, void *C, int ldc) {
    XFT_REQUIRE(w != nullptr && A != nullptr && C != nullptr, "%s: null argument", fn);
    XFT_REQUIRE(M > 0, "%s: M=%d must be positive", fn, M);
    XFT_REQUIRE(lda >= w->pw.K && (lda % 8) == 0, "%s: lda=%d must be >= K=%d and a multiple of 8", fn, lda, w->pw.K);
    XFT_REQUIRE(((uintptr_t)A & 15) == 0, "%s: A must be 16-byte aligned", fn);
    (void)ldc;
    return 0;
}

namespace xfthip {

int gemm_rows_dev(xfthip_weight_t w, int m_max, int m_hint, const int *rows_dev, const void *A, int lda, void *C, int ldc, int c_dtype,
        hipStream_t stream) {
    if (int rc = check_common("gemm_rows_dev", w, m_max, A, lda, C, ldc)) return rc;
    const PackedWeight &pw = w->pw;
    XFT_REQUIRE(rows_dev != nullptr && pw.kind != XFTHIP_W_W8A8, "gemm_rows_dev: needs a device row record and a weight-only kind");
    XFT_REQUIRE(c_dtype == XFTHIP_F32 || c_dtype == XFTHIP_BF16, "gemm_rows_dev: c_dtype must be f32 or bf16");
    const int gateup = (pw.flags & XFTHIP_WF_GATEUP) ? 1 : 0;
    XFT_REQUIRE(ldc >= (gateup ? pw.N / 2 : pw.N), "gemm_rows_dev: ldc=%d too small", ldc);
    SkinnyParams p = {};
    p.M = m_max;
    p.A = (const uint16_t *)A;
    p.lda = lda;
    p.C = C;
    p.ldc = ldc;
    p.c_dtype = c_dtype;
    p.epi = XFTHIP_EPI_NONE;
    p.gateup = gateup;
    p.rows_dev = rows_dev;
    p.m_hint = m_hint;
    if (m_max <= 32) return qgemm_skinny(pw, p, stream);
    return qgemm_mfma(pw, p, stream);
}

int gemm_grouped_rows_dev(const xfthip_weight_t *w, int n_group, const GroupWeight *table_dev, int rows_max, int rows_each_max,
        const int *rows_dev, int rows_stride, const void *A, int lda, void *C, int ldc, int c_dtype, hipStream_t stream) {
    XFT_REQUIRE(w && n_group >= 1 && table_dev && rows_dev && rows_stride >= 3, "gemm_grouped_rows_dev: bad group arguments");
    if (int rc = check_common("gemm_grouped_rows_dev", w[0], rows_max, A, lda, C, ldc)) return rc;
    XFT_REQUIRE(rows_each_max >= 1 && rows_each_max <= rows_max, "gemm_grouped_rows_dev: bad row bounds %d / %d", rows_each_max, rows_max);
    const PackedWeight &pw = w[0]->pw;
    XFT_REQUIRE(pw.kind != XFTHIP_W_W8A8, "gemm_grouped_rows_dev: needs a weight-only kind");
    for (int e = 1; e < n_group; ++e) {
        XFT_REQUIRE(w[e] != nullptr, "gemm_grouped_rows_dev: weight %d is null", e);
        const PackedWeight &o = w[e]->pw;
        XFT_REQUIRE(o.kind == pw.kind && o.K == pw.K && o.N == pw.N && o.flags == pw.flags && (o.zero != nullptr) == (pw.zero != nullptr),
                "gemm_grouped_rows_dev: weight %d differs from weight 0 in kind, shape or layout", e);
    }
    XFT_REQUIRE(c_dtype == XFTHIP_F32 || c_dtype == XFTHIP_BF16, "gemm_grouped_rows_dev: c_dtype must be f32 or bf16");
    const int gateup = (pw.flags & XFTHIP_WF_GATEUP) ? 1 : 0;
    XFT_REQUIRE(ldc >= (gateup ? pw.N / 2 : pw.N), "gemm_grouped_rows_dev: ldc=%d too small", ldc);
    SkinnyParams p = {};
    p.M = rows_max;
    p.A = (const uint16_t *)A;
    p.lda = lda;
    p.C = C;
    p.ldc = ldc;
    p.c_dtype = c_dtype;
    p.epi = XFTHIP_EPI_NONE;
    p.gateup = gateup;
    p.rows_dev = rows_dev;
    p.group = table_dev;
    p.group_n = n_group;
    p.rows_stride = rows_stride;
    if (rows_each_max <= 32) {
        XFT_REQUIRE(pw.KT * ktile_of(pw.kind) == pw.K, "gemm_grouped_rows_dev: the few-row form needs K = %d to be a whole number of %d-row weight tiles",
                pw.K, ktile_of(pw.kind));
        p.M = rows_each_max; // the few-row kernel: a grid row a weight, each with at most this many rows
        return qgemm_skinny(pw, p, stream);
    }
    return qgemm_mfma(pw, p, stream);
}

} // namespace xfthip

extern "C" {

int xfthip_gemm(xfthip_weight_t w, int M, const void *A, int lda, void *C, int ldc, int c_dtype, int epilogue,
        const float *bias, const void *res, int ldres, int res_dtype, float gamma, xfthip_stream_t stream) {
    if (int rc = check_common("xfthip_gemm", w, M, A, lda, C, ldc)) return rc;
    const PackedWeight &pw = w->pw;
    XFT_REQUIRE(ldc >= pw.N, "xfthip_gemm: ldc=%d < N=%d", ldc, pw.N);
    XFT_REQUIRE(c_dtype == XFTHIP_F32 || c_dtype == XFTHIP_BF16, "xfthip_gemm: c_dtype must be f32 or bf16");
    XFT_REQUIRE(epilogue >= XFTHIP_EPI_NONE && epilogue <= XFTHIP_EPI_RESEXT, "xfthip_gemm: unknown epilogue %d", epilogue);
    XFT_REQUIRE(epilogue != XFTHIP_EPI_BIAS || bias != nullptr, "xfthip_gemm: bias epilogue without bias");
    const bool needs_res = epilogue == XFTHIP_EPI_RESMUL || epilogue == XFTHIP_EPI_RESIDENTIAL || epilogue == XFTHIP_EPI_RESEXT;
    XFT_REQUIRE(!needs_res || (res != nullptr && ldres >= pw.N), "xfthip_gemm: epilogue %d needs res with ldres >= N", epilogue);
    XFT_REQUIRE(!needs_res || (res_dtype >= XFTHIP_F32 && res_dtype <= XFTHIP_FP16), "xfthip_gemm: bad res_dtype %d", res_dtype);
    XFT_REQUIRE(!(pw.flags & XFTHIP_WF_GATEUP), "xfthip_gemm: weight was packed for xfthip_gemm_gateup_silu");
    if (pw.kind == XFTHIP_W_W8A8)
        return gemm_w8a8_from_bf16(w, M, A, lda, C, ldc, c_dtype, epilogue, bias, res, ldres, res_dtype, gamma, (hipStream_t)stream);

    SkinnyParams p = {};
    p.M = M;
    p.A = (const uint16_t *)A;
    p.lda = lda;
    p.C = C;
    p.ldc = ldc;
    p.c_dtype = c_dtype;
    p.epi = epilogue;
    p.bias = bias;
    p.res = res;
    p.ldres = ldres;
    p.res_dtype = res_dtype;
    p.gamma = gamma;
    p.gateup = 0;
    if (M <= 32) return qgemm_skinny(pw, p, (hipStream_t)stream);
    return qgemm_mfma(pw, p, (hipStream_t)stream);
}

int xfthip_gemm_gateup_silu(xfthip_weight_t w, int M, const void *A, int lda, void *out, int ldo, int out_dtype,
        xfthip_stream_t stream) {
    if (int rc = check_common("xfthip_gemm_gateup_silu", w, M, A, lda, out, ldo)) return rc;
    const PackedWeight &pw = w->pw;
    XFT_REQUIRE(pw.flags & XFTHIP_WF_GATEUP, "xfthip_gemm_gateup_silu: weight was not created with XFTHIP_WF_GATEUP");
    XFT_REQUIRE(ldo >= pw.N / 2, "xfthip_gemm_gateup_silu: ldo=%d < I=%d", ldo, pw.N / 2);
    XFT_REQUIRE(out_dtype == XFTHIP_F32 || out_dtype == XFTHIP_BF16, "xfthip_gemm_gateup_silu: out_dtype must be f32 or bf16");
    XFT_REQUIRE(pw.kind != XFTHIP_W_W8A8, "xfthip_gemm_gateup_silu: W8A8 weights take the unfused path (xfthip_gemm + SwiGLU)");
    SkinnyParams p = {};
    p.M = M;
    p.A = (const uint16_t *)A;
    p.lda = lda;
    p.C = out;
    p.ldc = ldo;
    p.c_dtype = out_dtype;
    p.gateup = 1;
    if (M <= 32) return qgemm_skinny(pw, p, (hipStream_t)stream);
    return qgemm_mfma(pw, p, (hipStream_t)stream);
}

int xfthip_gemm_gateup_silu_rmsnorm(xfthip_weight_t w, int M, const float *x, int ldx, const float *norm_weight, float eps,
        void *out, int ldo, int out_dtype, xfthip_stream_t stream) {
    XFT_REQUIRE(w && x && norm_weight && out, "xfthip_gemm_gateup_silu_rmsnorm: null argument");
    const PackedWeight &pw = w->pw;
    XFT_REQUIRE(pw.flags & XFTHIP_WF_GATEUP, "xfthip_gemm_gateup_silu_rmsnorm: weight was not created with XFTHIP_WF_GATEUP");
    XFT_REQUIRE(M > 0 && skinny_can_fuse_norm(pw, M),
            "xfthip_gemm_gateup_silu_rmsnorm: needs 1 <= M <= 4, K a whole number of weight tiles and M rows of K in 36 KB of LDS (M=%d K=%d)",
            M, pw.K);
    XFT_REQUIRE(ldx >= pw.K && ldx % 4 == 0 && ((uintptr_t)x & 15) == 0, "xfthip_gemm_gateup_silu_rmsnorm: x rows must be 16-byte aligned, ldx >= K");
    XFT_REQUIRE(ldo >= pw.N / 2, "xfthip_gemm_gateup_silu_rmsnorm: ldo=%d < I=%d", ldo, pw.N / 2);
    XFT_REQUIRE(out_dtype == XFTHIP_F32 || out_dtype == XFTHIP_BF16, "xfthip_gemm_gateup_silu_rmsnorm: out_dtype must be f32 or bf16");
    SkinnyParams p = {};
    p.M = M;
    p.C = out;
    p.ldc = ldo;
    p.c_dtype = out_dtype;
    p.gateup = 1;
    p.norm_x = x, p.ldx = ldx, p.norm_w = norm_weight, p.norm_eps = eps;
    return qgemm_skinny(pw, p, (hipStream_t)stream);
}

int xfthip_gemm_qkv_rmsnorm_rope(xfthip_weight_t w, xfthip_kvcache_t cache, int M, const float *x, int ldx, const float *norm_weight,
        float eps, void *q_out, int ldq, int q_heads, const float *cos_table, const float *sin_table, int position,
        const int *position_dev, xfthip_stream_t stream) {
    XFT_REQUIRE(w && cache && x && norm_weight && q_out && cos_table && sin_table, "xfthip_gemm_qkv_rmsnorm_rope: null argument");
    const PackedWeight &pw = w->pw;
    const KvView &kv = cache->kv;
    XFT_REQUIRE(!(pw.flags & XFTHIP_WF_GATEUP) && pw.kind != XFTHIP_W_W8A8, "xfthip_gemm_qkv_rmsnorm_rope: unsupported weight");
    XFT_REQUIRE(M > 0 && M <= kv.B && skinny_can_fuse_norm(pw, M),
            "xfthip_gemm_qkv_rmsnorm_rope: needs 1 <= M <= min(4, cache batch) and K a whole number of weight tiles (M=%d K=%d)", M, pw.K);
    XFT_REQUIRE(!kv.int8 && kv.D == 128, "xfthip_gemm_qkv_rmsnorm_rope: needs an FP16 cache with head size 128");
    XFT_REQUIRE(q_heads > 0 && (q_heads + 2 * kv.H) * 128 == pw.N, "xfthip_gemm_qkv_rmsnorm_rope: weight has %d columns, expected (%d + 2 * %d) * 128",
            pw.N, q_heads, kv.H);
    XFT_REQUIRE(ldx >= pw.K && ldx % 4 == 0 && ((uintptr_t)x & 15) == 0, "xfthip_gemm_qkv_rmsnorm_rope: x rows must be 16-byte aligned, ldx >= K");
    XFT_REQUIRE(ldq >= q_heads * 128, "xfthip_gemm_qkv_rmsnorm_rope: ldq=%d < %d", ldq, q_heads * 128);
    XFT_REQUIRE(position_dev != nullptr || (position >= 0 && position < cache->maxSeq),
            "xfthip_gemm_qkv_rmsnorm_rope: position %d outside the cache (max_seq %d)", position, cache->maxSeq);
    SkinnyParams p = {};
    p.M = M;
    p.C = q_out;
    p.ldc = ldq;
    p.c_dtype = XFTHIP_BF16;
    p.norm_x = x, p.ldx = ldx, p.norm_w = norm_weight, p.norm_eps = eps;
    p.rope = 1, p.cosT = cos_table, p.sinT = sin_table, p.pos_dev = position_dev, p.pos_host = position;
    p.qH = q_heads, p.kvH = kv.H, p.kv = kv;
    return qgemm_skinny(pw, p, (hipStream_t)stream);
}

} // extern "C"
