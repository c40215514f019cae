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

} // extern "C"
