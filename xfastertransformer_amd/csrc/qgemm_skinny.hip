// Dequant-fused weight-only GEMM for few activation rows (M <= 32): the decode-time shape.
// Replaces MMHelper::compute* (reference src/utils/matmul_helper.h:565-1705) for
// INT8 / UINT4 / NF4 / BF16 weights against bf16 activations.  The kernel lives in
// qgemm_skinny_impl.h; this file checks the fused options and picks the weight kind.
#include "qgemm.h"

namespace xfthip {

int qgemm_skinny_int8(const SkinnyParams &p, hipStream_t stream);
int qgemm_skinny_uint4(const SkinnyParams &p, hipStream_t stream);
int qgemm_skinny_nf4(const SkinnyParams &p, hipStream_t stream);
int qgemm_skinny_bf16(const SkinnyParams &p, hipStream_t stream);

// LDS of the RMSNorm prologue: M rows of K + 8 bf16 values
static inline size_t skinny_norm_lds_bytes(int M, int K) {
    return (size_t)M * (K + 8) * 2;
}

bool skinny_can_fuse_norm(const PackedWeight &pw, int M) {
    return M <= 4 && pw.kind != XFTHIP_W_W8A8 && pw.KT * ktile_of(pw.kind) == pw.K && pw.K % 4 == 0
            && skinny_norm_lds_bytes(M, pw.K) <= (size_t)36 * 1024;
}

int qgemm_skinny(const PackedWeight &pw, const SkinnyParams &p0, hipStream_t stream) {
    SkinnyParams p = p0;
    if (p.group && (p.norm_x || p.rope || !p.rows_dev || pw.KT * ktile_of(pw.kind) != pw.K)) {
        set_error("qgemm_skinny: a group of weights needs device row records and K a whole number of weight tiles, and takes no norm "
                  "prologue or RoPE epilogue");
        return 2;
    }
    if (p.norm_x && !skinny_can_fuse_norm(pw, p.M)) {
        set_error("qgemm_skinny: RMSNorm prologue not available for M=%d K=%d kind=%d", p.M, pw.K, pw.kind);
        return 2;
    }
    if (p.rope && (p.M > 32 || p.M > p.kv.B || p.kvH != p.kv.H || p.gateup || (p.qH + 2 * p.kvH) * 128 != pw.N || p.kv.int8 != 0 || p.kv.D != 128
                || (p.M > 16 && p.norm_x))) {
        set_error("qgemm_skinny: RoPE / cache-append epilogue needs M <= 32 rows (one per cache row), head size 128, an FP16 cache and a "
                  "[K, (q+2kv)*128] weight");
        return 2;
    }
    p.packed = pw.packed;
    p.scale = pw.scale;
    p.zero = pw.zero;
    p.KT = pw.KT;
    p.NTILES = pw.NTILES;
    p.K = pw.K;
    p.N = pw.N;
    switch (pw.kind) {
        case XFTHIP_W_INT8: return qgemm_skinny_int8(p, stream);
        case XFTHIP_W_UINT4: return qgemm_skinny_uint4(p, stream);
        case XFTHIP_W_NF4: return qgemm_skinny_nf4(p, stream);
        case XFTHIP_W_BF16: return qgemm_skinny_bf16(p, stream);
        default: set_error("qgemm_skinny: weight kind %d not supported", pw.kind); return 2;
    }
}

} // namespace xfthip
