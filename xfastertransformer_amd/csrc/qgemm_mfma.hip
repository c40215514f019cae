// Dequant-fused weight-only GEMM for many activation rows (M > 32): the prefill shape.
// Replaces MMHelper::compute* (reference src/utils/matmul_helper.h:565-1705) at large M, where
// the reference switches to AMX (oneDNN) kernels.  The kernel lives in qgemm_mfma_impl.h; this
// file picks the weight kind.
#include "qgemm.h"

namespace xfthip {

int qgemm_mfma_int8(const SkinnyParams &p, hipStream_t stream);
int qgemm_mfma_int8z(const SkinnyParams &p, hipStream_t stream);
int qgemm_mfma_uint4(const SkinnyParams &p, hipStream_t stream);
int qgemm_mfma_nf4(const SkinnyParams &p, hipStream_t stream);
int qgemm_mfma_bf16(const SkinnyParams &p, hipStream_t stream);

int qgemm_mfma(const PackedWeight &pw, const SkinnyParams &p0, hipStream_t stream) {
    SkinnyParams p = p0;
    p.packed = pw.packed;
    p.scale = pw.scale;
    p.zero = pw.zero;
    p.KT = pw.KT;
    p.NTILES = pw.NTILES;
    p.K = pw.K;
    p.N = pw.N;
    switch (pw.kind) {
        case XFTHIP_W_INT8:
            if (p.zero) return qgemm_mfma_int8z(p, stream);
            return qgemm_mfma_int8(p, stream);
        case XFTHIP_W_UINT4: return qgemm_mfma_uint4(p, stream);
        case XFTHIP_W_NF4: return qgemm_mfma_nf4(p, stream);
        case XFTHIP_W_BF16: return qgemm_mfma_bf16(p, stream);
        default: set_error("qgemm_mfma: weight kind %d not supported", pw.kind); return 2;
    }
}

} // namespace xfthip
