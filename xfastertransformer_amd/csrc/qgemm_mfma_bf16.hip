// Instantiations of the M > 32 weight-only GEMM for BF16 weights.
#include "qgemm_mfma_impl.h"

namespace xfthip {

int qgemm_mfma_bf16(const SkinnyParams &p, hipStream_t stream) {
    return dispatch_big_tile<XFTHIP_W_BF16, false>(p, stream);
}

} // namespace xfthip
