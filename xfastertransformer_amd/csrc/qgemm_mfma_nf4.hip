// Instantiations of the M > 32 weight-only GEMM for NF4 weights.
#include "qgemm_mfma_impl.h"

namespace xfthip {

int qgemm_mfma_nf4(const SkinnyParams &p, hipStream_t stream) {
    return dispatch_big_tile<XFTHIP_W_NF4, false>(p, stream);
}

} // namespace xfthip
