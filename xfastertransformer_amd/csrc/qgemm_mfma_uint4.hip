// Instantiations of the M > 32 weight-only GEMM for UINT4 weights.
#include "qgemm_mfma_impl.h"

namespace xfthip {

int qgemm_mfma_uint4(const SkinnyParams &p, hipStream_t stream) {
    return dispatch_big_tile<XFTHIP_W_UINT4, true>(p, stream);
}

} // namespace xfthip
