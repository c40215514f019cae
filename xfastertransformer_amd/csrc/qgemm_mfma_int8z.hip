// Instantiations of the M > 32 weight-only GEMM for INT8 with zero points weights.
#include "qgemm_mfma_impl.h"

namespace xfthip {

int qgemm_mfma_int8z(const SkinnyParams &p, hipStream_t stream) {
    return dispatch_big_tile<XFTHIP_W_INT8, true>(p, stream);
}

} // namespace xfthip
