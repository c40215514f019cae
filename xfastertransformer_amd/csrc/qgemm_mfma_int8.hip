// Instantiations of the M > 32 weight-only GEMM for symmetric INT8 weights.
#include "qgemm_mfma_impl.h"

namespace xfthip {

int qgemm_mfma_int8(const SkinnyParams &p, hipStream_t stream) {
    return dispatch_big_tile<XFTHIP_W_INT8, false>(p, stream);
}

} // namespace xfthip
