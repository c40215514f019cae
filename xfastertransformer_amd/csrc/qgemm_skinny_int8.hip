// Instantiations of the M <= 32 weight-only GEMM for INT8 weights.
#include "qgemm_skinny_impl.h"

namespace xfthip {

int qgemm_skinny_int8(const SkinnyParams &p, hipStream_t stream) {
    return dispatch_shape<XFTHIP_W_INT8>(p, stream);
}

} // namespace xfthip
