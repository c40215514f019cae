// Instantiations of the M <= 32 weight-only GEMM for NF4 weights.
#include "qgemm_skinny_impl.h"

namespace xfthip {

int qgemm_skinny_nf4(const SkinnyParams &p, hipStream_t stream) {
    return dispatch_shape<XFTHIP_W_NF4>(p, stream);
}

} // namespace xfthip
