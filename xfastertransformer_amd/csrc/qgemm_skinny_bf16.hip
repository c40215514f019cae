// Instantiations of the M <= 32 weight-only GEMM for BF16 weights.
#include "qgemm_skinny_impl.h"

namespace xfthip {

int qgemm_skinny_bf16(const SkinnyParams &p, hipStream_t stream) {
    return dispatch_shape<XFTHIP_W_BF16>(p, stream);
}

} // namespace xfthip
