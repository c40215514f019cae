// Private device layout of one layer's KV cache.
#pragma once
#include "common.h"

struct xfthip_kvcache;

namespace xfthip {

// keys   : [B][H][S][D]                 (S = maxSeq rounded up to 32)
// values : [B][H][S/32][D][32 slots]    token t of a block sits in slot v_slot(t & 31)
// scales : [B][H][S] fp32 (INT8 only), one per (token, head) for keys and for values
// The value block is the transposed tile an MFMA "A" operand wants (token index contiguous);
// the slot permutation makes the 8 tokens one lane group multiplies (4g..4g+3 and
// 16+4g..16+4g+3, the rows it holds of two 16-token score tiles) adjacent: 16 bytes (fp16)
// or 8 bytes (int8) per lane.
struct KvView {
    int int8;
    int B, H, S, D;
    void *k, *v;
    float *kscale, *vscale;
};

__host__ __device__ inline int v_slot(int t) {
    // t = 16a + 4g + r  ->  8g + 4a + r
    return ((t >> 2) & 3) * 8 + (t >> 4) * 4 + (t & 3);
}

} // namespace xfthip

namespace xfthip {
// xfthip_rope_kvstore with the option of leaving the query block alone (a second append of the
// same rows into another cache must not rotate q twice)
int rope_kvstore_impl(xfthip_kvcache *c, void *qkv, int dtype, int stride, int B, int S, int qHeads, const float *embCos,
        const float *embSin, int past, const int *past_dev, bool rotate_q, hipStream_t stream);
} // namespace xfthip

struct xfthip_kvcache {
    xfthip::KvView kv;
    int maxSeq; // as requested by the caller
};
