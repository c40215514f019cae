// Parameter blocks of the persistent whole-step decode kernel (decode_mega.hip).
#pragma once
#include "kvcache.h"

namespace xfthip {

struct MegaLayer {
    const uint8_t *wqkv, *wo, *wgu, *wdown; // packed INT8 tiles
    const float *sqkv, *so, *sgu, *sdown; // per-column scales, packed column order
    int kt_qkv, kt_o, kt_gu, kt_down; // tiles along K (padded to whole batches of 4)
    const float *ln1, *ln2;
    KvView kv;
};

struct MegaParams {
    const MegaLayer *layers;
    int nlayers, M, hidden, inter, qH, kvH;
    float *x; // [M][hidden] residual stream
    uint16_t *q, *att, *h; // bf16 scratch: rotated queries, attention output, SwiGLU output
    int *pos; // [M] tokens already in the cache
    const float *cosT, *sinT;
    float rms_eps, scale;
    float *ws;
    unsigned int *tickets;
    int nsplit;
    const uint16_t *embedding; // fp16 [vocab][hidden]
    int *ids; // [M] in: token to embed, out: argmax of this step
    const float *final_norm;
    const uint8_t *lm_head; // packed BF16 tiles
    int kt_lm, vocab;
    float *logits;
    int *idlog; // [steps][M]
    int *step;
    int act_pitch; // LDS activation row pitch (elements): max K of any phase + 8
    int red_off; // byte offset of the K-slice partial sums behind the activation rows
    unsigned int *counter; // [0] global arrivals, [64 * (1 + g)] arrivals of the workgroups with blockIdx % 8 == g
    int *abort_flag;
    unsigned int spin_limit;
    unsigned long long *trace; // optional: [0] kernel start, [i] time workgroup 0 left barrier i (100 MHz ticks)
    int trace_cap;
};

// occupancy of the kernel (workgroups per compute unit) and its launch (preceded by the counter reset)
size_t mega_lds_bytes(int M, int act_pitch);
int mega_decode_max_blocks(int *blocks_per_cu, size_t lds_bytes);
int mega_decode_launch(const MegaParams &p, int grid, size_t lds_bytes, hipStream_t stream);

} // namespace xfthip
