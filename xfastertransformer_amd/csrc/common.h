// Shared declarations of the gfx950 library: error plumbing, element types, the packed
// weight descriptor and small device helpers.  Internal header (the public C-ABI is
// include/xft_hip.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string>

#include "../../include/xft_hip.h"
#include "bf16_convert.h"

namespace xfthip {

void set_error(const char *fmt, ...);

#define XFT_CHECK_HIP(expr)                                                                         \
    do {                                                                                            \
        hipError_t _e = (expr);                                                                     \
        if (_e != hipSuccess) {                                                                     \
            xfthip::set_error("%s:%d: %s failed: %s", __FILE__, __LINE__, #expr, hipGetErrorString(_e)); \
            return 1;                                                                               \
        }                                                                                           \
    } while (0)

#define XFT_REQUIRE(cond, ...)               \
    do {                                     \
        if (!(cond)) {                       \
            xfthip::set_error(__VA_ARGS__);  \
            return 2;                        \
        }                                    \
    } while (0)

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

// ---- packed weight layout ---------------------------------------------------------------
// The matrix is cut into tiles of 16 output columns (n) by KTILE input rows (k); a tile is
// 1 KiB = 64 lanes x 16 bytes, laid out so that lane l of a wavefront reads bytes
// [16 l, 16 l + 16) and finds there the K-consecutive codes of column n = 16 nt + (l & 15)
// for the k range its MFMA operand slot needs (lane group g = l >> 4):
//   INT8 / W8A8 : KTILE 64,  16 codes/lane, k = 64 kt + 16 g + j
//   UINT4 / NF4 : KTILE 128, 32 codes/lane, k = 128 kt + 32 g + c, code c = 8 d + e lives in
//                 dword d at nibble e/2 (e even) or 4 + e/2 (e odd), so that
//                 ((w >> 4p) & 0x000F000F) yields the pair (e = 2p, e = 2p + 1)
//   BF16        : KTILE 32,  8 values/lane, k = 32 kt + 8 g + j
// Tiles of one column block are contiguous along k: offset = (nt * KT + kt) * 1024 bytes.
struct PackedWeight {
    int kind;
    int K, N; // logical shape
    int KT, NTILES; // tiles along k and n
    int ktile; // rows per tile
    int flags;
    int inter; // XFTHIP_WF_GATEUP: I (half of N); columns are stored gate/up interleaved per 16
    uint8_t *packed; // device
    float *scale; // device [NTILES*16], in packed column order
    float *zero; // device or nullptr
    float *colsum; // device (W8A8) or nullptr
    size_t packed_bytes;
};

__host__ __device__ inline int ktile_of(int kind) {
    return (kind == XFTHIP_W_INT8 || kind == XFTHIP_W_W8A8) ? 64 : (kind == XFTHIP_W_BF16 ? 32 : 128);
}

// logical column -> packed column
__host__ __device__ inline int packed_col(int n, int inter) {
    if (inter <= 0) return n;
    int isUp = n >= inter;
    int j = isUp ? n - inter : n;
    return (j >> 4) * 32 + (isUp ? 16 : 0) + (j & 15);
}
// packed column -> logical column
__host__ __device__ inline int logical_col(int np, int inter) {
    if (inter <= 0) return np;
    int blk = np >> 5, r = np & 31;
    int j = blk * 16 + (r & 15);
    return (r >= 16) ? j + inter : j;
}

// NormalFloat4 code values (QLoRA, Dettmers et al. 2023, appendix E): the one copy the device tables of the
// pack / unpack kernels and of both GEMM kernels are initialised from
#define XFTHIP_NF4_CODE_VALUES                                                                              \
    {-1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f, -0.28444138169288635f,       \
            -0.18477343022823334f, -0.09105003625154495f, 0.0f, 0.07958029955625534f, 0.16093020141124725f, \
            0.24611230194568634f, 0.33791524171829224f, 0.44070982933044434f, 0.5626170039176941f,          \
            0.7229568362236023f, 1.0f}

// ---- numeric helpers -----------------------------------------------------------------
__device__ inline uint32_t f2u(float f) { return __float_as_uint(f); }
__device__ inline float u2f(uint32_t u) { return __uint_as_float(u); }

// fp32 -> bf16 exactly as the reference's bfloat16_t assignment (bf16_convert.h)
__device__ inline uint16_t f32_to_bf16_ref(float f) { return f32_bits_to_bf16_ref(f2u(f)); }
__device__ inline float bf16_to_f32(uint16_t b) { return u2f((uint32_t)b << 16); }

__device__ inline uint16_t f32_to_fp16_bits(float f) {
    _Float16 h = (_Float16)f; // v_cvt_f16_f32: IEEE round-to-nearest-even
    return __builtin_bit_cast(uint16_t, h);
}
__device__ inline float fp16_bits_to_f32(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }

__device__ inline float load_as_f32(const void *p, int dtype, size_t idx) {
    if (dtype == XFTHIP_F32) return ((const float *)p)[idx];
    if (dtype == XFTHIP_BF16) return bf16_to_f32(((const uint16_t *)p)[idx]);
    return fp16_bits_to_f32(((const uint16_t *)p)[idx]);
}
__device__ inline void store_from_f32(void *p, int dtype, size_t idx, float v) {
    if (dtype == XFTHIP_F32)
        ((float *)p)[idx] = v;
    else if (dtype == XFTHIP_BF16)
        ((uint16_t *)p)[idx] = f32_to_bf16_ref(v);
    else
        ((uint16_t *)p)[idx] = f32_to_fp16_bits(v);
}

// Loads and stores that are coherent across the chip's XCDs without cache maintenance.  Each
// XCD has its own L2; ordinary accesses only become visible to another XCD after an L2
// write-back on one side and an invalidate on the other.  Relaxed atomics at device scope go
// past the non-coherent lines instead, which is what workgroups of ONE kernel need when they
// hand small amounts of data to each other.  dev_drain() waits until this wave's stores have
// been acknowledged; follow it by a block barrier before signalling other workgroups.
__device__ inline float ld_dev(const float *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ inline int ld_dev(const int *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ inline uint32_t ld_dev(const uint32_t *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ inline unsigned long long ld_dev(const unsigned long long *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline void st_dev(float *p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ inline void st_dev(uint32_t *p, uint32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ inline void st_dev(uint16_t *p, uint16_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// 16 bytes (8 bf16 / fp16 values) from a 16-byte aligned address
__device__ inline void ld_dev16(const void *p, uint32_t (&out)[4]) {
    const unsigned long long a = ld_dev((const unsigned long long *)p), b = ld_dev((const unsigned long long *)p + 1);
    out[0] = (uint32_t)a, out[1] = (uint32_t)(a >> 32), out[2] = (uint32_t)b, out[3] = (uint32_t)(b >> 32);
}
__device__ inline void dev_drain() {
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): every load returned, every store acknowledged
}

// exp on the device: the reference uses a degree-5 polynomial (src/utils/bert_util.h:26-75)
// accurate to ~1e-7 relative; __expf is within the same distance of exp().
__device__ inline float fast_exp(float x) { return __expf(x); }

int device_cu_count();
// Scratch memory of the stand-alone entry points: one buffer per (purpose, device, stream), so that calls on different
// streams never share one (calls on one stream are ordered).  Returns a buffer of at least `bytes`; a buffer that has
// to grow is replaced (which waits for the device).  Allocates on first use for a stream: not during a stream capture
// (xfthip_graph_begin reserves what the recordable entry points need; a caller that captures by itself makes one
// eager call on that stream first).  zero_new: a new buffer starts cleared.
enum ScratchPurpose {
    kScratchGemmSplit, // fp32 parts of a K-split weight-only GEMM
    kScratchAttnParts, // split-KV partial results of xfthip_attention
    kScratchAttnTickets,
    kScratchW8a8Codes, // quantised activation rows of xfthip_gemm_w8a8_from_bf16
    kScratchW8a8Stats,
    kScratchPagedParts, // context splits of xfthip_paged_attention_decode
    kScratchPagedQkv, // fused q|k|v rows of xfthip_paged_attention_prefill
    kScratchPurposes
};
int stream_scratch(ScratchPurpose purpose, hipStream_t stream, size_t bytes, bool zero_new, void **out);
// While one of these lives, the calling thread's stream_scratch calls take the buffers of `key` whatever stream they
// name: for work recorded on a capture stream of the library's own that will be launched on `key`.
struct ScratchKeyScope {
    explicit ScratchKeyScope(hipStream_t key);
    ~ScratchKeyScope();
    ScratchKeyScope(const ScratchKeyScope &) = delete;
    ScratchKeyScope &operator=(const ScratchKeyScope &) = delete;
};
// Split-KV merge workspace of the attention kernel: partial (max, sum, output) slots and one
// ticket per column group (tickets are zero between launches).
struct AttnWorkspace {
    float *ws = nullptr;
    unsigned int *tickets = nullptr;
    int slots = 0;
};
int attention_workspace_create(AttnWorkspace *w, int slots); // allocates; not for use during stream capture
void attention_workspace_destroy(AttnWorkspace *w);
// resolves the device address of the statically allocated workspace behind xfthip_attention_static
// for the current device (idempotent, allocates nothing)
int attention_static_scratch_init();
// the attention launch behind xfthip_attention, with a length hint for callers whose positions live
// in device memory, the workspace to use (nullptr = the shared one) and whether a workspace that is
// too small is an error (otherwise the split count is lowered to fit)
int attention_launch(xfthip_kvcache_t c, const void *q, int qStride, void *out, int oStride, int out_dtype, int B, int S,
        int qHeads, float scale, int past, const int *past_dev, int len_hint, hipStream_t stream, const AttnWorkspace *wsp = nullptr,
        bool strict = false);
// the split count the launch picks for `units` (batch x kv head x column group) workgroups
int attention_split_count(int len, int units);

} // namespace xfthip

struct xfthip_weight {
    xfthip::PackedWeight pw;
};
