// Causal GQA attention over the KV cache: decode (one new token), prefill and chunked
// prefill in one kernel.  Replaces the reference's crossAttnByHead / crossAttnShardedHead /
// selfScaledDpAttention (src/kernels/attention_kernels.h) and their small_gemm* helpers.
//
// Work decomposition.  The "columns" of a workgroup are up to 16 (query token, query head)
// pairs that share one KV head (for decode: the G heads of a GQA group).  Keys and values
// stream from HBM exactly once per column group:
//   S^T[token][col] = K[token][:] . Q[col][:]        MFMA 16x16x32 f16, A = K tile (16 tokens
//                                                     x 32 dims, one 128-bit load per lane)
//   O^T[dim][col]  += V^T[dim][token] . P^T[token][col]   A = V tile from the token-innermost
//                                                     value layout, B = probabilities straight
//                                                     from the score registers
// Scores, running max / sum and the output accumulate in fp32 (online softmax).  The KV
// sequence is split over gridDim.x workgroups and over the 4 waves of each; partial
// (max, sum, O) triples are merged in LDS and, across workgroups, by whichever workgroup of
// the column group finishes last (ticket counter, no spinning), the same statistic merge crossAttnShardedHead does (attention_kernels.h:931-983).
// INT8 caches are widened to fp16 in registers (exact); the per-token key scale multiplies
// the score column, the value scale multiplies the probability (gemm_kernel_ext.cpp:471-500,
// gemm_kernel_ext2.cpp:75-91).
#include <atomic>
#include <mutex>


#include "attention_dev.h"
#include "attention_prefill.h"

namespace xfthip {

// launch bounds: three workgroups a CU.  The next block's keys are requested as soon as this block's scores are
// scaled and its values once this block's P.V products are issued, into the registers those have just left; at 128
// registers (four workgroups a CU) the compiler spills to keep that order and everything is slower, at 168 it fits
// (146 FP16, 168 INT8).  Against four workgroups a CU that request each block only when they need it: INT8 cache,
// batch 64 x 16384 tokens 594 -> 388 us (5.7 TB/s), 16 x 4096 42 -> 30 us; FP16 725 -> 713 us (6.0 TB/s), 16 x 4096
// 61 -> 44 us, 64 x 1024 58 -> 48 us.
// With at most one block a wave (short contexts at small batches) nothing can be requested ahead: that form keeps
// the plain order, the shorter program (few workgroups then: the same launch bounds do no harm).
template <bool INT8, bool PIPE>
__global__ __launch_bounds__(256, 3) void attn_kernel(AttnParams p) {
    __shared__ AttnLds<4> lds;
    attn_unit<INT8, 4, PIPE>(p, blockIdx.x, blockIdx.y % p.kv.H, blockIdx.y / p.kv.H, blockIdx.z, lds, [] { __syncthreads(); });
}

constexpr int kTicketParts = 8, kMaxParts = 32;
// merges the parts of a launch of attn_kernel that took no tickets: grid (columns of a group, groups), at most 128 parts
__global__ __launch_bounds__(128) void attn_merge_kernel(AttnParams p) {
    __shared__ float s_pm[128], s_f[128];
    attn_merge_unit(p, blockIdx.y, blockIdx.x, s_pm, s_f);
}

// 32 x 32 MFMA tiles, 32 columns a wave, K / V blocks shared through LDS (attention_prefill.h); two workgroups a CU
// Workgroups are handed to the 8 XCDs in turn by their linear index, and each XCD has an L2 of its own: the
// (sequence, KV head) pairs are dealt to the XCDs (pair = 8 k + XCD), and an XCD walks the column groups of one
// pair, longest history first, before it starts the next, so that the workgroups resident on an XCD share one or
// two pairs' keys and values in its L2 instead of all of them.
template <bool INT8, int CT>
__global__ __launch_bounds__(256, (CT == 1 ? 2 : 1)) void attn_prefill32_kernel(AttnParams p, int ncg, int npairs) {
    // INT8 cache: two buffers of widened blocks; FP16 cache: three 16 KB buffers the blocks are loaded into directly
    __shared__ __attribute__((aligned(16))) unsigned char lds[INT8 ? 2 * kP32BufBytes : 3 * 16384];
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int pair = (slot / ncg) * 8 + xcd;
    if (pair >= npairs) return;
    attn_prefill32_unit<4, CT, INT8>(p, pair % p.kv.H, ncg - 1 - slot % ncg, pair / p.kv.H, lds);
}

// Split-KV merge workspace: `slots` partial-result slots of kSlotFloats floats and one ticket per
// column group.  Plain xfthip_attention calls take one per stream from the library's per-stream scratch
// (allocated on a stream's first call); a model owns its own.
int attention_workspace_create(AttnWorkspace *w, int slots) {
    w->ws = nullptr, w->tickets = nullptr, w->slots = 0;
    XFT_CHECK_HIP(hipMalloc((void **)&w->ws, (size_t)slots * kSlotFloats * sizeof(float)));
    XFT_CHECK_HIP(hipMalloc((void **)&w->tickets, (size_t)slots * sizeof(unsigned int)));
    XFT_CHECK_HIP(hipMemset(w->tickets, 0, (size_t)slots * sizeof(unsigned int)));
    XFT_CHECK_HIP(hipDeviceSynchronize());
    w->slots = slots;
    return 0;
}

void attention_workspace_destroy(AttnWorkspace *w) {
    if (w->ws) (void)hipFree(w->ws);
    if (w->tickets) (void)hipFree(w->tickets);
    w->ws = nullptr, w->tickets = nullptr, w->slots = 0;
}

// the workspace of plain calls on `stream`
static int attention_stream_workspace(hipStream_t stream, AttnWorkspace *w) {
    void *parts = nullptr, *tickets = nullptr;
    if (int rc = stream_scratch(kScratchAttnParts, stream, (size_t)kWsSlots * kSlotFloats * sizeof(float), false, &parts)) return rc;
    if (int rc = stream_scratch(kScratchAttnTickets, stream, (size_t)kWsSlots * sizeof(unsigned int), true, &tickets)) return rc;
    w->ws = (float *)parts, w->tickets = (unsigned int *)tickets, w->slots = kWsSlots;
    return 0;
}

// ---- statically allocated workspace of xfthip_attention_static ---------------------------------
// Device memory that exists from the moment the code object is loaded: callers that must not
// allocate (stream capture, serving loops that forbid hipMalloc) get the split-KV partials and the
// tickets from here.  Each device holds its own copy at its own address; in host code the array's
// name is only a handle for hipGetSymbolAddress, never a pointer to pass to a kernel.
constexpr int kStaticSlots = 1024;
constexpr size_t kStaticTicketOffset = (size_t)kStaticSlots * kSlotFloats * sizeof(float);
static __device__ __align__(256) unsigned char scratch[kStaticTicketOffset + (size_t)kStaticSlots * sizeof(unsigned int)];

constexpr int kMaxDevices = 64;
static std::atomic<void *> g_scratch_ptr[kMaxDevices] = {}; // written once under g_scratch_mu, read without it
static std::mutex g_scratch_mu;

// Resolves (once per device, with that device current) the device address of `scratch` and clears
// the tickets.  Allocates nothing.  Called by xfthip_init and by the entry point's first call on a device.
int attention_static_scratch_init() {
    int dev = -1;
    XFT_CHECK_HIP(hipGetDevice(&dev));
    XFT_REQUIRE(dev >= 0 && dev < kMaxDevices, "attention_static_scratch_init: device index %d out of range", dev);
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (g_scratch_ptr[dev].load(std::memory_order_acquire) != nullptr) return 0;
    void *ptr = nullptr;
    XFT_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    XFT_REQUIRE(ptr != nullptr, "attention_static_scratch_init: no device address for the static scratch");
    XFT_CHECK_HIP(hipMemset((unsigned char *)ptr + kStaticTicketOffset, 0, (size_t)kStaticSlots * sizeof(unsigned int)));
    XFT_CHECK_HIP(hipDeviceSynchronize());
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    return 0;
}

} // namespace xfthip

using namespace xfthip;

// len_hint: upper bound of the visible sequence length when the positions live in device memory
// (0 = unknown, the cache length is assumed); it only steers the split count.
// wsp: the workspace to merge splits through (nullptr = the library's shared one, allocated on first
// use).  strict: fail instead of lowering the split count when the workspace is too small.
int xfthip::attention_launch(xfthip_kvcache_t c, const void *q, int qStride, void *out, int oStride, int out_dtype, int B, int S,
        int qHeads, float scale, int past, const int *past_dev, int len_hint, hipStream_t stream, const AttnWorkspace *wsp,
        bool strict) {
    XFT_REQUIRE(c && q && out, "xfthip_attention: null argument");
    XFT_REQUIRE(B > 0 && B <= c->kv.B, "xfthip_attention: batch %d exceeds cache batch %d", B, c->kv.B);
    XFT_REQUIRE(S > 0 && qHeads > 0 && qHeads % c->kv.H == 0, "xfthip_attention: bad S=%d or qHeads=%d (kvHeads=%d)", S, qHeads,
            c->kv.H);
    XFT_REQUIRE(c->kv.D == 128, "xfthip_attention: head size %d unsupported", c->kv.D);
    XFT_REQUIRE(out_dtype == XFTHIP_BF16 || out_dtype == XFTHIP_F32, "xfthip_attention: out_dtype must be bf16 or f32");
    XFT_REQUIRE(qStride >= qHeads * 128 && (qStride % 8) == 0 && ((uintptr_t)q & 15) == 0,
            "xfthip_attention: q must be 16-byte aligned with qStride >= qHeads*128 and %% 8 == 0");
    XFT_REQUIRE(oStride >= qHeads * 128, "xfthip_attention: oStride too small");
    XFT_REQUIRE(past_dev != nullptr || (past >= 0 && past + S <= c->maxSeq),
            "xfthip_attention: past %d + S %d exceeds the cache length %d", past, S, c->maxSeq);
    AttnParams p = {};
    p.kv = c->kv;
    p.q = (const uint16_t *)q;
    p.qStride = qStride;
    p.out = out;
    p.oStride = oStride;
    p.out_dtype = out_dtype;
    p.B = B;
    p.S = S;
    p.G = qHeads / c->kv.H;
    p.scale = scale;
    p.past = past;
    p.past_dev = past_dev;
    p.CG = (S * p.G + 15) / 16;
    // Many columns per KV head (prefill, long chunks): the form in which a wave walks the whole visible sequence
    // for its 32 columns through LDS blocks shared by its workgroup, taken once such waves fill the device.
    {
        const long waves1 = (long)B * c->kv.H * p.CG; // waves with one column tile each
        if (S > 1 && waves1 >= 4L * device_cu_count()) {
            p.nsplit = 1;
            const int ncg = (S * p.G + 127) / 128, npairs = B * c->kv.H;
            dim3 grid(8 * ((npairs + 7) / 8) * ncg);
            if (c->kv.int8) hipLaunchKernelGGL((attn_prefill32_kernel<true, 1>), grid, dim3(256), 0, stream, p, ncg, npairs);
            else hipLaunchKernelGGL((attn_prefill32_kernel<false, 1>), grid, dim3(256), 0, stream, p, ncg, npairs);
            XFT_CHECK_HIP(hipGetLastError());
            return 0;
        }
    }
    // split the KV sequence so that the launch has about one workgroup a CU (attention_split_count); the longest
    // visible sequence is bounded by the cache length when the real one lives in device memory
    const int len = past_dev ? ((len_hint > 0 && len_hint < c->maxSeq) ? len_hint : c->maxSeq) : past + S;
    const int wgs = B * c->kv.H * p.CG;
    int nsplit = attention_split_count(len, wgs);
    AttnWorkspace of_stream;
    if (nsplit > 1) {
        if (wsp == nullptr) {
            if (int rc = attention_stream_workspace(stream, &of_stream)) return rc;
            wsp = &of_stream;
        }
        if ((size_t)wgs * nsplit > (size_t)wsp->slots) {
            XFT_REQUIRE(!strict,
                    "xfthip_attention_static: %d column groups x %d sequence splits need %zu partial-result slots, the static "
                    "scratch holds %d; use xfthip_attention for this shape",
                    wgs, nsplit, (size_t)wgs * nsplit, wsp->slots);
            while (nsplit > 1 && (size_t)wgs * nsplit > (size_t)wsp->slots) --nsplit;
        }
    }
    p.nsplit = nsplit;
    p.ws = wsp ? wsp->ws : nullptr;
    // up to kTicketParts parts the last workgroup of a column group merges them; beyond, a second launch does (8 KV
    // heads, 2048 tokens, 16 parts: 11.7 us merged by the last workgroup, 10.2 by the launch; 4096 tokens 13.7 / 12.7)
    const bool merge_launch = nsplit > kTicketParts;
    p.tickets = (wsp && !merge_launch) ? wsp->tickets : nullptr;
    dim3 grid(nsplit, c->kv.H * p.CG, B);
    // more than one 32-token block a wave somewhere: the form that requests blocks ahead
    const bool pipe = (len + 31) / 32 > 4 * nsplit;
    if (c->kv.int8) {
        if (pipe) hipLaunchKernelGGL((attn_kernel<true, true>), grid, dim3(256), 0, stream, p);
        else hipLaunchKernelGGL((attn_kernel<true, false>), grid, dim3(256), 0, stream, p);
    } else {
        if (pipe) hipLaunchKernelGGL((attn_kernel<false, true>), grid, dim3(256), 0, stream, p);
        else hipLaunchKernelGGL((attn_kernel<false, false>), grid, dim3(256), 0, stream, p);
    }
    if (merge_launch) {
        const int cols = S * p.G < 16 ? S * p.G : 16;
        hipLaunchKernelGGL(attn_merge_kernel, dim3(cols, wgs), dim3(128), 0, stream, p);
    }
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

int xfthip::attention_split_count(int len, int units) {
    // Measured over batch 1 .. 64, 8 and 32 KV heads, 512 .. 16384 tokens, both cache kinds: a launch is fastest with
    // about one workgroup a CU.  With at least that many (batch, KV head, column group) units nothing is split, and the
    // partials, tickets and merge fall away with it (64 sequences x 8 KV heads x 512 tokens: 35 -> 27 us FP16, 26 ->
    // 17 us INT8, against two parts); below, the sequence is cut into CUs / units parts, twice that where this gives
    // at most 4 parts and the sequence has 2048 tokens or more (16 x 8 KV heads x 4096 tokens INT8: 37.5 us with 2
    // parts, 32.8 with 4), every wave keeping at least one 32-token block, 32 parts at most (batch 1, 8 KV heads,
    // 16384 tokens: 23.0 us with 16 parts, 20.2 with 32, 23.0 with 64; INT8 21.6 / 16.2 / 16.9).
    const int nblk = (len + 31) / 32;
    const int cus = device_cu_count();
    if (units >= cus) return 1;
    int nsplit = cus / units;
    if (nsplit <= 4 && nblk >= 64) nsplit *= 2;
    const int cap = (nblk + 3) / 4;
    if (nsplit > cap) nsplit = cap;
    if (nsplit > kMaxParts) nsplit = kMaxParts;
    if (nsplit < 1) nsplit = 1;
    while (nsplit > 1 && (size_t)units * nsplit > (size_t)kWsSlots) --nsplit;
    return nsplit;
}

extern "C" int xfthip_attention(xfthip_kvcache_t c, const void *q, int qStride, void *out, int oStride, int out_dtype,
        int B, int S, int qHeads, float scale, int past, const int *past_dev, xfthip_stream_t stream) {
    return attention_launch(c, q, qStride, out, oStride, out_dtype, B, S, qHeads, scale, past, past_dev, 0, (hipStream_t)stream,
            nullptr, false);
}

extern "C" int xfthip_attention_static(xfthip_kvcache_t c, const void *q, int qStride, void *out, int oStride, int out_dtype,
        int B, int S, int qHeads, float scale, int past, const int *past_dev, xfthip_stream_t stream) {
    int dev = -1;
    XFT_CHECK_HIP(hipGetDevice(&dev));
    XFT_REQUIRE(dev >= 0 && dev < kMaxDevices, "xfthip_attention_static: device index %d out of range", dev);
    if (g_scratch_ptr[dev].load(std::memory_order_acquire) == nullptr)
        if (int rc = attention_static_scratch_init()) return rc;
    unsigned char *base = (unsigned char *)g_scratch_ptr[dev].load(std::memory_order_acquire);
    AttnWorkspace w;
    w.ws = (float *)base;
    w.tickets = (unsigned int *)(base + kStaticTicketOffset);
    w.slots = kStaticSlots;
    return attention_launch(c, q, qStride, out, oStride, out_dtype, B, S, qHeads, scale, past, past_dev, 0, (hipStream_t)stream, &w,
            true);
}
