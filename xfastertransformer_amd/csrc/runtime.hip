// Runtime plumbing behind the C-ABI: device selection, error text, memory, streams, events.
#include <stdarg.h>
#include <string.h>

#include <map>
#include <mutex>
#include <tuple>

#include "common.h"
#include "qgemm.h"

namespace xfthip {

static thread_local char g_err[1024] = "";
static int g_device = -1;
static int g_cus = 0;
static std::mutex g_mu;

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int device_cu_count() {
    return g_cus > 0 ? g_cus : 256;
}

namespace {
struct ScratchEntry {
    void *ptr = nullptr;
    size_t bytes = 0;
};
std::mutex g_scratch_registry_mu;
std::map<std::tuple<int, int, hipStream_t>, ScratchEntry> g_scratch_registry;
thread_local bool g_scratch_key_set = false;
thread_local hipStream_t g_scratch_key = nullptr;
} // namespace

ScratchKeyScope::ScratchKeyScope(hipStream_t key) {
    g_scratch_key_set = true;
    g_scratch_key = key;
}
ScratchKeyScope::~ScratchKeyScope() {
    g_scratch_key_set = false;
}

int stream_scratch(ScratchPurpose purpose, hipStream_t stream, size_t bytes, bool zero_new, void **out) {
    int dev = 0;
    XFT_CHECK_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lk(g_scratch_registry_mu);
    ScratchEntry &e = g_scratch_registry[std::make_tuple((int)purpose, dev, g_scratch_key_set ? g_scratch_key : stream)];
    if (e.bytes < bytes) {
        if (e.ptr) {
            XFT_CHECK_HIP(hipDeviceSynchronize()); // work already queued may still use the smaller buffer
            (void)hipFree(e.ptr);
            e.ptr = nullptr, e.bytes = 0;
        }
        XFT_CHECK_HIP(hipMalloc(&e.ptr, bytes));
        if (zero_new) {
            XFT_CHECK_HIP(hipMemset(e.ptr, 0, bytes));
            XFT_CHECK_HIP(hipDeviceSynchronize());
        }
        e.bytes = bytes;
    }
    *out = e.ptr;
    return 0;
}

} // namespace xfthip

using namespace xfthip;

namespace xfthip {
typedef uint32_t cp16 __attribute__((ext_vector_type(4)));
// plain grid-stride copy, 16 bytes per lane: the known-traffic kernel that HBM byte counters are
// calibrated against
__global__ void stream_copy_kernel(const cp16 *__restrict__ src, cp16 *__restrict__ dst, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) dst[i] = src[i];
}
// read-only stream: every workgroup reads a contiguous share with 8 independent 16-byte loads a lane in flight and
// keeps an XOR of what it read (stored only if it matches a value it never does): what reading `n` chunks costs with
// no arithmetic behind it, launch ramp and tail included - the floor the weight-streaming kernels are held against
__global__ __launch_bounds__(256) void stream_read_kernel(const cp16 *__restrict__ src, size_t n_per_block, size_t n, unsigned *sink) {
    const size_t begin = (size_t)blockIdx.x * n_per_block;
    const size_t end = begin + n_per_block < n ? begin + n_per_block : n;
    cp16 acc = {0u, 0u, 0u, 0u};
    for (size_t i = begin + threadIdx.x; i < end; i += 256 * 8) {
        cp16 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = i + (size_t)u * 256 < end ? src[i + (size_t)u * 256] : cp16 {0u, 0u, 0u, 0u};
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= v[u];
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9E3779B9u && sink) sink[0] = 1u;
}
} // namespace xfthip

extern "C" {

const char *xfthip_last_error(void) {
    return g_err;
}

int xfthip_init(int device) {
    std::lock_guard<std::mutex> lk(g_mu);
    int n = 0;
    XFT_CHECK_HIP(hipGetDeviceCount(&n));
    XFT_REQUIRE(n > 0, "xfthip_init: no HIP device visible");
    XFT_REQUIRE(device >= 0 && device < n, "xfthip_init: device %d out of range (have %d)", device, n);
    XFT_CHECK_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    XFT_CHECK_HIP(hipGetDeviceProperties(&prop, device));
    XFT_REQUIRE(strncmp(prop.gcnArchName, "gfx950", 6) == 0,
            "xfthip_init: this library is built for gfx950 only, device %d is %s", device, prop.gcnArchName);
    g_device = device;
    g_cus = prop.multiProcessorCount;
    // the statically allocated attention workspace: resolve its address on this device now, so
    // that xfthip_attention_static never has to during a stream capture
    return attention_static_scratch_init();
}

int xfthip_finalize(void) {
    if (g_device < 0) return 0;
    XFT_CHECK_HIP(hipDeviceSynchronize());
    return 0;
}

int xfthip_device_info(char *name, int name_len, int *compute_units, size_t *hbm_bytes) {
    XFT_REQUIRE(g_device >= 0, "xfthip_device_info: call xfthip_init first");
    hipDeviceProp_t prop;
    XFT_CHECK_HIP(hipGetDeviceProperties(&prop, g_device));
    if (name && name_len > 0) snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (hbm_bytes) *hbm_bytes = prop.totalGlobalMem;
    return 0;
}

int xfthip_malloc(void **ptr, size_t bytes) {
    XFT_REQUIRE(ptr != nullptr, "xfthip_malloc: null out pointer");
    *ptr = nullptr;
    if (bytes == 0) bytes = 16;
    XFT_CHECK_HIP(hipMalloc(ptr, bytes));
    return 0;
}

int xfthip_free(void *ptr) {
    if (ptr) XFT_CHECK_HIP(hipFree(ptr));
    return 0;
}

int xfthip_memcpy_h2d(void *dst, const void *src_host, size_t bytes, xfthip_stream_t stream) {
    if (bytes == 0) return 0;
    XFT_CHECK_HIP(hipMemcpyAsync(dst, src_host, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
    XFT_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream)); // pageable host memory: make the call safe
    return 0;
}

int xfthip_memcpy_d2h(void *dst_host, const void *src, size_t bytes, xfthip_stream_t stream) {
    if (bytes == 0) return 0;
    XFT_CHECK_HIP(hipMemcpyAsync(dst_host, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
    XFT_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int xfthip_memcpy_d2d(void *dst, const void *src, size_t bytes, xfthip_stream_t stream) {
    if (bytes == 0) return 0;
    XFT_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
    return 0;
}

int xfthip_copy_kernel(void *dst, const void *src, size_t bytes, xfthip_stream_t stream) {
    XFT_REQUIRE(dst && src && bytes % 16 == 0 && (((uintptr_t)dst | (uintptr_t)src) & 15) == 0,
            "xfthip_copy_kernel: pointers and size must be 16-byte aligned");
    if (bytes == 0) return 0;
    const size_t n = bytes / 16;
    const int blocks = (int)((n + 1023) / 1024 < 8192 ? (n + 1023) / 1024 : 8192);
    hipLaunchKernelGGL(xfthip::stream_copy_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const xfthip::cp16 *)src,
            (xfthip::cp16 *)dst, n);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

int xfthip_read_kernel(const void *src, size_t bytes, int blocks, xfthip_stream_t stream) {
    XFT_REQUIRE(src && bytes % 16 == 0 && ((uintptr_t)src & 15) == 0, "xfthip_read_kernel: pointer and size must be 16-byte aligned");
    if (bytes == 0) return 0;
    const size_t n = bytes / 16;
    if (blocks <= 0) blocks = 2 * device_cu_count();
    const size_t per = (n + blocks - 1) / blocks;
    hipLaunchKernelGGL(xfthip::stream_read_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const xfthip::cp16 *)src, per, n,
            (unsigned *)nullptr);
    XFT_CHECK_HIP(hipGetLastError());
    return 0;
}

int xfthip_device_memory(size_t *free_bytes, size_t *total_bytes) {
    size_t f = 0, t = 0;
    XFT_CHECK_HIP(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return 0;
}

int xfthip_memset(void *dst, int value, size_t bytes, xfthip_stream_t stream) {
    if (bytes == 0) return 0;
    XFT_CHECK_HIP(hipMemsetAsync(dst, value, bytes, (hipStream_t)stream));
    return 0;
}

int xfthip_stream_create(xfthip_stream_t *stream) {
    hipStream_t s;
    XFT_CHECK_HIP(hipStreamCreate(&s)); // default priority only
    *stream = (xfthip_stream_t)s;
    return 0;
}

int xfthip_stream_destroy(xfthip_stream_t stream) {
    if (stream) XFT_CHECK_HIP(hipStreamDestroy((hipStream_t)stream));
    return 0;
}

int xfthip_stream_synchronize(xfthip_stream_t stream) {
    XFT_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int xfthip_device_synchronize(void) {
    XFT_CHECK_HIP(hipDeviceSynchronize());
    return 0;
}

int xfthip_graph_begin(xfthip_stream_t stream) {
    XFT_REQUIRE(stream != nullptr, "xfthip_graph_begin: capture needs a stream of its own, not the null stream");
    // what the recordable entry points take from the per-stream scratch must exist before the capture starts
    if (int rc = qgemm_split_reserve((hipStream_t)stream)) return rc;
    XFT_CHECK_HIP(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
    return 0;
}

int xfthip_graph_end(xfthip_stream_t stream, xfthip_graph_t *graph) {
    XFT_REQUIRE(stream != nullptr && graph != nullptr, "xfthip_graph_end: null argument");
    hipGraph_t g = nullptr;
    XFT_CHECK_HIP(hipStreamEndCapture((hipStream_t)stream, &g));
    hipGraphExec_t exec = nullptr;
    const hipError_t e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    XFT_CHECK_HIP(e);
    *graph = (xfthip_graph_t)exec;
    return 0;
}

int xfthip_graph_launch(xfthip_graph_t graph, xfthip_stream_t stream) {
    XFT_REQUIRE(graph != nullptr, "xfthip_graph_launch: null graph");
    XFT_CHECK_HIP(hipGraphLaunch((hipGraphExec_t)graph, (hipStream_t)stream));
    return 0;
}

int xfthip_graph_destroy(xfthip_graph_t graph) {
    if (graph) XFT_CHECK_HIP(hipGraphExecDestroy((hipGraphExec_t)graph));
    return 0;
}

int xfthip_event_create(xfthip_event_t *ev) {
    hipEvent_t e;
    XFT_CHECK_HIP(hipEventCreate(&e));
    *ev = (xfthip_event_t)e;
    return 0;
}

int xfthip_event_destroy(xfthip_event_t ev) {
    if (ev) XFT_CHECK_HIP(hipEventDestroy((hipEvent_t)ev));
    return 0;
}

int xfthip_event_record(xfthip_event_t ev, xfthip_stream_t stream) {
    XFT_CHECK_HIP(hipEventRecord((hipEvent_t)ev, (hipStream_t)stream));
    return 0;
}

int xfthip_event_synchronize(xfthip_event_t ev) {
    XFT_CHECK_HIP(hipEventSynchronize((hipEvent_t)ev));
    return 0;
}

int xfthip_event_elapsed_ms(xfthip_event_t start, xfthip_event_t stop, float *ms) {
    XFT_CHECK_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return 0;
}

} // extern "C"
