// Runtime half of the C ABI: device selection, the single in-order stream, buffers,
// copies, events.  Replaces what the reference gets from krnl's Device / Buffer.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "agh_internal.h"

namespace agh {

static std::recursive_mutex g_mutex;
static bool g_init = false;
static int g_device = -1;
static int g_cus = 0;
static hipStream_t g_stream = nullptr;
// A second in-order stream for work the caller declares independent (agh_branch_*).  `g_cur` is the
// stream entry points launch on: g_stream, or g_side between agh_branch_begin and agh_branch_end.  Each
// stream has its own workspace (two split-K GEMMs may then run side by side).
static hipStream_t g_side = nullptr;
static hipStream_t g_cur = nullptr;
static bool g_side_dirty = false;  // the branch stream has work the main stream has not waited for
constexpr int kBranchEvents = 64;
static hipEvent_t g_events[kBranchEvents];
static int g_event_next = 0;
static void *g_ws = nullptr, *g_ws_side = nullptr;
static size_t g_ws_bytes = 0, g_ws_side_bytes = 0;
static thread_local char g_err[512] = "";

std::recursive_mutex &api_mutex() { return g_mutex; }
hipStream_t stream() { return g_cur; }
bool initialized() { return g_init; }
int compute_units() { return g_cus; }

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(hipError_t e, const char *what) {
    snprintf(g_err, sizeof(g_err), "%s: %s (%d)", what, hipGetErrorString(e), (int)e);
    return (int)e > 0 ? (int)e : 999;
}

int workspace(size_t bytes, void **ptr) {
    const bool side = g_cur == g_side && g_side != nullptr;
    void *&ws = side ? g_ws_side : g_ws;
    size_t &have = side ? g_ws_side_bytes : g_ws_bytes;
    if (bytes > have) {
        // in-order stream: earlier kernels using the old block must finish first
        AGH_HIP(hipStreamSynchronize(g_cur));
        if (ws) AGH_HIP(hipFree(ws));
        ws = nullptr;
        have = 0;
        size_t want = bytes < (size_t)(8u << 20) ? (size_t)(8u << 20) : bytes;
        AGH_HIP(hipMalloc(&ws, want));
        have = want;
    }
    *ptr = ws;
    return AGH_OK;
}

static hipEvent_t next_event() {
    hipEvent_t e = g_events[g_event_next];
    g_event_next = (g_event_next + 1) % kBranchEvents;
    return e;
}

}  // namespace agh

using namespace agh;

extern "C" {

int agh_init(int device_index) {
    std::lock_guard<std::recursive_mutex> lock(g_mutex);
    if (g_init) {
        if (device_index == g_device) return AGH_OK;
        return fail(AGH_EINVAL, "agh_init: already initialised on device %d", g_device);
    }
    int count = 0;
    AGH_HIP(hipGetDeviceCount(&count));
    if (device_index < 0 || device_index >= count)
        return fail(AGH_EINVAL, "agh_init: device index %d out of range (found %d devices)", device_index, count);
    AGH_HIP(hipSetDevice(device_index));
    // latency matters for launch-bound work (a LeNet5 inference is tens of microseconds): spin, do not
    // sleep, in synchronising calls.  Best effort: the flag cannot change once the device is active.
    (void)hipSetDeviceFlags(hipDeviceScheduleSpin);
    (void)hipGetLastError();
    hipDeviceProp_t prop;
    AGH_HIP(hipGetDeviceProperties(&prop, device_index));
    g_cus = prop.multiProcessorCount;
    AGH_HIP(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
    AGH_HIP(hipStreamCreateWithFlags(&g_side, hipStreamNonBlocking));  // default priority, like g_stream
    for (int i = 0; i < kBranchEvents; ++i) AGH_HIP(hipEventCreateWithFlags(&g_events[i], hipEventDisableTiming));
    g_cur = g_stream;
    g_side_dirty = false;
    g_device = device_index;
    g_init = true;
    return AGH_OK;
}

int agh_shutdown(void) {
    std::lock_guard<std::recursive_mutex> lock(g_mutex);
    if (!g_init) return AGH_OK;
    AGH_HIP(hipStreamSynchronize(g_stream));
    AGH_HIP(hipStreamSynchronize(g_side));
    if (g_ws) AGH_HIP(hipFree(g_ws));
    if (g_ws_side) AGH_HIP(hipFree(g_ws_side));
    g_ws = g_ws_side = nullptr;
    g_ws_bytes = g_ws_side_bytes = 0;
    for (int i = 0; i < kBranchEvents; ++i) (void)hipEventDestroy(g_events[i]);
    AGH_HIP(hipStreamDestroy(g_side));
    AGH_HIP(hipStreamDestroy(g_stream));
    g_stream = g_side = g_cur = nullptr;
    g_init = false;
    g_device = -1;
    return AGH_OK;
}

const char *agh_last_error_string(void) { return g_err; }

int agh_device_info(char *name, size_t name_len, int *compute_units, size_t *total_mem_bytes) {
    AGH_API_ENTER();
    hipDeviceProp_t prop;
    AGH_HIP(hipGetDeviceProperties(&prop, g_device));
    if (name && name_len) {
        snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
    }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (total_mem_bytes) *total_mem_bytes = prop.totalGlobalMem;
    return AGH_OK;
}

int agh_malloc(void **ptr, size_t bytes) {
    AGH_API_ENTER();
    if (!ptr) return fail(AGH_ENULL, "agh_malloc: null out pointer");
    *ptr = nullptr;
    // zero-length tensors are legal in the reference; hand back a real 256-byte block
    AGH_HIP(hipMalloc(ptr, bytes ? bytes : 256));
    return AGH_OK;
}

int agh_free(void *ptr) {
    AGH_API_ENTER();
    if (!ptr) return AGH_OK;
    // the buffer may still be read by queued kernels
    AGH_HIP(hipStreamSynchronize(g_stream));
    if (g_side_dirty) AGH_HIP(hipStreamSynchronize(g_side));
    AGH_HIP(hipFree(ptr));
    return AGH_OK;
}

int agh_memcpy_h2d(void *dst, const void *src, size_t bytes) {
    AGH_API_ENTER();
    if (bytes == 0) return AGH_OK;
    if (!dst || !src) return fail(AGH_ENULL, "agh_memcpy_h2d: null pointer");
    AGH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g_stream));
    return AGH_OK;
}

int agh_memcpy_d2h(void *dst, const void *src, size_t bytes) {
    AGH_API_ENTER();
    if (bytes == 0) return AGH_OK;
    if (!dst || !src) return fail(AGH_ENULL, "agh_memcpy_d2h: null pointer");
    AGH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, g_stream));
    AGH_HIP(hipStreamSynchronize(g_stream));
    return AGH_OK;
}

int agh_memcpy_d2d(void *dst, const void *src, size_t bytes) {
    AGH_API_ENTER();
    if (bytes == 0) return AGH_OK;
    if (!dst || !src) return fail(AGH_ENULL, "agh_memcpy_d2d: null pointer");
    AGH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, g_stream));
    return AGH_OK;
}

int agh_memcpy_d2h_async(void *dst, const void *src, size_t bytes) {
    AGH_API_ENTER();
    if (bytes == 0) return AGH_OK;
    if (!dst || !src) return fail(AGH_ENULL, "agh_memcpy_d2h_async: null pointer");
    AGH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, g_stream));
    return AGH_OK;
}

int agh_host_alloc(void **ptr, size_t bytes) {
    AGH_API_ENTER();
    if (!ptr) return fail(AGH_ENULL, "agh_host_alloc: null out pointer");
    *ptr = nullptr;
    AGH_HIP(hipHostMalloc(ptr, bytes ? bytes : 64, hipHostMallocDefault));
    return AGH_OK;
}

int agh_host_free(void *ptr) {
    AGH_API_ENTER();
    if (!ptr) return AGH_OK;
    AGH_HIP(hipStreamSynchronize(g_stream));
    AGH_HIP(hipHostFree(ptr));
    return AGH_OK;
}

int agh_graph_begin(void) {
    AGH_API_ENTER();
    AGH_HIP(hipStreamBeginCapture(g_stream, hipStreamCaptureModeThreadLocal));
    return AGH_OK;
}

int agh_graph_end(void **graph_exec) {
    AGH_API_ENTER();
    if (!graph_exec) return fail(AGH_ENULL, "agh_graph_end: null out pointer");
    *graph_exec = nullptr;
    hipGraph_t graph = nullptr;
    if (g_cur != g_stream) return fail(AGH_EINVAL, "agh_graph_end: still inside a branch");
    if (g_side_dirty) {  // an arm left open would make the capture invalid
        hipEvent_t e = next_event();
        AGH_HIP(hipEventRecord(e, g_side));
        AGH_HIP(hipStreamWaitEvent(g_stream, e, 0));
        g_side_dirty = false;
    }
    AGH_HIP(hipStreamEndCapture(g_stream, &graph));
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return hip_fail(e, "hipGraphInstantiate");
    *graph_exec = (void *)exec;
    return AGH_OK;
}

int agh_graph_launch(void *graph_exec) {
    AGH_API_ENTER();
    if (!graph_exec) return fail(AGH_ENULL, "agh_graph_launch: null graph");
    AGH_HIP(hipGraphLaunch((hipGraphExec_t)graph_exec, g_stream));
    return AGH_OK;
}

int agh_graph_destroy(void *graph_exec) {
    AGH_API_ENTER();
    if (!graph_exec) return AGH_OK;
    AGH_HIP(hipStreamSynchronize(g_stream));
    AGH_HIP(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
    return AGH_OK;
}

int agh_sync(void) {
    AGH_API_ENTER();
    AGH_HIP(hipStreamSynchronize(g_stream));
    if (g_side_dirty) {
        AGH_HIP(hipStreamSynchronize(g_side));
        g_side_dirty = false;
    }
    return AGH_OK;
}

int agh_branch_begin(void) {
    AGH_API_ENTER();
    if (g_cur != g_stream) return fail(AGH_EINVAL, "agh_branch_begin: already inside a branch");
    hipEvent_t e = next_event();
    AGH_HIP(hipEventRecord(e, g_stream));
    AGH_HIP(hipStreamWaitEvent(g_side, e, 0));
    g_cur = g_side;
    g_side_dirty = true;
    return AGH_OK;
}

int agh_branch_end(void) {
    AGH_API_ENTER();
    if (g_cur != g_side) return fail(AGH_EINVAL, "agh_branch_end: not inside a branch");
    g_cur = g_stream;
    return AGH_OK;
}

int agh_branch_join(void) {
    AGH_API_ENTER();
    if (g_cur != g_stream) return fail(AGH_EINVAL, "agh_branch_join: still inside a branch");
    if (!g_side_dirty) return AGH_OK;
    hipEvent_t e = next_event();
    AGH_HIP(hipEventRecord(e, g_side));
    AGH_HIP(hipStreamWaitEvent(g_stream, e, 0));
    g_side_dirty = false;
    return AGH_OK;
}

void *agh_stream(void) { return (void *)g_stream; }

int agh_event_create(void **event) {
    AGH_API_ENTER();
    if (!event) return fail(AGH_ENULL, "agh_event_create: null out pointer");
    hipEvent_t e;
    AGH_HIP(hipEventCreate(&e));
    *event = (void *)e;
    return AGH_OK;
}

int agh_event_destroy(void *event) {
    AGH_API_ENTER();
    if (!event) return AGH_OK;
    AGH_HIP(hipEventDestroy((hipEvent_t)event));
    return AGH_OK;
}

int agh_event_record(void *event) {
    AGH_API_ENTER();
    if (!event) return fail(AGH_ENULL, "agh_event_record: null event");
    AGH_HIP(hipEventRecord((hipEvent_t)event, g_stream));
    return AGH_OK;
}

int agh_event_elapsed_ms(void *start, void *stop, float *ms) {
    AGH_API_ENTER();
    if (!start || !stop || !ms) return fail(AGH_ENULL, "agh_event_elapsed_ms: null argument");
    AGH_HIP(hipEventSynchronize((hipEvent_t)stop));
    AGH_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return AGH_OK;
}

}  // extern "C"
