// Runtime half of the C ABI: device selection, the in-order streams, the caching buffer
// allocator, copies, events, graphs.  Replaces what the reference gets from krnl's Device / Buffer.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <map>
#include <unordered_map>
#include <vector>

#include "agh_internal.h"

// Fixed scratch of agh_gemm_bf16_noalloc: split-K partials for callers that may not allocate.  In host
// code this name is only a handle for hipGetSymbolAddress; the device address is looked up once in
// agh_init (g_scratch_ptr) and that pointer is what kernels receive.
static __device__ __align__(256) unsigned char scratch[AGH_NOALLOC_SCRATCH_BYTES];

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
// Fork / join events.  Eager work and a capture in progress draw from separate rings, so an event that a captured
// graph's edges were built from is never re-recorded by eager work (and the other way round).
constexpr int kBranchEvents = 64;
static hipEvent_t g_events[kBranchEvents], g_capture_events[kBranchEvents];
static int g_event_next = 0, g_capture_event_next = 0;
static bool g_capturing = false;   // between agh_graph_begin and agh_graph_end
static int g_live_graphs = 0;      // graph executables not yet destroyed: their nodes hold workspace pointers
static void *g_scratch_ptr = nullptr;  // device address of `scratch` on g_device
static thread_local char g_err[512] = "";

// Library-owned workspace of one stream.  A block that a live graph may reference is retired, not
// freed, when a larger one is needed; retired blocks go at agh_shutdown or when the last graph is
// destroyed.  Growth at least doubles, so the retired blocks together are smaller than the live one.
struct Workspace {
    void *ptr = nullptr;
    size_t bytes = 0;
};
static Workspace g_ws, g_ws_side;
static std::vector<void *> g_ws_retired;

// ---- caching allocator behind agh_malloc / agh_free ----
// Freed blocks are kept, by size, and handed out again without touching the driver.  Work is issued in
// order on one stream, so a block freed by the host while kernels that use it are still queued is safe
// to reuse: whatever is launched on it later runs after them.  The only other stream is the branch
// stream: a block freed while that stream had unjoined work remembers the branch it may belong to, and
// reusing it on the main stream first makes the main stream wait for the branch stream.
struct CachedBlock {
    void *ptr;
    uint64_t side_seq;  // branch number current when it was freed with the branch stream busy, else 0
};
static std::multimap<size_t, CachedBlock> g_free_blocks;     // by capacity
static std::unordered_map<void *, size_t> g_live_blocks;     // capacity of every block handed out
static size_t g_cached_bytes = 0, g_cache_limit = (size_t)64 << 30;
// Blocks freed while a graph is being captured: they can neither be handed to the driver nor (their capacity class
// being taken by agh_malloc, which a capture refuses anyway) reused before the capture ends; agh_graph_end files them.
struct DeferredFree {
    void *ptr;
    size_t cap;  // 0: not from this allocator's books, goes back to the driver
};
static std::vector<DeferredFree> g_deferred_frees;
static uint64_t g_side_seq = 0, g_side_joined_seq = 0;

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

static int release_retired_workspaces() {
    for (void *p : g_ws_retired) AGH_HIP(hipFree(p));
    g_ws_retired.clear();
    return AGH_OK;
}

int workspace(size_t bytes, void **ptr) {
    const bool side = g_cur == g_side && g_side != nullptr;
    Workspace &ws = side ? g_ws_side : g_ws;
    if (bytes > ws.bytes) {
        if (g_capturing)
            return fail(AGH_ERANGE, "workspace: %zu bytes needed while capturing a graph, %zu available: run the sequence "
                        "once eagerly before agh_graph_begin", bytes, ws.bytes);
        size_t want = bytes < (size_t)(8u << 20) ? (size_t)(8u << 20) : bytes;
        if (want < 2 * ws.bytes) want = 2 * ws.bytes;
        void *fresh = nullptr;
        AGH_HIP(hipMalloc(&fresh, want));
        if (ws.ptr) {
            if (g_live_graphs > 0) {
                g_ws_retired.push_back(ws.ptr);  // a captured node may still name it
            } else {
                // in-order stream: earlier kernels using the old block must finish first
                AGH_HIP(hipStreamSynchronize(g_cur));
                AGH_HIP(hipFree(ws.ptr));
            }
        }
        ws.ptr = fresh;
        ws.bytes = want;
    }
    *ptr = ws.ptr;
    return AGH_OK;
}

int static_workspace(size_t bytes, void **ptr) {
    if (g_cur != g_stream)
        return fail(AGH_EINVAL, "agh_gemm_bf16_noalloc: called inside a branch, where it would share the fixed scratch "
                    "buffer with the main stream's calls");
    if (bytes > (size_t)AGH_NOALLOC_SCRATCH_BYTES)
        return fail(AGH_ERANGE, "agh_gemm_bf16_noalloc: this shape needs %zu bytes of split-K scratch, the fixed buffer "
                    "holds %zu: use agh_gemm_bf16", bytes, (size_t)AGH_NOALLOC_SCRATCH_BYTES);
    if (!g_scratch_ptr) return fail(AGH_ENOINIT, "agh_gemm_bf16_noalloc: the fixed scratch buffer has no device address");
    *ptr = g_scratch_ptr;
    return AGH_OK;
}

static hipEvent_t next_event() {
    if (g_capturing) {
        hipEvent_t e = g_capture_events[g_capture_event_next];
        g_capture_event_next = (g_capture_event_next + 1) % kBranchEvents;
        return e;
    }
    hipEvent_t e = g_events[g_event_next];
    g_event_next = (g_event_next + 1) % kBranchEvents;
    return e;
}

// Later work on the main stream waits for everything issued so far on the branch stream.
static int join_side() {
    if (!g_side_dirty) return AGH_OK;
    hipEvent_t e = next_event();
    AGH_HIP(hipEventRecord(e, g_side));
    AGH_HIP(hipStreamWaitEvent(g_stream, e, 0));
    g_side_joined_seq = g_side_seq;
    // inside a branch more work for the branch stream may follow: it stays dirty
    g_side_dirty = g_cur == g_side;
    return AGH_OK;
}

// The host waits for both streams.
static int sync_all() {
    AGH_HIP(hipStreamSynchronize(g_stream));
    if (g_side_dirty) {
        AGH_HIP(hipStreamSynchronize(g_side));
        g_side_joined_seq = g_side_seq;
        g_side_dirty = g_cur == g_side;
    }
    return AGH_OK;
}

// capacity classes: 256 B steps up to 4 KiB, then four classes per octave (waste < 25 %)
static size_t block_capacity(size_t bytes) {
    if (bytes <= 4096) return bytes ? (bytes + 255) & ~(size_t)255 : 256;
    size_t top = (size_t)1 << (63 - __builtin_clzll((unsigned long long)bytes));
    size_t step = top >> 2;
    return (bytes + step - 1) & ~(step - 1);
}

static int release_cached_blocks() {
    if (int rc = sync_all()) return rc;
    for (auto &kv : g_free_blocks) AGH_HIP(hipFree(kv.second.ptr));
    g_free_blocks.clear();
    g_cached_bytes = 0;
    return AGH_OK;
}

// Files the blocks that were freed during a capture (called once the capture has ended, successfully or not).
static int flush_deferred_frees() {
    std::vector<DeferredFree> todo;
    todo.swap(g_deferred_frees);
    for (const DeferredFree &d : todo) {
        if (d.cap == 0 || d.cap > g_cache_limit) {
            if (int rc = sync_all()) return rc;
            AGH_HIP(hipFree(d.ptr));
            continue;
        }
        if (g_cached_bytes + d.cap > g_cache_limit)
            if (int rc = release_cached_blocks()) return rc;
        g_free_blocks.emplace(d.cap, CachedBlock{d.ptr, g_side_dirty ? g_side_seq : 0});
        g_cached_bytes += d.cap;
    }
    return AGH_OK;
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
    for (int i = 0; i < kBranchEvents; ++i) {
        AGH_HIP(hipEventCreateWithFlags(&g_events[i], hipEventDisableTiming));
        AGH_HIP(hipEventCreateWithFlags(&g_capture_events[i], hipEventDisableTiming));
    }
    // this device's copy of the fixed scratch array (the device is current)
    g_scratch_ptr = nullptr;
    AGH_HIP(hipGetSymbolAddress(&g_scratch_ptr, HIP_SYMBOL(scratch)));
    g_cur = g_stream;
    g_side_dirty = false;
    g_capturing = false;
    g_live_graphs = 0;
    g_side_seq = g_side_joined_seq = 0;
    if (const char *s = getenv("AGH_CACHE_LIMIT_MB"))
        if (*s) g_cache_limit = (size_t)strtoull(s, nullptr, 10) << 20;
    g_device = device_index;
    g_init = true;
    return AGH_OK;
}

int agh_shutdown(void) {
    std::lock_guard<std::recursive_mutex> lock(g_mutex);
    if (!g_init) return AGH_OK;
    AGH_HIP(hipStreamSynchronize(g_stream));
    AGH_HIP(hipStreamSynchronize(g_side));
    g_side_dirty = false;
    if (int rc = release_cached_blocks()) return rc;
    // blocks the caller still holds stay valid (and keep their capacity on record is pointless once the
    // library is down: a later agh_free after a new agh_init falls back to hipFree)
    g_live_blocks.clear();
    if (g_ws.ptr) AGH_HIP(hipFree(g_ws.ptr));
    if (g_ws_side.ptr) AGH_HIP(hipFree(g_ws_side.ptr));
    g_ws = Workspace();
    g_ws_side = Workspace();
    if (int rc = release_retired_workspaces()) return rc;
    for (int i = 0; i < kBranchEvents; ++i) {
        (void)hipEventDestroy(g_events[i]);
        (void)hipEventDestroy(g_capture_events[i]);
    }
    AGH_HIP(hipStreamDestroy(g_side));
    AGH_HIP(hipStreamDestroy(g_stream));
    g_stream = g_side = g_cur = nullptr;
    g_scratch_ptr = nullptr;
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
    if (g_capturing) return fail(AGH_EINVAL, "agh_malloc: not allowed while capturing a graph");
    // zero-length tensors are legal in the reference; they get a real 256-byte block
    const size_t cap = block_capacity(bytes);
    auto it = g_free_blocks.lower_bound(cap);
    if (it != g_free_blocks.end() && it->first == cap) {
        CachedBlock blk = it->second;
        g_free_blocks.erase(it);
        g_cached_bytes -= cap;
        // last used by a branch the main stream has not waited for: wait now
        if (g_cur == g_stream && blk.side_seq > g_side_joined_seq) {
            if (int rc = join_side()) return rc;
        }
        g_live_blocks[blk.ptr] = cap;
        *ptr = blk.ptr;
        return AGH_OK;
    }
    void *fresh = nullptr;
    hipError_t e = hipMalloc(&fresh, cap);
    if (e == hipErrorOutOfMemory) {  // give the cache back to the driver and try once more
        (void)hipGetLastError();
        if (int rc = release_cached_blocks()) return rc;
        e = hipMalloc(&fresh, cap);
    }
    if (e != hipSuccess) return hip_fail(e, "hipMalloc");
    g_live_blocks[fresh] = cap;
    *ptr = fresh;
    return AGH_OK;
}

int agh_free(void *ptr) {
    AGH_API_ENTER();
    if (!ptr) return AGH_OK;
    auto it = g_live_blocks.find(ptr);
    if (g_capturing) {
        // No wait, no driver call and no reuse inside a capture: the block is set aside and filed by agh_graph_end.
        // (Typical case: a host-side temporary dropped by the garbage collector while a step is being recorded.)
        if (it == g_live_blocks.end()) {
            g_deferred_frees.push_back(DeferredFree{ptr, 0});
        } else {
            g_deferred_frees.push_back(DeferredFree{ptr, it->second});
            g_live_blocks.erase(it);
        }
        return AGH_OK;
    }
    if (it == g_live_blocks.end()) {
        // not from this allocator's books (allocated before an agh_shutdown): hand it to the driver
        if (int rc = sync_all()) return rc;
        AGH_HIP(hipFree(ptr));
        return AGH_OK;
    }
    const size_t cap = it->second;
    g_live_blocks.erase(it);
    if (g_cached_bytes + cap > g_cache_limit) {
        if (int rc = release_cached_blocks()) return rc;  // waits for both streams
        if (cap > g_cache_limit) {
            AGH_HIP(hipFree(ptr));
            return AGH_OK;
        }
    }
    // No wait: kernels still queued on the main stream run before anything launched on the block later.
    g_free_blocks.emplace(cap, CachedBlock{ptr, g_side_dirty ? g_side_seq : 0});
    g_cached_bytes += cap;
    return AGH_OK;
}

int agh_cache_release(void) {
    AGH_API_ENTER();
    if (g_capturing) return fail(AGH_EINVAL, "agh_cache_release: not allowed while capturing a graph");
    if (int rc = release_cached_blocks()) return rc;  // waits for both streams
    if (g_live_graphs == 0) {  // no captured node names the workspaces: they can go too
        if (g_ws.ptr) AGH_HIP(hipFree(g_ws.ptr));
        if (g_ws_side.ptr) AGH_HIP(hipFree(g_ws_side.ptr));
        g_ws = Workspace();
        g_ws_side = Workspace();
        return release_retired_workspaces();
    }
    return AGH_OK;
}

int agh_cache_stats(size_t *cached_bytes, size_t *cached_blocks, size_t *live_blocks) {
    AGH_API_ENTER();
    if (cached_bytes) *cached_bytes = g_cached_bytes;
    if (cached_blocks) *cached_blocks = g_free_blocks.size();
    if (live_blocks) *live_blocks = g_live_blocks.size();
    return AGH_OK;
}

int agh_workspace_stats(size_t *workspace_bytes, size_t *retired_blocks) {
    AGH_API_ENTER();
    if (workspace_bytes) *workspace_bytes = g_ws.bytes + g_ws_side.bytes;
    if (retired_blocks) *retired_blocks = g_ws_retired.size();
    return AGH_OK;
}

int agh_memcpy_h2d(void *dst, const void *src, size_t bytes) {
    AGH_API_ENTER();
    if (bytes == 0) return AGH_OK;
    if (!dst || !src) return fail(AGH_ENULL, "agh_memcpy_h2d: null pointer");
    AGH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g_cur));
    return AGH_OK;
}

int agh_memcpy_d2h(void *dst, const void *src, size_t bytes) {
    AGH_API_ENTER();
    if (bytes == 0) return AGH_OK;
    if (!dst || !src) return fail(AGH_ENULL, "agh_memcpy_d2h: null pointer");
    if (g_capturing) return fail(AGH_EINVAL, "agh_memcpy_d2h: waits, not allowed while capturing (use agh_memcpy_d2h_async)");
    // the bytes may come from a branch that has not been joined: on the main stream, wait for it first
    if (g_cur == g_stream && g_side_dirty) {
        AGH_HIP(hipStreamSynchronize(g_side));
        g_side_joined_seq = g_side_seq;
        g_side_dirty = false;
    }
    AGH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, g_cur));
    AGH_HIP(hipStreamSynchronize(g_cur));
    return AGH_OK;
}

int agh_memcpy_d2d(void *dst, const void *src, size_t bytes) {
    AGH_API_ENTER();
    if (bytes == 0) return AGH_OK;
    if (!dst || !src) return fail(AGH_ENULL, "agh_memcpy_d2d: null pointer");
    AGH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, g_cur));
    return AGH_OK;
}

int agh_memcpy_d2h_async(void *dst, const void *src, size_t bytes) {
    AGH_API_ENTER();
    if (bytes == 0) return AGH_OK;
    if (!dst || !src) return fail(AGH_ENULL, "agh_memcpy_d2h_async: null pointer");
    AGH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, g_cur));
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
    if (int rc = sync_all()) return rc;
    AGH_HIP(hipHostFree(ptr));
    return AGH_OK;
}

int agh_graph_begin(void) {
    AGH_API_ENTER();
    if (g_capturing) return fail(AGH_EINVAL, "agh_graph_begin: already capturing");
    if (g_cur != g_stream) return fail(AGH_EINVAL, "agh_graph_begin: inside a branch");
    // work left on the branch stream is not part of the graph: the capture starts from a joined state
    if (int rc = join_side()) return rc;
    AGH_HIP(hipStreamBeginCapture(g_stream, hipStreamCaptureModeThreadLocal));
    g_capturing = true;
    return AGH_OK;
}

int agh_graph_end(void **graph_exec) {
    AGH_API_ENTER();
    if (!graph_exec) return fail(AGH_ENULL, "agh_graph_end: null out pointer");
    *graph_exec = nullptr;
    if (!g_capturing) return fail(AGH_EINVAL, "agh_graph_end: no capture in progress");
    hipGraph_t graph = nullptr;
    if (g_cur != g_stream) return fail(AGH_EINVAL, "agh_graph_end: still inside a branch");
    // an arm left open would make the capture invalid
    if (int rc = join_side()) {
        g_capturing = false;
        (void)hipStreamEndCapture(g_stream, &graph);
        if (graph) (void)hipGraphDestroy(graph);
        (void)flush_deferred_frees();
        return rc;
    }
    g_capturing = false;
    const hipError_t ec = hipStreamEndCapture(g_stream, &graph);
    if (ec != hipSuccess) {
        (void)flush_deferred_frees();
        return hip_fail(ec, "hipStreamEndCapture");
    }
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) {
        (void)flush_deferred_frees();
        return hip_fail(e, "hipGraphInstantiate");
    }
    ++g_live_graphs;
    *graph_exec = (void *)exec;
    return flush_deferred_frees();
}

int agh_graph_launch(void *graph_exec) {
    AGH_API_ENTER();
    if (!graph_exec) return fail(AGH_ENULL, "agh_graph_launch: null graph");
    if (g_capturing) return fail(AGH_EINVAL, "agh_graph_launch: not allowed while capturing a graph");
    if (g_cur != g_stream) return fail(AGH_EINVAL, "agh_graph_launch: inside a branch");
    // A graph captured with a branch names the branch stream's workspace in its fork arm; eager branch work that has
    // not been joined may still be using that block, so the replay is ordered behind it.
    if (int rc = join_side()) return rc;
    AGH_HIP(hipGraphLaunch((hipGraphExec_t)graph_exec, g_stream));
    return AGH_OK;
}

int agh_graph_destroy(void *graph_exec) {
    AGH_API_ENTER();
    if (!graph_exec) return AGH_OK;
    if (int rc = sync_all()) return rc;
    AGH_HIP(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
    if (g_live_graphs > 0 && --g_live_graphs == 0) return release_retired_workspaces();
    return AGH_OK;
}

int agh_sync(void) {
    AGH_API_ENTER();
    if (g_capturing) return fail(AGH_EINVAL, "agh_sync: not allowed while capturing a graph");
    return sync_all();
}

int agh_branch_begin(void) {
    AGH_API_ENTER();
    if (g_cur != g_stream) return fail(AGH_EINVAL, "agh_branch_begin: already inside a branch");
    hipEvent_t e = next_event();
    AGH_HIP(hipEventRecord(e, g_stream));
    AGH_HIP(hipStreamWaitEvent(g_side, e, 0));
    g_cur = g_side;
    g_side_dirty = true;
    ++g_side_seq;
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
    return join_side();
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
