// Runtime entry points: device memory for cgtGPU arrays, copies, streams,
// events, error reporting.
#include "common.h"
#include <algorithm>
#include <cstring>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace cgt_amd {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

void clear_error() { g_err[0] = 0; }

struct StreamWorkspaces {
    float* ptr[kWsUsers] = {};
    size_t bytes[kWsUsers] = {};
    bool in_graph[kWsUsers] = {};     // current block was current while a capture began: a graph may hold its address
    std::vector<void*> retired;       // outgrown, no graph can reference them: freed at the stream's next synchronize
    std::vector<void*> retired_kept;  // outgrown, possibly baked into a graph: freed with the stream
};
static std::mutex g_ws_mutex;
static std::unordered_map<void*, StreamWorkspaces> g_ws;

float* stream_workspace(void* stream, WorkspaceUser user, size_t bytes, const char* what) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    StreamWorkspaces& w = g_ws[stream];
    if (w.bytes[user] >= bytes) return w.ptr[user];
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(as_stream(stream), &cap) != hipSuccess) (void)hipGetLastError();
    if (cap != hipStreamCaptureStatusNone) {
        set_error("%s: the workspace would have to grow to %zu bytes while the stream is being captured; "
                  "run the sequence once on this stream before capturing it", what, bytes);
        return nullptr;
    }
    // Grow geometrically (at least 1.5 x the block that is outgrown): a caller whose shapes
    // rise call by call then retires O(log) blocks, not one per call.
    void* p = nullptr;
    size_t want = bytes < ((size_t)1 << 20) ? ((size_t)1 << 20) : bytes;
    const size_t geometric = w.bytes[user] + w.bytes[user] / 2;
    bool padded = geometric > want;
    if (padded) want = geometric;
    if (hipMalloc(&p, want) != hipSuccess && padded) {      // the padded request does not fit: the exact one may
        (void)hipGetLastError();
        want = bytes;
        p = nullptr;
        if (hipMalloc(&p, want) != hipSuccess) p = nullptr;
    }
    if (!p) {
        (void)hipGetLastError();
        set_error("%s: cannot allocate a workspace of %zu bytes", what, want);
        return nullptr;
    }
    if (w.ptr[user]) (w.in_graph[user] ? w.retired_kept : w.retired).push_back(w.ptr[user]);
    w.ptr[user] = static_cast<float*>(p);
    w.bytes[user] = want;
    w.in_graph[user] = false;
    return w.ptr[user];
}

// A capture begins on `stream`: whatever the graph records may hold the current blocks' addresses.
static void pin_stream_workspaces(void* stream) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    auto it = g_ws.find(stream);
    if (it == g_ws.end()) return;
    for (int u = 0; u < kWsUsers; ++u)
        if (it->second.ptr[u]) it->second.in_graph[u] = true;
}

// After `stream` (null: every stream) has been synchronized nothing in flight reads the
// outgrown blocks that no graph references: free them.
static void free_retired_workspaces(void* stream, bool all) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    for (auto& kv : g_ws) {
        if (!all && kv.first != stream) continue;
        for (void* p : kv.second.retired) (void)hipFree(p);
        kv.second.retired.clear();
    }
}

void release_stream_workspaces(void* stream) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    auto it = g_ws.find(stream);
    if (it == g_ws.end()) return;
    for (int u = 0; u < kWsUsers; ++u)
        if (it->second.ptr[u]) (void)hipFree(it->second.ptr[u]);
    for (void* p : it->second.retired) (void)hipFree(p);
    for (void* p : it->second.retired_kept) (void)hipFree(p);
    g_ws.erase(it);
}

// Device-to-device copy as a kernel: every workgroup streams its own contiguous region,
// UNROLL 16-byte loads in flight per lane (issued unconditionally from clamped indices),
// non-temporal 16-byte stores.  Head and tail bytes that are not whole aligned units go
// through a byte loop of the first workgroup.
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
template <int UNROLL>
__global__ __launch_bounds__(256) void stream_copy_kernel(const v4u* __restrict__ src, v4u* __restrict__ dst,
                                                          long units, long units_per_wg,
                                                          const unsigned char* __restrict__ src_bytes,
                                                          unsigned char* __restrict__ dst_bytes, long head, long tail_at,
                                                          long nbytes) {
    const long base = (long)blockIdx.x * units_per_wg;
    long end = base + units_per_wg;
    if (end > units) end = units;
    for (long u = base + threadIdx.x; u < end; u += 256 * UNROLL) {
        v4u v[UNROLL];
#pragma unroll
        for (int i = 0; i < UNROLL; ++i) {
            long idx = u + (long)i * 256;
            v[i] = __builtin_nontemporal_load(src + (idx < end ? idx : end - 1));
        }
#pragma unroll
        for (int i = 0; i < UNROLL; ++i) {
            long idx = u + (long)i * 256;
            if (idx < end) __builtin_nontemporal_store(v[i], dst + idx);
        }
    }
    if (blockIdx.x == 0) {
        for (long i = threadIdx.x; i < head; i += 256) dst_bytes[i] = src_bytes[i];
        for (long i = tail_at + threadIdx.x; i < nbytes; i += 256) dst_bytes[i] = src_bytes[i];
    }
}

// Region per workgroup and loads in flight of the copy kernel (units of 16 bytes); settable
// for measurement through cgt_amd_stream_copy_tune.
// Measured on 1 GiB (and the same order at 256 MiB and 103 MiB): 16 KiB regions with 4 loads
// in flight 6.0-6.3 TB/s, 64 KiB with 8 in flight 5.5-5.7, 1 MiB regions 5.4; the runtime's own
// device-to-device memcpy 4.8 TB/s.  Many short-lived workgroups beat few long-lived ones.
static long g_copy_units_per_wg = 1024;     // 16 KiB
static int g_copy_unroll = 4;

int launch_stream_copy(void* dest, const void* src, long nbytes, void* stream) {
    const unsigned char* s8 = static_cast<const unsigned char*>(src);
    unsigned char* d8 = static_cast<unsigned char*>(dest);
    // whole units where source and destination are 16-byte aligned together
    long head = (16 - (long)((uintptr_t)d8 & 15)) & 15;
    if (head > nbytes) head = nbytes;
    long units = 0;
    if ((((uintptr_t)(s8 + head)) & 15) == 0) units = (nbytes - head) / 16;
    else head = 0;
    const long tail_at = head + units * 16;
    long per = g_copy_units_per_wg;
    long blocks = units > 0 ? cdiv(units, per) : 1;
    const v4u* sv = reinterpret_cast<const v4u*>(s8 + head);
    v4u* dv = reinterpret_cast<v4u*>(d8 + head);
    dim3 grid((unsigned)blocks), block(256);
    hipStream_t st = as_stream(stream);
    switch (g_copy_unroll) {
        case 4: stream_copy_kernel<4><<<grid, block, 0, st>>>(sv, dv, units, per, s8, d8, head, tail_at, nbytes); break;
        case 16: stream_copy_kernel<16><<<grid, block, 0, st>>>(sv, dv, units, per, s8, d8, head, tail_at, nbytes); break;
        default: stream_copy_kernel<8><<<grid, block, 0, st>>>(sv, dv, units, per, s8, d8, head, tail_at, nbytes); break;
    }
    CGT_LAUNCH_CHECK("stream_copy");
    return CGT_AMD_OK;
}

// A workgroup fills 4096 words: the words before the first 16-byte boundary and after the last one
// singly (first workgroup), the rest as aligned 16-byte units, four per thread.
__global__ __launch_bounds__(256) void fill_u32_kernel(unsigned int* __restrict__ dst, unsigned int v, long n, long head, long units) {
    v4u* body = reinterpret_cast<v4u*>(dst + head);
    const v4u q = {v, v, v, v};
    const long u0 = (long)blockIdx.x * 1024 + threadIdx.x;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const long u = u0 + k * 256;
        if (u < units) body[u] = q;
    }
    if (blockIdx.x == 0) {
        for (long i = threadIdx.x; i < head; i += 256) dst[i] = v;
        for (long i = head + 4 * units + threadIdx.x; i < n; i += 256) dst[i] = v;
    }
}

}  // namespace cgt_amd

using namespace cgt_amd;

CGT_API int cgt_amd_version(void) { return 100; }

CGT_API const char* cgt_amd_last_error(void) { return g_err; }

CGT_API int cgt_amd_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

CGT_API int cgt_amd_device_name(char* buf, int buflen) {
    CGT_ARG_CHECK(buf && buflen > 0, "device_name: bad buffer");
    int dev = 0;
    CGT_HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    CGT_HIP_TRY(hipGetDeviceProperties(&prop, dev));
    snprintf(buf, buflen, "%s %s CUs=%d clock=%dMHz", prop.gcnArchName, prop.name,
             prop.multiProcessorCount, prop.clockRate / 1000);
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_mem_info(long* free_bytes, long* total_bytes) {
    CGT_ARG_CHECK(free_bytes && total_bytes, "mem_info: null pointer");
    size_t f = 0, t = 0;
    CGT_HIP_TRY(hipMemGetInfo(&f, &t));
    *free_bytes = (long)f;
    *total_bytes = (long)t;
    return CGT_AMD_OK;
}

CGT_API void* cgt_amd_alloc(long nbytes) {
    if (nbytes < 0) {
        set_error("alloc: negative size %ld", nbytes);
        return nullptr;
    }
    void* p = nullptr;
    // A zero-byte array still needs a distinct non-null pointer.
    hipError_t e = hipMalloc(&p, nbytes > 0 ? (size_t)nbytes : 16);
    if (e != hipSuccess) {
        set_error("hipMalloc(%ld) failed: %s", nbytes, hipGetErrorString(e));
        return nullptr;
    }
    return p;
}

CGT_API int cgt_amd_free(void* ptr) {
    if (!ptr) return CGT_AMD_OK;
    CGT_HIP_TRY(hipFree(ptr));
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_memcpy(int dest_devtype, int src_devtype, void* dest, const void* src,
                           long nbytes) {
    CGT_ARG_CHECK(nbytes >= 0, "memcpy: negative size");
    if (nbytes == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(dest && src, "memcpy: null pointer");
    if (dest_devtype == CGT_AMD_CPU && src_devtype == CGT_AMD_CPU) {
        memcpy(dest, src, (size_t)nbytes);
        return CGT_AMD_OK;
    }
    hipMemcpyKind kind;
    if (src_devtype == CGT_AMD_CPU && dest_devtype == CGT_AMD_GPU) kind = hipMemcpyHostToDevice;
    else if (src_devtype == CGT_AMD_GPU && dest_devtype == CGT_AMD_CPU) kind = hipMemcpyDeviceToHost;
    else if (src_devtype == CGT_AMD_GPU && dest_devtype == CGT_AMD_GPU) kind = hipMemcpyDeviceToDevice;
    else {
        set_error("memcpy: invalid devtypes %d <- %d", dest_devtype, src_devtype);
        return CGT_AMD_ERR_ARG;
    }
    CGT_HIP_TRY(hipMemcpy(dest, src, (size_t)nbytes, kind));
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_memcpy_async(int dest_devtype, int src_devtype, void* dest, const void* src,
                                 long nbytes, void* stream) {
    CGT_ARG_CHECK(nbytes >= 0, "memcpy_async: negative size");
    if (nbytes == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(dest && src, "memcpy_async: null pointer");
    hipMemcpyKind kind;
    if (src_devtype == CGT_AMD_CPU && dest_devtype == CGT_AMD_GPU) kind = hipMemcpyHostToDevice;
    else if (src_devtype == CGT_AMD_GPU && dest_devtype == CGT_AMD_CPU) kind = hipMemcpyDeviceToHost;
    else if (src_devtype == CGT_AMD_GPU && dest_devtype == CGT_AMD_GPU) kind = hipMemcpyDeviceToDevice;
    else {
        set_error("memcpy_async: invalid devtypes %d <- %d", dest_devtype, src_devtype);
        return CGT_AMD_ERR_ARG;
    }
    if (kind == hipMemcpyDeviceToDevice) {
        // the library's own copy kernel where the ranges are disjoint (it streams faster than
        // the runtime's copy here); overlapping ranges keep memmove semantics through the runtime
        const unsigned char* s8 = static_cast<const unsigned char*>(src);
        unsigned char* d8 = static_cast<unsigned char*>(dest);
        if (d8 + nbytes <= s8 || s8 + nbytes <= d8) return launch_stream_copy(dest, src, nbytes, stream);
    }
    CGT_HIP_TRY(hipMemcpyAsync(dest, src, (size_t)nbytes, kind, as_stream(stream)));
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_stream_copy(void* dest, const void* src, long nbytes, void* stream) {
    CGT_ARG_CHECK(nbytes >= 0, "stream_copy: negative size");
    if (nbytes == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(dest && src, "stream_copy: null pointer");
    const unsigned char* s8 = static_cast<const unsigned char*>(src);
    unsigned char* d8 = static_cast<unsigned char*>(dest);
    CGT_ARG_CHECK(d8 + nbytes <= s8 || s8 + nbytes <= d8, "stream_copy: source and destination overlap");
    return launch_stream_copy(dest, src, nbytes, stream);
}

CGT_API int cgt_amd_stream_copy_tune(long bytes_per_workgroup, int loads_in_flight) {
    CGT_ARG_CHECK(bytes_per_workgroup >= 4096 && bytes_per_workgroup % 4096 == 0,
                  "stream_copy_tune: the region of a workgroup is a multiple of 4096 bytes");
    CGT_ARG_CHECK(loads_in_flight == 4 || loads_in_flight == 8 || loads_in_flight == 16,
                  "stream_copy_tune: 4, 8 or 16 loads in flight");
    g_copy_units_per_wg = bytes_per_workgroup / 16;
    g_copy_unroll = loads_in_flight;
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_fill_u32(void* dst, unsigned int value, long count, void* stream) {
    CGT_ARG_CHECK(count >= 0, "fill: negative count");
    if (count == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(dst, "fill: null pointer");
    CGT_ARG_CHECK(reinterpret_cast<uintptr_t>(dst) % 4 == 0, "fill: the destination must be 4-byte aligned");
    long head = (long)((16 - (reinterpret_cast<uintptr_t>(dst) & 15)) & 15) / 4;
    if (head > count) head = count;
    const long units = (count - head) / 4;
    const long blocks = std::max(1L, cdiv(units, 1024L));
    CGT_ARG_CHECK(blocks < (1L << 31), "fill: too many words");
    fill_u32_kernel<<<dim3((unsigned)blocks), dim3(256), 0, as_stream(stream)>>>(
        static_cast<unsigned int*>(dst), value, count, head, units);
    CGT_LAUNCH_CHECK("fill_u32");
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_synchronize(void* stream) {
    if (stream) CGT_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    else CGT_HIP_TRY(hipDeviceSynchronize());
    free_retired_workspaces(stream, stream == nullptr);
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_stream_create(void** stream) {
    CGT_ARG_CHECK(stream, "stream_create: null");
    hipStream_t s;
    CGT_HIP_TRY(hipStreamCreate(&s));  // default priority only
    *stream = s;
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_stream_destroy(void* stream) {
    if (!stream) return CGT_AMD_OK;
    // the stream's work may still use its workspaces: drain it before they go
    CGT_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    release_stream_workspaces(stream);
    CGT_HIP_TRY(hipStreamDestroy(as_stream(stream)));
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_event_create(void** event) {
    CGT_ARG_CHECK(event, "event_create: null");
    hipEvent_t e;
    CGT_HIP_TRY(hipEventCreate(&e));
    *event = e;
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_event_destroy(void* event) {
    if (event) CGT_HIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(event)));
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_event_record(void* event, void* stream) {
    CGT_ARG_CHECK(event, "event_record: null");
    CGT_HIP_TRY(hipEventRecord(static_cast<hipEvent_t>(event), as_stream(stream)));
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_stream_wait_event(void* stream, void* event) {
    CGT_ARG_CHECK(event, "stream_wait_event: null event");
    CGT_HIP_TRY(hipStreamWaitEvent(as_stream(stream), static_cast<hipEvent_t>(event), 0));
    return CGT_AMD_OK;
}

// ---- stream capture: a fixed sequence of launches recorded once, replayed as one graph

CGT_API int cgt_amd_graph_capture_begin(void* stream) {
    CGT_ARG_CHECK(stream, "graph_capture_begin: needs a created stream (the default stream cannot be captured)");
    pin_stream_workspaces(stream);
    CGT_HIP_TRY(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal));
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_graph_capture_end(void* stream, void** graph_exec) {
    CGT_ARG_CHECK(stream && graph_exec, "graph_capture_end: null");
    hipGraph_t graph = nullptr;
    CGT_HIP_TRY(hipStreamEndCapture(as_stream(stream), &graph));
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) {
        set_error("hipGraphInstantiate failed: %s", hipGetErrorString(e));
        return CGT_AMD_ERR_HIP;
    }
    *graph_exec = exec;
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_graph_launch(void* graph_exec, void* stream) {
    CGT_ARG_CHECK(graph_exec, "graph_launch: null graph");
    CGT_HIP_TRY(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), as_stream(stream)));
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_graph_destroy(void* graph_exec) {
    if (graph_exec) CGT_HIP_TRY(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec)));
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_event_elapsed_ms(void* start, void* stop, float* ms) {
    CGT_ARG_CHECK(start && stop && ms, "event_elapsed: null");
    CGT_HIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
    CGT_HIP_TRY(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
    return CGT_AMD_OK;
}
