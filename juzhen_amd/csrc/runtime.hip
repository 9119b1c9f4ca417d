// Runtime entry points: device query, memory, copies, stream selection.
// Replaces the allocation/copy half of the reference's device API
// (cpp/hipkernels.cpp:463-569) without rocRAND/hipBLAS handles.
#include "common.hpp"

#include <cstdint>

#include <algorithm>
#include <atomic>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace jz {

namespace {
std::atomic<hipStream_t> g_stream{nullptr};
std::atomic<int> g_cus{0};
// One workspace per stream that has asked for one: launches on different
// streams may run concurrently and must not share partial-result storage.  A
// slot is given back when its stream is destroyed through jzhip_stream_destroy.
constexpr int kMaxWorkspaces = 64;
struct WorkspaceSlot {
    std::atomic<float*> ptr{nullptr};   // nullptr: slot free
    std::atomic<hipStream_t> owner{nullptr};   // read by the lock-free scan while a slot is being reused
};
WorkspaceSlot g_ws[kMaxWorkspaces];
std::atomic<int> g_ws_count{0};         // slots ever used (scan bound)
std::mutex g_ws_mutex;
}  // namespace

hipStream_t stream() { return g_stream.load(std::memory_order_relaxed); }

int num_cus() {
    int c = g_cus.load(std::memory_order_relaxed);
    if (c > 0) return c;
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) {
        (void)hipGetLastError();
        return 256;  // MI355X; only used to size grids
    }
    c = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    g_cus.store(c, std::memory_order_relaxed);
    return c;
}

float* workspace() {
    const hipStream_t s = stream();
    const int n = g_ws_count.load(std::memory_order_acquire);
    for (int i = 0; i < n; ++i) {
        float* p = g_ws[i].ptr.load(std::memory_order_acquire);
        if (p && g_ws[i].owner.load(std::memory_order_acquire) == s) return p;
    }
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    const int m = g_ws_count.load(std::memory_order_acquire);
    int slot = -1;
    for (int i = 0; i < m; ++i) {
        float* p = g_ws[i].ptr.load(std::memory_order_acquire);
        if (p && g_ws[i].owner.load(std::memory_order_acquire) == s) return p;
        if (!p && slot < 0) slot = i;
    }
    if (slot < 0) {
        if (m == kMaxWorkspaces) return nullptr;
        slot = m;
    }
    void* p = nullptr;
    if (hipMalloc(&p, kWorkspaceFloats * sizeof(float)) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    g_ws[slot].owner.store(s, std::memory_order_release);
    g_ws[slot].ptr.store(static_cast<float*>(p), std::memory_order_release);
    if (slot == m) g_ws_count.store(m + 1, std::memory_order_release);
    return static_cast<float*>(p);
}

// The stream is going away: wait for it and free its workspace.
int release_workspace(hipStream_t s) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    const int m = g_ws_count.load(std::memory_order_acquire);
    for (int i = 0; i < m; ++i) {
        float* p = g_ws[i].ptr.load(std::memory_order_acquire);
        if (p && g_ws[i].owner.load(std::memory_order_acquire) == s) {
            int rc = rc_of(hipStreamSynchronize(s));
            g_ws[i].ptr.store(nullptr, std::memory_order_release);
            const int rc2 = rc_of(hipFree(p));
            return rc ? rc : rc2;
        }
    }
    return 0;
}

size_t workspace_total_bytes() {
    size_t n = 0;
    const int m = g_ws_count.load(std::memory_order_acquire);
    for (int i = 0; i < m; ++i)
        if (g_ws[i].ptr.load(std::memory_order_acquire)) n += kWorkspaceFloats * sizeof(float);
    return n;
}

}  // namespace jz

JZ_API int jzhip_version(void) { return 100; }

JZ_API int jzhip_runtime_available(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n > 0 ? 1 : 0;
}

JZ_API const char* jzhip_error_string(int rc) {
    if (rc == 0) return "success";
    if (rc == -1) return "jzhip: invalid argument";
    if (rc == -2) return "jzhip: workspace allocation failed";
    if (rc == -3) return "jzhip: size exceeds the fixed scratch of the no-allocation entry point";
    return hipGetErrorString(static_cast<hipError_t>(rc));
}

JZ_API int jzhip_num_compute_units(void) {
    if (!jzhip_runtime_available()) return 0;
    return jz::num_cus();
}

JZ_API int jzhip_malloc(float** ptr, size_t count) {
    if (ptr == nullptr) return -1;
    *ptr = nullptr;
    if (count == 0) count = 1;
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, count * sizeof(float));
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return static_cast<int>(e);
    }
    *ptr = static_cast<float*>(p);
    return 0;
}

JZ_API int jzhip_free(float* ptr) {
    if (ptr == nullptr) return 0;
    return jz::rc_of(hipFree(ptr));
}

namespace {
constexpr size_t kKernelCopyBytes = size_t(1) << 20;
int sync_copy(void* dst, const void* src, size_t count, hipMemcpyKind kind) {
    if (count == 0) return 0;
    if (dst == nullptr || src == nullptr) return -1;
    hipStream_t s = jz::stream();
    hipError_t e = hipMemcpyAsync(dst, src, count * sizeof(float), kind, s);
    if (e != hipSuccess) return static_cast<int>(e);
    return jz::rc_of(hipStreamSynchronize(s));
}
}  // namespace

JZ_API int jzhip_memcpy_h2d(float* dst_device, const float* src_host, size_t count) {
    return sync_copy(dst_device, src_host, count, hipMemcpyHostToDevice);
}
JZ_API int jzhip_memcpy_d2h(float* dst_host, const float* src_device, size_t count) {
    return sync_copy(dst_host, src_device, count, hipMemcpyDeviceToHost);
}
JZ_API int jzhip_memcpy_d2d(float* dst_device, const float* src_device, size_t count) {
    // Device-to-device copies stay asynchronous: a copy kernel keeps stream
    // order and does not stall the host the way hipMemcpy does.
    return jzhip_copy(dst_device, src_device, count);
}

JZ_API int jzhip_host_alloc(void** ptr, size_t bytes) {
    if (ptr == nullptr) return -1;
    *ptr = nullptr;
    if (bytes == 0) bytes = 1;
    void* p = nullptr;
    hipError_t e = hipHostMalloc(&p, bytes, hipHostMallocDefault);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return static_cast<int>(e);
    }
    *ptr = p;
    return 0;
}
JZ_API int jzhip_host_free(void* ptr) {
    if (ptr == nullptr) return 0;
    return jz::rc_of(hipHostFree(ptr));
}
JZ_API int jzhip_memcpy_h2d_async(void* dst_device, const void* src_host, size_t bytes) {
    if (bytes == 0) return 0;
    if (dst_device == nullptr || src_host == nullptr) return -1;
    // A small copy from page-locked memory (a batch of ids) is done by a kernel
    // that reads the host buffer through its device alias: it stays on the
    // compute queue, where a DMA copy between kernels costs a hand-over to the
    // copy engine and back that is far longer than the transfer.
    if (bytes <= kKernelCopyBytes && bytes % sizeof(float) == 0 &&
        reinterpret_cast<uintptr_t>(dst_device) % sizeof(float) == 0 &&
        reinterpret_cast<uintptr_t>(src_host) % sizeof(float) == 0) {
        hipPointerAttribute_t at;
        if (hipPointerGetAttributes(&at, src_host) == hipSuccess && at.type == hipMemoryTypeHost &&
            at.devicePointer != nullptr)
            return jzhip_copy(static_cast<float*>(dst_device), static_cast<const float*>(at.devicePointer),
                              bytes / sizeof(float));
        (void)hipGetLastError();   // pageable memory is not known to the runtime: not an error here
    }
    return jz::rc_of(hipMemcpyAsync(dst_device, src_host, bytes, hipMemcpyHostToDevice, jz::stream()));
}
JZ_API int jzhip_memcpy_d2h_async(void* dst_host, const void* src_device, size_t bytes) {
    if (bytes == 0) return 0;
    if (dst_host == nullptr || src_device == nullptr) return -1;
    return jz::rc_of(hipMemcpyAsync(dst_host, src_device, bytes, hipMemcpyDeviceToHost, jz::stream()));
}

// ── recording a sequence of calls and replaying it as one graph launch ───────
namespace {
std::mutex g_graph_mutex;
hipStream_t g_record_stream = nullptr;   // created on first use, lives until the process ends
hipStream_t g_stream_before = nullptr;   // the current stream when recording began
std::atomic<int> g_recording{0};
// the streams every recorded graph has been replayed on since it was made: a
// replay runs on the current stream of its launch, never on the record stream,
// and destroying the executable graph must wait for those
std::unordered_map<void*, std::vector<hipStream_t>> g_replay_streams;
}  // namespace

JZ_API int jzhip_graph_begin(void) {
    std::lock_guard<std::mutex> lock(g_graph_mutex);
    if (g_recording.load(std::memory_order_acquire)) return -1;
    if (!g_record_stream) {
        // a blocking stream of default priority: it keeps the implicit ordering with the null stream
        int rc = jz::rc_of(hipStreamCreateWithFlags(&g_record_stream, hipStreamDefault));
        if (rc) return rc;
    }
    g_stream_before = jz::stream();
    int rc = jz::rc_of(hipStreamSynchronize(g_stream_before));
    if (rc) return rc;
    jz::g_stream.store(g_record_stream, std::memory_order_relaxed);
    // the recording stream's workspace must exist before recording starts
    if (!jz::workspace()) {
        jz::g_stream.store(g_stream_before, std::memory_order_relaxed);
        return -2;
    }
    rc = jz::rc_of(hipStreamBeginCapture(g_record_stream, hipStreamCaptureModeRelaxed));
    if (rc) {
        jz::g_stream.store(g_stream_before, std::memory_order_relaxed);
        return rc;
    }
    g_recording.store(1, std::memory_order_release);
    return 0;
}

JZ_API int jzhip_graph_end(void** out_graph) {
    std::lock_guard<std::mutex> lock(g_graph_mutex);
    if (!g_recording.load(std::memory_order_acquire)) return -1;
    hipGraph_t graph = nullptr;
    int rc = jz::rc_of(hipStreamEndCapture(g_record_stream, &graph));
    g_recording.store(0, std::memory_order_release);
    jz::g_stream.store(g_stream_before, std::memory_order_relaxed);
    if (rc) return rc;
    if (!out_graph) {
        (void)hipGraphDestroy(graph);
        return -1;
    }
    hipGraphExec_t exec = nullptr;
    rc = jz::rc_of(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
    (void)hipGraphDestroy(graph);
    if (rc) return rc;
    *out_graph = exec;
    return 0;
}

JZ_API int jzhip_graph_recording(void) { return g_recording.load(std::memory_order_acquire); }

JZ_API int jzhip_graph_launch(void* graph) {
    if (!graph || g_recording.load(std::memory_order_acquire)) return -1;
    // on the current stream, the null stream included
    const hipStream_t s = jz::stream();
    {
        std::lock_guard<std::mutex> lock(g_graph_mutex);
        std::vector<hipStream_t>& used = g_replay_streams[graph];
        if (std::find(used.begin(), used.end(), s) == used.end()) used.push_back(s);
    }
    return jz::rc_of(hipGraphLaunch(static_cast<hipGraphExec_t>(graph), s));
}

JZ_API int jzhip_graph_destroy(void* graph) {
    if (!graph) return 0;
    if (g_recording.load(std::memory_order_acquire)) return -1;   // a wait would break the recording
    // Replays may still be running on the streams they were launched on; their
    // kernels read the executable graph's argument storage and the buffers the
    // caller frees next, so wait for every such stream before the graph goes.
    std::vector<hipStream_t> used;
    {
        std::lock_guard<std::mutex> lock(g_graph_mutex);
        auto it = g_replay_streams.find(graph);
        if (it != g_replay_streams.end()) {
            used.swap(it->second);
            g_replay_streams.erase(it);
        }
    }
    int rc = 0;
    for (hipStream_t s : used) {
        const int r = jz::rc_of(hipStreamSynchronize(s));
        if (r && !rc) rc = r;
    }
    const int rc2 = jz::rc_of(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph)));
    return rc ? rc : rc2;
}

JZ_API int jzhip_set_stream(void* hip_stream) {
    if (g_recording.load(std::memory_order_acquire)) return -1;   // the recording owns the current stream
    jz::g_stream.store(static_cast<hipStream_t>(hip_stream), std::memory_order_relaxed);
    return 0;
}
JZ_API void* jzhip_get_stream(void) { return jz::stream(); }

JZ_API int jzhip_synchronize(void) { return jz::rc_of(hipStreamSynchronize(jz::stream())); }

JZ_API size_t jzhip_workspace_bytes(void) { return jz::workspace_total_bytes(); }

JZ_API int jzhip_stream_create(void** out_stream) {
    if (!out_stream) return -1;
    hipStream_t s = nullptr;
    // default priority; non-blocking so that it does not serialise against the null stream
    const int rc = jz::rc_of(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *out_stream = rc ? nullptr : s;
    return rc;
}
JZ_API int jzhip_stream_destroy(void* hip_stream) {
    if (!hip_stream) return 0;
    if (jz::stream() == static_cast<hipStream_t>(hip_stream)) jzhip_set_stream(nullptr);
    int rc = jz::release_workspace(static_cast<hipStream_t>(hip_stream));
    // replays launched on this stream must be over before its handle goes stale
    // in the per-graph lists jzhip_graph_destroy walks
    bool listed = false;
    {
        std::lock_guard<std::mutex> lock(g_graph_mutex);
        for (auto& kv : g_replay_streams) {
            auto& v = kv.second;
            auto it = std::find(v.begin(), v.end(), static_cast<hipStream_t>(hip_stream));
            if (it != v.end()) {
                v.erase(it);
                listed = true;
            }
        }
    }
    if (listed) {
        const int r = jz::rc_of(hipStreamSynchronize(static_cast<hipStream_t>(hip_stream)));
        if (r && !rc) rc = r;
    }
    const int rc2 = jz::rc_of(hipStreamDestroy(static_cast<hipStream_t>(hip_stream)));
    return rc ? rc : rc2;
}
JZ_API int jzhip_event_create(void** out_event) {
    if (!out_event) return -1;
    hipEvent_t e = nullptr;
    const int rc = jz::rc_of(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    *out_event = rc ? nullptr : e;
    return rc;
}
JZ_API int jzhip_event_destroy(void* event) {
    if (!event) return 0;
    return jz::rc_of(hipEventDestroy(static_cast<hipEvent_t>(event)));
}
JZ_API int jzhip_event_record(void* event) {
    if (!event) return -1;
    return jz::rc_of(hipEventRecord(static_cast<hipEvent_t>(event), jz::stream()));
}
JZ_API int jzhip_event_synchronize(void* event) {
    if (!event) return -1;
    return jz::rc_of(hipEventSynchronize(static_cast<hipEvent_t>(event)));
}
JZ_API int jzhip_stream_wait_event(void* event) {
    if (!event) return -1;
    return jz::rc_of(hipStreamWaitEvent(jz::stream(), static_cast<hipEvent_t>(event), 0));
}
