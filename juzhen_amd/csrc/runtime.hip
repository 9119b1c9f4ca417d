// Runtime entry points: device query, memory, copies, stream selection.
// Replaces the allocation/copy half of the reference's device API
// (cpp/hipkernels.cpp:463-569) without rocRAND/hipBLAS handles.
#include "common.hpp"

#include <atomic>
#include <mutex>

namespace jz {

namespace {
std::atomic<hipStream_t> g_stream{nullptr};
std::atomic<int> g_cus{0};
std::atomic<float*> g_workspace{nullptr};
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
    float* w = g_workspace.load(std::memory_order_acquire);
    if (w) return w;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    w = g_workspace.load(std::memory_order_acquire);
    if (w) return w;
    void* p = nullptr;
    if (hipMalloc(&p, kWorkspaceFloats * sizeof(float)) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    g_workspace.store(static_cast<float*>(p), std::memory_order_release);
    return static_cast<float*>(p);
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

JZ_API int jzhip_set_stream(void* hip_stream) {
    jz::g_stream.store(static_cast<hipStream_t>(hip_stream), std::memory_order_relaxed);
    return 0;
}
JZ_API void* jzhip_get_stream(void) { return jz::stream(); }

JZ_API int jzhip_synchronize(void) { return jz::rc_of(hipStreamSynchronize(jz::stream())); }

JZ_API size_t jzhip_workspace_bytes(void) {
    return jz::g_workspace.load(std::memory_order_acquire) ? jz::kWorkspaceFloats * sizeof(float) : 0;
}
