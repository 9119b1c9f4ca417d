// Flat elementwise kernels: one skeleton, one float4 per thread, a grid that
// covers the data once, scalar tail folded into the same launch.  Every op is
// HBM-bound (4-12 bytes per element).  Measured on MI355X at 2^28 elements, a
// copy written this way streams 6.1 TB/s; the same copy as a capped grid-stride
// loop with four vectors in flight per thread reaches 4.3 TB/s, because the
// resident workgroups then touch addresses spread over the whole buffer instead
// of one moving window of DRAM pages.
//
// This file is compiled with -ffp-contract=off: the CPU oracle rounds after
// every multiply and add (cpp/core.hpp:414-469 built with -ffp-contract=off),
// and gfx950's fp32 mul/add/div/sqrt are IEEE correctly rounded, so the
// multiply-add chains here are bit-identical to the oracle.
#include "common.hpp"
#include "activations.hpp"

#include <cmath>

namespace jz {
namespace {

// ── functors ─────────────────────────────────────────────────────────────
struct FillF {
    float v;
    __device__ float operator()() const { return v; }
};
struct CopyF {
    __device__ float operator()(float x) const { return x; }
};
struct ExpF {
    __device__ float operator()(float x) const { return expf(x); }
};
struct LogF {
    __device__ float operator()(float x) const { return logf(x); }
};
struct TanhF {
    __device__ float operator()(float x) const { return tanhf(x); }
};
struct DTanhF {
    // cpp/matrix.hpp:300-302 evaluates 1 - tanh(x)*tanh(x) in double and narrows
    // on store; the subtraction cancels for |x| > 2, so fp32 would lose the
    // element's relative accuracy.  Same arithmetic here.
    __device__ float operator()(float x) const {
        const double t = tanh(static_cast<double>(x));
        return static_cast<float>(1.0 - t * t);
    }
};
struct SquareF {
    __device__ float operator()(float x) const { return x * x; }
};
struct AffineF {  // cpp/core.hpp:453-469: s1*x + b
    float s1, a;
    __device__ float operator()(float x) const { return s1 * x + a; }
};
struct EleminvF {  // cpp/core.hpp:472-482: double division, then narrowing
    double l;
    __device__ float operator()(float x) const { return static_cast<float>(l / static_cast<double>(x)); }
};
struct ReluF {  // ml/util.cuh:74-77
    __device__ float operator()(float x) const { return relu_f(x); }
};
struct DReluF {  // ml/util.cuh:79-82
    __device__ float operator()(float x) const { return drelu_f(x); }
};
struct SqrtF {  // cpp/juzhen.hpp:71-79
    __device__ float operator()(float x) const { return sqrtf(x); }
};
struct ClampF {  // ml/util.cuh:84-89
    float lo, hi;
    __device__ float operator()(float x) const { return x < lo ? lo : (x > hi ? hi : x); }
};
struct GeluF {  // 0.5*x*(1+erf(x/sqrt(2)))
    __device__ float operator()(float x) const { return gelu_f(x); }
};
struct AxpbyF {  // cpp/core.hpp:414-449: s1*a + s2*b
    float s1, s2;
    __device__ float operator()(float a, float b) const { return s1 * a + s2 * b; }
};
struct MseGradF {  // ml/layer.hpp:214-216: 2.0 * (input - output) / nb, each step rounded
    float inv_nb;
    __device__ float operator()(float pred, float target) const { return ((pred - target) * 2.0f) * inv_nb; }
};
struct HadamardF {  // cpp/matrix.hpp:428-474
    __device__ float operator()(float a, float b) const { return a * b; }
};
struct DReluMulF {  // hadmd(d_relu(pre), up): up * mask
    __device__ float operator()(float pre, float up) const { return up * drelu_f(pre); }
};
struct DGeluMulF {  // up * d/dx gelu(pre)
    __device__ float operator()(float x, float up) const { return up * dgelu_f(x); }
};

// ── kernels ──────────────────────────────────────────────────────────────
template <int NIN, class F>
__device__ __forceinline__ float apply1(const F& f, float a, float b) {
    if constexpr (NIN == 0) {
        return f();
    } else if constexpr (NIN == 1) {
        return f(a);
    } else {
        return f(a, b);
    }
}

template <int NIN, class F>
__device__ __forceinline__ float4 apply4(const F& f, const float4& a, const float4& b) {
    float4 r;
    r.x = apply1<NIN>(f, a.x, b.x);
    r.y = apply1<NIN>(f, a.y, b.y);
    r.z = apply1<NIN>(f, a.z, b.z);
    r.w = apply1<NIN>(f, a.w, b.w);
    return r;
}

// n4 float4 vectors followed by `tail` (<4) scalars; thread i owns vector i.
// NT: loads and stores with the non-temporal hint (launches that stream past the cache).
template <int NIN, class F, bool NT>
__global__ __launch_bounds__(kBlock) void ew_vec_kernel(F f, float* out, const float* a,
                                                        const float* b, size_t n4, int tail) {
    const size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i < n4) {
        float4 va, vb;
        if constexpr (NIN >= 1) va = load4<NT>(a + 4 * i);
        if constexpr (NIN >= 2) vb = load4<NT>(b + 4 * i);
        store4<NT>(out + 4 * i, apply4<NIN>(f, va, vb));
    }
    if (blockIdx.x == 0 && static_cast<int>(threadIdx.x) < tail) {
        const size_t j = n4 * 4 + threadIdx.x;
        float xa = 0.f, xb = 0.f;
        if constexpr (NIN >= 1) xa = a[j];
        if constexpr (NIN >= 2) xb = b[j];
        out[j] = apply1<NIN>(f, xa, xb);
    }
}

// Fallback for pointers that are not 16-byte aligned (sub-buffer views).
template <int NIN, class F>
__global__ __launch_bounds__(kBlock) void ew_scalar_kernel(F f, float* out, const float* a,
                                                           const float* b, size_t n) {
    const size_t stride = static_cast<size_t>(gridDim.x) * kBlock;
    for (size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) {
        float xa = 0.f, xb = 0.f;
        if constexpr (NIN >= 1) xa = a[i];
        if constexpr (NIN >= 2) xb = b[i];
        out[i] = apply1<NIN>(f, xa, xb);
    }
}

template <int NIN, class F>
int launch_ew(F f, float* out, const float* a, const float* b, size_t n) {
    if (n == 0) return 0;
    if (out == nullptr) return -1;
    if (NIN >= 1 && a == nullptr) return -1;
    if (NIN >= 2 && b == nullptr) return -1;
    const bool vec = aligned16(out) && (NIN < 1 || aligned16(a)) && (NIN < 2 || aligned16(b));
    hipStream_t s = stream();
    if (vec) {
        const size_t n4 = n / 4;
        const int tail = static_cast<int>(n % 4);
        const size_t blocks = n4 ? (n4 + kBlock - 1) / kBlock : 1;
        if (blocks > 0x7fffffffull) return -1;
        // distinct buffers of the launch (an in-place form keeps its one buffer in the cache
        // for twice as long); a fill is as fast without the hint
        const int buffers = 1 + (NIN >= 1 && a != out) + (NIN >= 2 && b != out && b != a);
        if (NIN >= 1 && streams_past_cache(buffers * n * sizeof(float)))
            ew_vec_kernel<NIN, F, true><<<static_cast<unsigned>(blocks), kBlock, 0, s>>>(f, out, a, b, n4, tail);
        else
            ew_vec_kernel<NIN, F, false><<<static_cast<unsigned>(blocks), kBlock, 0, s>>>(f, out, a, b, n4, tail);
    } else {
        const unsigned grid = grid_for(n, kBlock);
        ew_scalar_kernel<NIN, F><<<grid, kBlock, 0, s>>>(f, out, a, b, n);
    }
    return launch_rc();
}

}  // namespace
}  // namespace jz

using namespace jz;

JZ_API int jzhip_fill(float* dst, size_t count, float value) {
    return launch_ew<0>(FillF{value}, dst, nullptr, nullptr, count);
}
JZ_API int jzhip_copy(float* dst, const float* src, size_t count) {
    if (dst == src) return 0;
    return launch_ew<1>(CopyF{}, dst, src, nullptr, count);
}
JZ_API int jzhip_exp(float* out, const float* in, size_t count) {
    return launch_ew<1>(ExpF{}, out, in, nullptr, count);
}
JZ_API int jzhip_exp_inplace(float* x, size_t count) { return jzhip_exp(x, x, count); }
JZ_API int jzhip_log(float* out, const float* in, size_t count) {
    return launch_ew<1>(LogF{}, out, in, nullptr, count);
}
JZ_API int jzhip_log_inplace(float* x, size_t count) { return jzhip_log(x, x, count); }
JZ_API int jzhip_axpby(float* out, const float* a, const float* b, size_t count, float s1,
                       float s2) {
    return launch_ew<2>(AxpbyF{s1, s2}, out, a, b, count);
}
JZ_API int jzhip_affine(float* out, const float* in, size_t count, float s1, float a) {
    return launch_ew<1>(AffineF{s1, a}, out, in, nullptr, count);
}
JZ_API int jzhip_affine_inplace(float* x, size_t count, float s1, float a) {
    return jzhip_affine(x, x, count, s1, a);
}
JZ_API int jzhip_hadamard(float* out, const float* a, const float* b, size_t count) {
    return launch_ew<2>(HadamardF{}, out, a, b, count);
}
JZ_API int jzhip_hadamard_inplace(float* x, const float* other, size_t count) {
    return jzhip_hadamard(x, x, other, count);
}
JZ_API int jzhip_eleminv(float* out, const float* in, size_t count, double l) {
    return launch_ew<1>(EleminvF{l}, out, in, nullptr, count);
}
JZ_API int jzhip_eleminv_inplace(float* x, size_t count, float l) {
    return jzhip_eleminv(x, x, count, static_cast<double>(l));
}
JZ_API int jzhip_square(float* out, const float* in, size_t count) {
    return launch_ew<1>(SquareF{}, out, in, nullptr, count);
}
JZ_API int jzhip_square_inplace(float* x, size_t count) { return jzhip_square(x, x, count); }
JZ_API int jzhip_tanh(float* out, const float* in, size_t count) {
    return launch_ew<1>(TanhF{}, out, in, nullptr, count);
}
JZ_API int jzhip_tanh_inplace(float* x, size_t count) { return jzhip_tanh(x, x, count); }
JZ_API int jzhip_dtanh(float* out, const float* in, size_t count) {
    return launch_ew<1>(DTanhF{}, out, in, nullptr, count);
}
JZ_API int jzhip_dtanh_inplace(float* x, size_t count) { return jzhip_dtanh(x, x, count); }
JZ_API int jzhip_relu(float* out, const float* in, size_t count) {
    return launch_ew<1>(ReluF{}, out, in, nullptr, count);
}
JZ_API int jzhip_drelu(float* out, const float* in, size_t count) {
    return launch_ew<1>(DReluF{}, out, in, nullptr, count);
}
JZ_API int jzhip_sqrt(float* out, const float* in, size_t count) {
    return launch_ew<1>(SqrtF{}, out, in, nullptr, count);
}
JZ_API int jzhip_clamp(float* out, const float* in, size_t count, float lo, float hi) {
    return launch_ew<1>(ClampF{lo, hi}, out, in, nullptr, count);
}
JZ_API int jzhip_mse_grad(float* out, const float* pred, const float* target, size_t count, float inv_nb) {
    return launch_ew<2>(MseGradF{inv_nb}, out, pred, target, count);
}
JZ_API int jzhip_drelu_mul(float* out, const float* pre, const float* up, size_t count) {
    return launch_ew<2>(DReluMulF{}, out, pre, up, count);
}
JZ_API int jzhip_gelu(float* out, const float* in, size_t count) {
    return launch_ew<1>(GeluF{}, out, in, nullptr, count);
}
JZ_API int jzhip_dgelu_mul(float* out, const float* pre, const float* up, size_t count) {
    return launch_ew<2>(DGeluMulF{}, out, pre, up, count);
}
