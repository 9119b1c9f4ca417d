// Activation functions shared by the elementwise kernels and the GEMM epilogue,
// so that a fused product rounds exactly like the separate passes it replaces.
#pragma once
#include <hip/hip_runtime.h>

namespace jz {

// ml/util.cuh:74-77
__device__ __forceinline__ float relu_f(float x) { return x > 0.0f ? x : 0.0f; }
// ml/util.cuh:79-82
__device__ __forceinline__ float drelu_f(float x) { return x > 0.0f ? 1.0f : 0.0f; }
// GELU in its exact (erf) form, x*Phi(x), and its derivative Phi(x) + x*phi(x).
// Phi is evaluated as a complementary error function of the Abramowitz-Stegun
// 7.1.26 shape, erfc(z) = t*P(t)*exp(-z^2) with t = 1/(1 + p*z), z = |x|/sqrt(2),
// with P refitted at degree 5 (p = 0.55) against erfcx so that x*Phi(x) stays
// within fp32 rounding of the closed form (4e-7 absolute on |x| <= 9) and the
// derivative within 2e-7: one reciprocal, one hardware exp2 and seven fused
// multiply-adds, against a branchy erff plus an expf.  The exponential is shared
// by Phi and phi, so the derivative costs two more multiplies.  The GEMM tails
// evaluate this per stored element; erff there cost 19-50 us per product.
struct GeluParts {
    float cdf;   // Phi(x)
    float e;     // exp(-x^2/2)
};
__device__ __forceinline__ GeluParts gelu_parts(float x) {
    const float ax = fabsf(x);
    const float z = ax * 0.70710678118654752440f;
    const float t = __builtin_amdgcn_rcpf(fmaf(0.55f, z, 1.0f));
    float pl = 0.107399047f;
    pl = fmaf(pl, t, -0.518342501f);
    pl = fmaf(pl, t, 0.760207088f);
    pl = fmaf(pl, t, -0.041821785f);
    pl = fmaf(pl, t, 0.390999575f);
    pl = fmaf(pl, t, 0.301558593f);
    // exp(-x^2/2) = exp2(-x^2 * log2(e)/2); far tails underflow to an exact zero
    const float e = __builtin_amdgcn_exp2f(-0.72134752044448170368f * (x * x));
    const float half_erfc = 0.5f * (pl * t) * e;
    GeluParts r;
    r.cdf = x >= 0.0f ? 1.0f - half_erfc : half_erfc;
    r.e = e;
    return r;
}
__device__ __forceinline__ float gelu_f(float x) { return x * gelu_parts(x).cdf; }
__device__ __forceinline__ float dgelu_f(float x) {
    const GeluParts g = gelu_parts(x);
    return g.cdf + x * (0.39894228040143267794f * g.e);
}

}  // namespace jz
