// Activation functions shared by the elementwise kernels and the GEMM epilogue,
// so that a fused product rounds exactly like the separate passes it replaces.
#pragma once
#include <hip/hip_runtime.h>

namespace jz {

// ml/util.cuh:74-77
__device__ __forceinline__ float relu_f(float x) { return x > 0.0f ? x : 0.0f; }
// ml/util.cuh:79-82
__device__ __forceinline__ float drelu_f(float x) { return x > 0.0f ? 1.0f : 0.0f; }
// 0.5*x*(1+erf(x/sqrt(2)))
__device__ __forceinline__ float gelu_f(float x) {
    return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}
// d/dx gelu(x) = Phi(x) + x*phi(x)
__device__ __forceinline__ float dgelu_f(float x) {
    const float cdf = 0.5f * (1.0f + erff(x * 0.70710678118654752440f));
    const float pdf = 0.39894228040143267794f * expf(-0.5f * x * x);
    return cdf + x * pdf;
}

}  // namespace jz
