// ROCm hook for ml/util.cuh: include at the very end of that file,
//
//     #ifdef ROCM_HIP
//     #include "../cpp/hipfused_util.hpp"
//     #endif
//
// mirroring the `#ifdef CUDA` / `#ifdef APPLE_SILICON` fused-Adam blocks the
// reference keeps there (ml/util.cuh:147-210).  adam_state<T> is complete at
// this point, so the overload declared in hipmatrix.cuh can be defined.
#ifndef JZ_HIPFUSED_UTIL_HPP
#define JZ_HIPFUSED_UTIL_HPP

inline Matrix<ROCMfloat> adam_update(Matrix<ROCMfloat>&& g, adam_state<ROCMfloat>& state) {
    return jz_rocm_adam_update(std::move(g), state);
}

#endif
