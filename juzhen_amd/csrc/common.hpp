// Shared host/device helpers for the gfx950 kernel library.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "jzhip.h"

#define JZ_API extern "C" __attribute__((visibility("default")))

namespace jz {

constexpr int kWave = 64;        // CDNA wavefront width
constexpr int kBlock = 256;      // default workgroup: 4 waves, one per SIMD

// ── host-side runtime state (runtime.hip) ───────────────────────────────
hipStream_t stream();
int num_cus();
// Reads and clears the sticky launch error, like the reference's
// hipGetLastError() after each launch (cpp/hipkernels.cpp:463-465).
inline int launch_rc() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : static_cast<int>(e);
}
inline int rc_of(hipError_t e) { return e == hipSuccess ? 0 : static_cast<int>(e); }
// Device scratch for two-phase reductions; created once, never resized.
// Returns nullptr on allocation failure. Capacity in floats.
float* workspace();
constexpr size_t kWorkspaceFloats = size_t(16) << 20;  // 64 MiB

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Grid size for a grid-stride kernel over `work` items with `per_block` items
// per block per sweep: enough blocks to cover the data, capped at a few
// resident blocks per CU so that 8 XCDs x 32 CUs stay busy.
inline unsigned grid_for(size_t work, size_t per_block, int blocks_per_cu = 8) {
    size_t need = (work + per_block - 1) / per_block;
    size_t cap = static_cast<size_t>(num_cus()) * blocks_per_cu;
    if (need < 1) need = 1;
    return static_cast<unsigned>(need < cap ? need : cap);
}

// Grid that covers `work` items exactly once (`per_block` items per block).
// Streaming kernels use this rather than a capped grid-stride loop: workgroups
// are dispatched in id order, so the resident ones then stream one compact,
// moving window of memory.
inline unsigned grid_cover(size_t work, size_t per_block) {
    size_t need = (work + per_block - 1) / per_block;
    if (need < 1) need = 1;
    if (need > 0x7fffffffull) need = 0x7fffffffull;  // kernels keep their stride loop for the excess
    return static_cast<unsigned>(need);
}

// A launch that moves one and a half times what the 256 MB last-level cache holds gains nothing from
// keeping its data there; its loads and stores then carry the non-temporal hint (a copy of
// 2 GB: 6.1 -> 6.4 TB/s, of 0.5 GB 5.8 -> 6.4; column sums of 1 GB 5.5 -> 6.3).  Below
// that size the plain forms stay: what one kernel writes the next one often reads back out
// of the cache (hinted loads of a 134 MB operand that was resident ran 15 % slower, a
// 268 MB slice 7-30 % slower; a product of two 134 MB operands into a third, 403 MB in all, is the
// smallest launch measured that gains: 5.5 -> 6.3 TB/s).  Kernels that profit from the cache for longer (the
// optimiser's moments from step to step, a column softmax that holds whole columns in
// registers) ask with a fraction of their bytes.
constexpr size_t kStreamingBytes = size_t(384) << 20;
inline bool streams_past_cache(size_t bytes) { return bytes >= kStreamingBytes; }

// ── wave64 reductions: DPP inside a 16-lane row, bpermute across rows ────
#ifdef __HIPCC__
typedef float jz_f4 __attribute__((ext_vector_type(4)));
template <bool NT>
__device__ __forceinline__ float4 load4(const float* p) {
    if constexpr (NT) {
        const jz_f4 t = __builtin_nontemporal_load(reinterpret_cast<const jz_f4*>(p));
        return make_float4(t.x, t.y, t.z, t.w);
    } else {
        return *reinterpret_cast<const float4*>(p);
    }
}
template <bool NT>
__device__ __forceinline__ float load1(const float* p) {
    if constexpr (NT) return __builtin_nontemporal_load(p);
    else return *p;
}
template <bool NT>
__device__ __forceinline__ void store1(float* p, float v) {
    if constexpr (NT) __builtin_nontemporal_store(v, p);
    else *p = v;
}
template <bool NT>
__device__ __forceinline__ void store4(float* p, const float4& v) {
    if constexpr (NT) {
        jz_f4 t;
        t.x = v.x; t.y = v.y; t.z = v.z; t.w = v.w;
        __builtin_nontemporal_store(t, reinterpret_cast<jz_f4*>(p));
    } else {
        *reinterpret_cast<float4*>(p) = v;
    }
}
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

struct SumOp {
    __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
struct MaxOp {
    __device__ __forceinline__ float operator()(float a, float b) const { return a > b ? a : b; }
};

// After the call every lane holds the reduction over the whole wavefront.
template <class Op>
__device__ __forceinline__ float wave_allreduce(float v, Op op) {
    v = op(v, dpp_mov<0xB1>(v));   // quad_perm [1,0,3,2]
    v = op(v, dpp_mov<0x4E>(v));   // quad_perm [2,3,0,1]
    v = op(v, dpp_mov<0x141>(v));  // row_half_mirror
    v = op(v, dpp_mov<0x140>(v));  // row_mirror: every lane has its row's value
    v = op(v, __shfl_xor(v, 16, kWave));
    v = op(v, __shfl_xor(v, 32, kWave));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) { return wave_allreduce(v, SumOp{}); }
__device__ __forceinline__ float wave_max(float v) { return wave_allreduce(v, MaxOp{}); }

// Block-wide reduction for blocks of NW waves; `smem` holds NW floats.
// Every thread gets the result.
template <int NW, class Op>
__device__ __forceinline__ float block_allreduce(float v, Op op, float* smem, float identity) {
    v = wave_allreduce(v, op);
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    __syncthreads();  // protect smem from a previous use
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    float r = identity;
#pragma unroll
    for (int w = 0; w < NW; ++w) r = op(r, smem[w]);
    return r;
}

// Work split for "one wavefront per column" kernels: wave w of nw owns the
// contiguous range [wave_begin, wave_end) of the n columns, so the waves that
// are resident together stream one compact window of memory.
__device__ __forceinline__ size_t wave_begin(size_t n, size_t w, size_t nw) {
    const size_t per = (n + nw - 1) / nw;
    const size_t b = w * per;
    return b < n ? b : n;
}
__device__ __forceinline__ size_t wave_end(size_t n, size_t w, size_t nw) {
    const size_t per = (n + nw - 1) / nw;
    const size_t e = (w + 1) * per;
    return e < n ? e : n;
}

// e^x for x <= 0 through the hardware exp2: x*log2(e) is formed with its
// rounding error (fma) and the error is folded back in, which keeps the result
// within about 2 ulp; libm's expf costs an order of magnitude more
// instructions and made the softmax the longest phase of the attention kernel
// (and a third of the time of the long-column softmax).
__device__ __forceinline__ float exp_neg(float x) {
    const float l2e = 1.44269504088896341f;
    x = x > -100.0f ? x : -100.0f;   // masked scores (-1e9) end as an exact +0
    const float t = x * l2e;
    const float err = fmaf(x, l2e, -t) + x * 1.92596299112661746e-8f;   // low bits of the product and of log2(e)
    return __builtin_amdgcn_exp2f(t) * (1.0f + 0.693147180559945309f * err);
}

// Unsigned division by a runtime-uniform divisor via multiply-high.
// Valid for n < 2^31 and 1 <= d < 2^31.
struct FastDiv {
    uint32_t mul;
    uint32_t shift;
    uint32_t d;
};
__device__ __forceinline__ uint32_t fdiv(uint32_t n, const FastDiv& f) {
    return f.d == 1 ? n : (__umulhi(n, f.mul) >> f.shift);
}
#endif

inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.d = d;
    if (d == 1) {
        f.mul = 0;
        f.shift = 0;
        return f;
    }
    uint32_t l = 0;
    while ((uint32_t(1) << l) < d) ++l;  // l = ceil(log2 d), 1..31
    // mul = floor(2^(32+l-1) / d) + 1 truncated to 32 bits works for n < 2^31
    uint64_t m = ((uint64_t(1) << (32 + l - 1)) / d) + 1;
    f.mul = static_cast<uint32_t>(m);
    f.shift = l - 1;
    return f;
}

}  // namespace jz
