// Device random numbers: counter-based Philox4x32-10 (Salmon et al., SC'11),
// four outputs per counter, so generation is stateless on the device and the
// host only tracks (seed, counter offset).  Replaces the rocRAND generator of
// the reference (cpp/hipkernels.cpp:471-608).  Parity with the CPU mt19937
// stream is not a goal: the reference's own tests only require finite values
// in range (tests/testRocmCpuParity.cu:214-224).
#include "common.hpp"

#include <mutex>

namespace jz {
namespace {

struct RngState {
    std::mutex mu;
    uint64_t seed = 0x6a7568656eULL;
    uint64_t offset = 0;  // counters consumed so far
};
RngState& rng_state() {
    static RngState s;
    return s;
}

__device__ __forceinline__ void philox_round(uint32_t (&c)[4], uint32_t k0, uint32_t k1) {
    const uint32_t hi0 = __umulhi(0xD2511F53u, c[0]), lo0 = 0xD2511F53u * c[0];
    const uint32_t hi1 = __umulhi(0xCD9E8D57u, c[2]), lo1 = 0xCD9E8D57u * c[2];
    const uint32_t n0 = hi1 ^ c[1] ^ k0, n2 = hi0 ^ c[3] ^ k1;
    c[0] = n0;
    c[1] = lo1;
    c[2] = n2;
    c[3] = lo0;
}

__device__ __forceinline__ void philox4x32_10(uint64_t counter, uint64_t seed, uint32_t (&out)[4]) {
    uint32_t c[4] = {static_cast<uint32_t>(counter), static_cast<uint32_t>(counter >> 32), 0u, 0u};
    uint32_t k0 = static_cast<uint32_t>(seed), k1 = static_cast<uint32_t>(seed >> 32);
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        philox_round(c, k0, k1);
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = c[i];
}

// NORMAL = false: U[0,1).  NORMAL = true: mean + stddev*N(0,1) (Box-Muller).
template <bool NORMAL>
__global__ __launch_bounds__(kBlock) void rng_kernel(float* dst, size_t n, uint64_t seed,
                                                     uint64_t offset, float mean, float stddev) {
    const size_t stride = static_cast<size_t>(gridDim.x) * kBlock;
    const size_t groups = (n + 3) / 4;
    for (size_t gidx = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x; gidx < groups; gidx += stride) {
        uint32_t r[4];
        philox4x32_10(offset + gidx, seed, r);
        float v[4];
        if constexpr (NORMAL) {
            constexpr float kTwoPi = 6.28318530717958647692f;
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const float u1 = (static_cast<float>(r[2 * p] >> 8) + 1.0f) * (1.0f / 16777216.0f);  // (0,1]
                const float u2 = static_cast<float>(r[2 * p + 1] >> 8) * (1.0f / 16777216.0f);       // [0,1)
                const float rad = sqrtf(-2.0f * logf(u1));
                float sn, cs;
                sincosf(kTwoPi * u2, &sn, &cs);
                v[2 * p] = mean + stddev * (rad * cs);
                v[2 * p + 1] = mean + stddev * (rad * sn);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = static_cast<float>(r[i] >> 8) * (1.0f / 16777216.0f);
        }
        const size_t base = gidx * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (base + i < n) dst[base + i] = v[i];
    }
}

template <bool NORMAL>
int generate(float* dst, size_t count, float mean, float stddev, uint64_t seed) {
    if (count == 0) return 0;
    if (!dst) return -1;
    uint64_t use_seed, use_off;
    {
        RngState& st = rng_state();
        std::lock_guard<std::mutex> lock(st.mu);
        if (seed != 0) {
            st.seed = seed;
            st.offset = 0;
        }
        use_seed = st.seed;
        use_off = st.offset;
        st.offset += (count + 3) / 4;
    }
    const unsigned grid = grid_for((count + 3) / 4, kBlock, 8);
    rng_kernel<NORMAL><<<grid, kBlock, 0, stream()>>>(dst, count, use_seed, use_off, mean, stddev);
    return launch_rc();
}

}  // namespace
}  // namespace jz

JZ_API int jzhip_rand_uniform(float* dst, size_t count, uint64_t seed) {
    return jz::generate<false>(dst, count, 0.f, 1.f, seed);
}

JZ_API int jzhip_rand_normal(float* dst, size_t count, float mean, float stddev, uint64_t seed) {
    return jz::generate<true>(dst, count, mean, stddev, seed);
}
