// Tile machinery shared by the fp32 MFMA kernels (gemm.hip, conv_gemm.hip):
// vector types, the K extent of an LDS stage, the global -> register -> LDS
// staging of one operand tile and the fragment reads that feed
// v_mfma_f32_32x32x2_f32.  Everything here has internal linkage.
#pragma once

#include "common.hpp"

namespace jz {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
// native vector type for staging registers (HIP's float4 is a struct around a
// union, which kept the staging array in scratch memory)
typedef float floatx4 __attribute__((ext_vector_type(4)));

#ifndef JZ_GEMM_OCC
#define JZ_GEMM_OCC 3
#endif
#ifndef JZ_GEMM_SETS
#define JZ_GEMM_SETS 2
#endif
#ifndef JZ_GEMM_BK
#define JZ_GEMM_BK 16
#endif
#ifndef JZ_GEMM_PAD
#define JZ_GEMM_PAD 4
#endif
constexpr int BK = JZ_GEMM_BK;     // K extent of one LDS stage
constexpr int kPad = JZ_GEMM_PAD;  // keeps 16-byte alignment of LDS rows, skews banks

// Global -> register staging for one operand tile of EXT (BM or BN) x BK.
// MNC = true : the operand is contiguous along its m/n index (A not
//              transposed, or B transposed): element (x, k) at p[k*ld + x].
// MNC = false: contiguous along k (A transposed, or B not transposed):
//              element (x, k) at p[x*ld + k].
// T is the number of 32-wide MFMA tiles a wave owns along this operand.  The
// LDS tile is [BK][EXT + kPad] with the T tiles of a wave interleaved inside
// each row (x = w*32T + i*32 + l is kept at w*32T + l*T + i), so that a lane
// fetches its T fragment values of one k with a single 4T-byte read at an
// immediate offset.
template <int EXT, bool MNC, int T>
struct TileLoader {
    static constexpr int kVecs = EXT * BK / 4;             // float4 per tile
    static constexpr int kPasses = (kVecs + kBlock - 1) / kBlock;
    // Interleaving two tiles turns the float4 of a contiguous operand into four
    // stride-2 stores; skewing each wave's 64-float group by two banks keeps the
    // 32 lanes of such a store on distinct banks.  The row pitch is rounded up to
    // 4 (mod 16) floats so that the four k-rows written by a k-contiguous
    // operand (lanes = 8 x-values times 4 k-quads) also land on distinct banks.
    static constexpr int kSkew = (T == 2) ? 2 : 0;
    static constexpr int kGroup = 32 * T + kSkew;          // floats per wave group in a row
    static constexpr int kRow = (EXT / (32 * T)) * kGroup;
    static constexpr int LD = kRow + ((4 - kRow % 16) + 16) % 16;

    static __device__ __forceinline__ int pos(int x) {
        return (x / (32 * T)) * kGroup + (x % 32) * T + (x / 32) % T;
    }
    static __device__ __forceinline__ void coords(int ps, int& x, int& k) {
        const int v = threadIdx.x + ps * kBlock;
        if constexpr (MNC) {
            x = (v % (EXT / 4)) * 4;
            k = v / (EXT / 4);
        } else {
            k = (v % (BK / 4)) * 4;
            x = v / (BK / 4);
        }
    }
    static __device__ __forceinline__ bool active(int ps) {
        return kVecs % kBlock == 0 || threadIdx.x + ps * kBlock < kVecs;
    }

    // Fast path (tile inside the matrix, ld % 4 == 0, 16-byte aligned base,
    // 256*ld*4 < 2^32): per-thread 32-bit element offsets from the tile origin
    // are computed once; each K stage adds them to a wave-uniform pointer.
    static __device__ __forceinline__ void offsets(unsigned (&off)[kPasses], unsigned ld) {
#pragma unroll
        for (int ps = 0; ps < kPasses; ++ps) {
            int x, k;
            coords(ps, x, k);
            off[ps] = MNC ? static_cast<unsigned>(k) * ld + x : static_cast<unsigned>(x) * ld + k;
        }
    }
    // origin: p advanced to (x0, k0) of the stage
    static __device__ __forceinline__ const float* origin(const float* p, size_t ld, int x0, int k0) {
        return MNC ? p + static_cast<size_t>(k0) * ld + x0 : p + static_cast<size_t>(x0) * ld + k0;
    }
    static __device__ __forceinline__ void load_fast(floatx4 (&reg)[kPasses], const float* __restrict__ org,
                                                     const unsigned (&off)[kPasses]) {
#pragma unroll
        for (int ps = 0; ps < kPasses; ++ps)
            if (active(ps)) reg[ps] = *reinterpret_cast<const floatx4*>(org + off[ps]);
    }

    // Bounds-checked path for edge tiles and unaligned operands.
    static __device__ __forceinline__ void load_checked(floatx4 (&reg)[kPasses], const float* __restrict__ p,
                                                        size_t ld, int x0, int k0, int X, int K) {
#pragma unroll
        for (int ps = 0; ps < kPasses; ++ps) {
            // (no early exit: the loop must unroll fully so reg[] stays in registers)
            if (active(ps)) {
                int x, k;
                coords(ps, x, k);
                const int gx = x0 + x, gk = k0 + k;
                floatx4 t = {0.f, 0.f, 0.f, 0.f};
                if constexpr (MNC) {
                    if (gk < K) {
                        const float* src = p + static_cast<size_t>(gk) * ld + gx;
                        if (gx + 0 < X) t.x = src[0];
                        if (gx + 1 < X) t.y = src[1];
                        if (gx + 2 < X) t.z = src[2];
                        if (gx + 3 < X) t.w = src[3];
                    }
                } else {
                    if (gx < X) {
                        const float* src = p + static_cast<size_t>(gx) * ld + gk;
                        if (gk + 0 < K) t.x = src[0];
                        if (gk + 1 < K) t.y = src[1];
                        if (gk + 2 < K) t.z = src[2];
                        if (gk + 3 < K) t.w = src[3];
                    }
                }
                reg[ps] = t;
            }
        }
    }

    // registers -> LDS
    static __device__ __forceinline__ void store(const floatx4 (&reg)[kPasses], float* __restrict__ s) {
#pragma unroll
        for (int ps = 0; ps < kPasses; ++ps) store_pass(reg, s, ps);
    }
    static __device__ __forceinline__ void store_pass(const floatx4 (&reg)[kPasses], float* __restrict__ s,
                                                      int ps) {
        {
            if (active(ps)) {
                int x, k;
                coords(ps, x, k);
                if constexpr (MNC) {
                    float* d = s + k * LD + pos(x);  // x % 4 == 0: the four values share a tile
                    if constexpr (T == 1) {
                        *reinterpret_cast<floatx4*>(d) = reg[ps];
                    } else {
                        d[0 * T] = reg[ps].x;
                        d[1 * T] = reg[ps].y;
                        d[2 * T] = reg[ps].z;
                        d[3 * T] = reg[ps].w;
                    }
                } else {
                    float* d = s + k * LD + pos(x);
                    d[0 * LD] = reg[ps].x;
                    d[1 * LD] = reg[ps].y;
                    d[2 * LD] = reg[ps].z;
                    d[3 * LD] = reg[ps].w;
                }
            }
        }
    }
};

// T fragment values of one lane, read from LDS with one 4T-byte access
template <int T>
struct Frag {
    typedef float vec __attribute__((ext_vector_type(T)));
    vec v;
    __device__ __forceinline__ void read(const float* p) { v = *reinterpret_cast<const vec*>(p); }
    __device__ __forceinline__ float operator[](int i) const { return v[i]; }
};
template <>
struct Frag<1> {
    float v;
    __device__ __forceinline__ void read(const float* p) { v = *p; }
    __device__ __forceinline__ float operator[](int) const { return v; }
};

}  // namespace
}  // namespace jz
