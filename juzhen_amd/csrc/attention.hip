// Batched causal self-attention core for TransformerLayer<ROCMfloat>: replaces
// the reference's per-(head, sequence) slice loop with its host-side mask
// writes (ml/layer.hpp:2967-3006, 3329-3363) by one fused launch forward and
// three launches backward (batched products and softmax kernels for shapes the
// fused kernel does not cover).  Same mathematics and the same buffer layouts as the
// reference's CUDA path (ml/layer.hpp:2880-2927, 3214-3283):
//   Q, K, V, H, dQ, dK, dV, dH : (d_k, S*B) column-major, head hh owns rows
//                                [hh*d_h, (hh+1)*d_h), sequence b columns [b*S, (b+1)*S)
//   A, dA                      : (S, S*B*heads), block hh*B + b is the S x S
//                                matrix A[query, key] of that head and sequence.
#include "common.hpp"

#include <cmath>
#include <mutex>
#include <type_traits>

namespace jz {
int gemm_batched2(const float* A, const float* B, float* C, int m, int n, int k, bool ta, bool tb,
                  int lda, int ldb, int ldc, long long sA, long long sB, long long sC, int batch,
                  long long sA2, long long sB2, long long sC2, int batch2, float alpha, float beta);
}


namespace jz {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// One workgroup per (head, sequence) block, everything for that block in one
// launch.  Forward (BWD = false):
//     P = softmax_keys(scale * K^T Q, causal mask)   -> A (kept for the backward pass)
//     H = V P
// Backward core (BWD = true), with P read back from A:
//     dA = V^T dH,  dS = P .* (dA - sum_keys(P .* dA)) * scale   -> dS
//     dQ = K dS
// (dV = dH P^T and dK = Q dS^T reduce over queries and stay batched GEMMs.)
//
// Both passes are "scores-like product, per-query row operation, second
// product": X1 (Q or dH) x M1 (K or V) gives a (keys x queries) matrix whose
// 16x16 MFMA tiles keep the query along the lanes and the keys along the
// accumulator registers, so the softmax (or its backward) is an in-register
// reduction plus two exchanges between the four lane groups, and the second
// product takes its B operand (P or dS) straight from those registers: the
// S x S matrix never goes through LDS and is written to HBM once.
//
// A wave owns 16 queries (all their keys: up to 16 tiles = 64 accumulator
// registers); sixteen waves cover S = 256, four per SIMD, assigned so that the
// causal triangle gives every SIMD the same work.  M1 is staged in LDS as
// [d][key], M2 as [key][d] (pitch DH+4); X1 fragments are read straight from
// global memory (each lane DH/4 consecutive floats of its query's column: lane
// group kq contracts d in [kq*DH/4, (kq+1)*DH/4)).
constexpr int kMaxKeys = 256;      // S <= 256
constexpr int kAttnThreads = 1024;  // sixteen waves, one group of 16 queries each, four per SIMD
// pitch of the [d][key] staging, whatever S is: the four lane groups of a
// fragment read rows DH/4 apart, which this pitch puts 16 banks apart, and the
// transposing staging stores stay conflict-free
template <int DH> constexpr int kLD1 = DH == 64 ? kMaxKeys + 1 : kMaxKeys + 2;

// One group of 16 queries against its first 4*NQ tiles of 16 keys (NQ
// compile-time so that the accumulator tiles stay in registers without
// predication); nkt <= 4*NQ tiles take part, the others are entirely masked.
// Lane (l16, kq): query 16g + l16; register v of score tile t is key
// 16t + 4kq + v (v_mfma_f32_16x16x4_f32 accumulator layout), so the softmax is
// an in-lane reduction plus two exchanges between the four lane groups, and
// step s of the second product contracts exactly the keys held in register s.
template <int DH, bool BWD, int NQ>
__device__ __forceinline__ void attn_group(float* __restrict__ out, int ld_out, float* __restrict__ Ablk,
                                           float* __restrict__ dSblk, float* __restrict__ stat, const float (&xf)[DH / 4],
                                           const float* t1, const float* t2, int S, int nkt, int g,
                                           int l16, int kq, float scale, int causal) {
    constexpr int HD4 = DH / 4;       // contraction steps of the first product
    constexpr int NDT = DH / 16;      // 16-row tiles of the second product's output
    constexpr int LD2 = DH + 4;
    constexpr int NT = 4 * NQ;
    constexpr int LD1 = kLD1<DH>;
    const int q = g * 16 + l16;       // query index inside the block
    // S x S block addressing: wave-uniform key row plus one lane offset
    const unsigned lane_off = static_cast<unsigned>(4 * kq) * static_cast<unsigned>(S) + q;

    // first product, four key tiles per contraction step (four independent MFMAs
    // cover the latency of the next step's LDS reads)
    floatx4 sc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) sc[t][v] = 0.0f;
#pragma unroll
    for (int tq = 0; tq < NQ; ++tq) {
        const float* base = t1 + 64 * tq;
        float a[4], n[4];
#pragma unroll
        for (int w = 0; w < 4; ++w) a[w] = base[16 * w];
#pragma unroll
        for (int kk = 0; kk < HD4; ++kk) {
            if (kk + 1 < HD4) {
#pragma unroll
                for (int w = 0; w < 4; ++w) n[w] = base[(kk + 1) * LD1 + 16 * w];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int w = 0; w < 4; ++w)
                sc[4 * tq + w] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[w], xf[kk], sc[4 * tq + w], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int w = 0; w < 4; ++w) a[w] = n[w];
        }
    }

    // per-query row operation over the nkt tiles that are not entirely masked
    if constexpr (!BWD) {
        float m = -1e30f;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if (t < nkt) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int key = 16 * t + 4 * kq + v;
                    float x = sc[t][v] * scale;
                    if (causal && key > q) x = -1e9f;   // ml/layer.hpp:2979-2994
                    sc[t][v] = x;
                    m = m > x ? m : x;
                }
            }
        }
        {
            float o = __shfl_xor(m, 16);
            m = m > o ? m : o;
            o = __shfl_xor(m, 32);
            m = m > o ? m : o;
        }
        float sum = 0.f;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if (t < nkt) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float e = exp_neg(sc[t][v] - m);
                    sc[t][v] = e;
                    sum += e;
                }
            }
        }
        sum += __shfl_xor(sum, 16);
        sum += __shfl_xor(sum, 32);
        const float inv = 1.0f / (sum + 1e-12f);
        if (stat) {
            // the probabilities are not kept: the backward pass recomputes them from the
            // query's maximum and reciprocal sum (S maxima, then S reciprocals per block)
            if (kq == 0) {
                stat[q] = m;
                stat[S + q] = inv;
            }
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                if (t < nkt) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) sc[t][v] *= inv;
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                if (t < nkt) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const float pv = sc[t][v] * inv;
                        sc[t][v] = pv;
                        (Ablk + static_cast<size_t>(16 * t + v) * S)[lane_off] = pv;
                    }
                }
            }
        }
    } else {
        // P is read twice (dot product, then dS) instead of being held in 4*NT more
        // registers; the other waves of the SIMD cover the latency.
        float dot = 0.f;
#pragma unroll
        for (int tq = 0; tq < NQ; ++tq) {
            float pv[16];
#pragma unroll
            for (int w = 0; w < 4; ++w)
                if (4 * tq + w < nkt) {
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        pv[4 * w + v] = (Ablk + static_cast<size_t>(16 * (4 * tq + w) + v) * S)[lane_off];
                }
#pragma unroll
            for (int w = 0; w < 4; ++w)
                if (4 * tq + w < nkt) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) dot += pv[4 * w + v] * sc[4 * tq + w][v];
                }
        }
        dot += __shfl_xor(dot, 16);
        dot += __shfl_xor(dot, 32);
#pragma unroll
        for (int tq = 0; tq < NQ; ++tq) {
            float pv[16];
#pragma unroll
            for (int w = 0; w < 4; ++w)
                if (4 * tq + w < nkt) {
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        pv[4 * w + v] = (Ablk + static_cast<size_t>(16 * (4 * tq + w) + v) * S)[lane_off];
                }
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const int t = 4 * tq + w;
                if (t < nkt) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const float ds = (pv[4 * w + v] * (sc[t][v] - dot)) * scale;
                        sc[t][v] = ds;
                        (dSblk + static_cast<size_t>(16 * t + v) * S)[lane_off] = ds;
                    }
                }
            }
        }
    }
    // key tiles past the causal range hold exact zeros (causal == 2: the caller
    // states that they already do, from an earlier call on the same buffer)
    if (causal != 2 && (BWD || !stat))
        for (int t = nkt; t < S / 16; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) ((BWD ? dSblk : Ablk) + static_cast<size_t>(16 * t + v) * S)[lane_off] = 0.0f;

    // second product: Out[d][query] = sum_key M2[d][key] * sc[key][query]; the
    // skipped tiles are a suffix, so the fragment prefetch can run ahead freely
    floatx4 oacc[NDT];
#pragma unroll
    for (int u = 0; u < NDT; ++u)
#pragma unroll
        for (int v = 0; v < 4; ++v) oacc[u][v] = 0.0f;
    float an[NDT];
#pragma unroll
    for (int u = 0; u < NDT; ++u) an[u] = t2[16 * u];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        if (t < nkt) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                float ac[NDT];
#pragma unroll
                for (int u = 0; u < NDT; ++u) ac[u] = an[u];
                if (4 * t + s + 1 < 4 * NT) {
                    const int keyn = s + 1 < 4 ? 16 * t + s + 1 : 16 * (t + 1);   // + 4kq is in t2
#pragma unroll
                    for (int u = 0; u < NDT; ++u) an[u] = t2[keyn * LD2 + 16 * u];
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < NDT; ++u)
                    oacc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(ac[u], sc[t][s], oacc[u], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    // Out(d, query): register v of tile u is d = 16u + 4kq + v
    float* dst = out + static_cast<size_t>(q) * ld_out + 4 * kq;
#pragma unroll
    for (int u = 0; u < NDT; ++u) *reinterpret_cast<floatx4*>(dst + 16 * u) = oacc[u];
}

template <int DH, bool BWD>
__global__ __launch_bounds__(kAttnThreads) void attn_core_kernel(
    float* __restrict__ Out, int ld_out, float* __restrict__ Aio, float* __restrict__ dS_out,
    float* __restrict__ stats, const float* __restrict__ X1, int ld_x1, const float* __restrict__ M1, const float* __restrict__ M2,
    int ld_m, int heads, int S, int B, float scale, int causal) {
    constexpr int HD4 = DH / 4;
    constexpr int LD2 = DH + 4;
    constexpr int LD1 = kLD1<DH>;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    // LDS columns / rows past S (up to the next multiple of 64) are read by the
    // tiles that complete a group of four but never enter a result.
    float* T1 = lds;                                    // [DH][LD1]
    float* T2 = lds + ((DH * LD1 + 3) / 4) * 4;         // [S rounded up to 64][LD2]

    const int blk = blockIdx.x;            // hh*B + b
    const int hh = blk / B, b = blk % B;
    const size_t col0 = static_cast<size_t>(b) * S;
    const float* m1 = M1 + col0 * ld_m + hh * DH;
    const float* m2 = M2 + col0 * ld_m + hh * DH;
    const float* x1 = X1 + col0 * ld_x1 + hh * DH;
    float* out = Out + col0 * ld_out + hh * DH;
    const size_t blk_off = static_cast<size_t>(blk) * S * S;
    float* Ablk = Aio ? Aio + blk_off : nullptr;
    float* dSblk = BWD ? dS_out + blk_off : nullptr;
    float* stat = (!BWD && stats) ? stats + static_cast<size_t>(blk) * 2 * S : nullptr;

    // the four waves of a SIMD (w, w+4, w+8, w+12) take query groups s, 7-s,
    // 8+s, 15-s: with the causal triangle every SIMD gets the same work
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int l16 = lane & 15, kq = lane >> 4;
    const int GQ = S / 16;
    const int ws = wave & 3, wj = wave >> 2;
    const int g = wj == 0 ? ws : wj == 1 ? 7 - ws : wj == 2 ? 8 + ws : 15 - ws;
    const bool mine = g < GQ;
    // this lane's X1 fragments (d = HD4*kq + kk for kk = 0..HD4-1), requested
    // before the staging so that they arrive behind it
    float xf[HD4];
    if (mine) {
        const float* src = x1 + static_cast<size_t>(g * 16 + l16) * ld_x1 + HD4 * kq;
#pragma unroll
        for (int i = 0; i < HD4 / 4; ++i) {
            const floatx4 t = *reinterpret_cast<const floatx4*>(src + 4 * i);
            xf[4 * i] = t.x; xf[4 * i + 1] = t.y; xf[4 * i + 2] = t.z; xf[4 * i + 3] = t.w;
        }
    }

    // stage M1 transposed and M2 as it lies: all global loads of a thread first
    // (they are independent), then the LDS stores
    {
        constexpr int kIters = (DH / 4) * kMaxKeys / kAttnThreads;
        const int total = (DH / 4) * S;
        floatx4 ra[kIters], rc[kIters];
#pragma unroll
        for (int i = 0; i < kIters; ++i) {
            const int v = threadIdx.x + i * kAttnThreads;
            if (v < total) {
                const int dq = v % (DH / 4), tok = v / (DH / 4);
                ra[i] = *reinterpret_cast<const floatx4*>(m1 + static_cast<size_t>(tok) * ld_m + 4 * dq);
                rc[i] = *reinterpret_cast<const floatx4*>(m2 + static_cast<size_t>(tok) * ld_m + 4 * dq);
            }
        }
#pragma unroll
        for (int i = 0; i < kIters; ++i) {
            const int v = threadIdx.x + i * kAttnThreads;
            if (v < total) {
                const int dq = v % (DH / 4), tok = v / (DH / 4);
                float* d1 = T1 + (4 * dq) * LD1 + tok;
                d1[0] = ra[i].x; d1[LD1] = ra[i].y; d1[2 * LD1] = ra[i].z; d1[3 * LD1] = ra[i].w;
                *reinterpret_cast<floatx4*>(T2 + tok * LD2 + 4 * dq) = rc[i];
            }
        }
    }
    __syncthreads();

    const float* t1 = T1 + (HD4 * kq) * LD1 + l16;
    const float* t2 = T2 + (4 * kq) * LD2 + l16;

    if (mine) {
        const int nkt = causal ? g + 1 : GQ;          // key tiles that are not entirely masked
        switch ((nkt + 3) / 4) {
        case 1: attn_group<DH, BWD, 1>(out, ld_out, Ablk, dSblk, stat, xf, t1, t2, S, nkt, g, l16, kq, scale, causal); break;
        case 2: attn_group<DH, BWD, 2>(out, ld_out, Ablk, dSblk, stat, xf, t1, t2, S, nkt, g, l16, kq, scale, causal); break;
        case 3: attn_group<DH, BWD, 3>(out, ld_out, Ablk, dSblk, stat, xf, t1, t2, S, nkt, g, l16, kq, scale, causal); break;
        default: attn_group<DH, BWD, 4>(out, ld_out, Ablk, dSblk, stat, xf, t1, t2, S, nkt, g, l16, kq, scale, causal); break;
        }
    }
}

size_t attn_core_lds_bytes(int d_h, int S) {
    const size_t S2 = static_cast<size_t>(S + 63) / 64 * 64;
    const size_t ld1 = d_h == 64 ? kLD1<64> : kLD1<32>;
    return ((d_h * ld1 + 3) / 4 * 4 + S2 * (d_h + 4)) * sizeof(float);
}

// The fused kernel covers head widths 32 and 64 with S a multiple of 32 up to
// 256 and 16-byte aligned operands; other shapes take the batched-GEMM path.
bool attn_core_ok(int d_h, int S, int heads, int B, const void* p0, const void* p1, const void* p2, const void* p3,
                  int ld_a, int ld_b, int ld_c) {
    if (!(d_h == 32 || d_h == 64)) return false;
    if (S % 32 != 0 || S > kMaxKeys) return false;
    if (static_cast<long long>(heads) * B > 0x7fffffffLL) return false;
    if (ld_a % 4 || ld_b % 4 || ld_c % 4) return false;
    return aligned16(p0) && aligned16(p1) && aligned16(p2) && aligned16(p3);
}

template <int DH, bool BWD>
int launch_attn_core(float* Out, int ld_out, float* Aio, float* dS, float* stats, const float* X1, int ld_x1,
                     const float* M1, const float* M2, int ld_m, int heads, int S, int B, float scale, int causal) {
    const size_t lds = attn_core_lds_bytes(DH, S);
    static std::once_flag once;   // per instantiation
    static int configure_rc = 0;
    std::call_once(once, [] {
        configure_rc = rc_of(hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_core_kernel<DH, BWD>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    });
    if (configure_rc) return configure_rc;
    attn_core_kernel<DH, BWD><<<heads * B, kAttnThreads, lds, stream()>>>(Out, ld_out, Aio, dS, stats, X1, ld_x1, M1, M2,
                                                                   ld_m, heads, S, B, scale, causal);
    return launch_rc();
}

}  // namespace
}  // namespace jz

JZ_API int jzhip_attention_fwd_ld(float* H, int ld_h, float* A, const float* Q, const float* K,
                                  const float* V, int ld_qkv, int d_k, int heads, int S, int B,
                                  int causal) {
    if (d_k <= 0 || heads <= 0 || S <= 0 || B <= 0 || d_k % heads != 0) return -1;
    if (!H || !A || !Q || !K || !V || ld_h < d_k || ld_qkv < d_k) return -1;
    if (causal < 0 || causal > 2) return -1;
    const int d_h = d_k / heads;
    const long long seq = static_cast<long long>(S) * ld_qkv;  // next sequence in Q/K/V
    const long long seq_h = static_cast<long long>(S) * ld_h;  // next sequence in H
    const long long blk = static_cast<long long>(S) * S;       // next score block
    const float scale = 1.0f / sqrtf(static_cast<float>(d_h));
    if (jz::attn_core_ok(d_h, S, heads, B, H, Q, K, V, ld_h, ld_qkv, ld_qkv)) {
        if (d_h == 64)
            return jz::launch_attn_core<64, false>(H, ld_h, A, nullptr, nullptr, Q, ld_qkv, K, V, ld_qkv, heads, S, B,
                                                   scale, causal);
        return jz::launch_attn_core<32, false>(H, ld_h, A, nullptr, nullptr, Q, ld_qkv, K, V, ld_qkv, heads, S, B, scale,
                                               causal);
    }
    // scores[q, k] = <Q_i[:, q], K_i[:, k]>
    int rc = jz::gemm_batched2(Q, K, A, S, S, d_h, true, false, ld_qkv, ld_qkv, S, seq, seq, blk, B, d_h, d_h,
                               blk * B, heads, 1.0f, 0.0f);
    if (rc) return rc;
    // A = softmax over keys of (scores*scale, masked)
    rc = jzhip_attn_softmax(A, A, S, B * heads, scale, causal != 0, 0);
    if (rc) return rc;
    // H_i = V_i * A_i^T
    return jz::gemm_batched2(V, A, H, d_h, S, S, false, true, ld_qkv, S, ld_h, seq, blk, seq_h, B, d_h,
                             blk * B, d_h, heads, 1.0f, 0.0f);
}

JZ_API int jzhip_attention_fwd(float* H, float* A, const float* Q, const float* K, const float* V,
                               int d_k, int heads, int S, int B, int causal) {
    return jzhip_attention_fwd_ld(H, d_k, A, Q, K, V, d_k, d_k, heads, S, B, causal);
}

JZ_API int jzhip_attention_bwd_ld(float* dQ, float* dK, float* dV, int ld_dqkv, float* dA_scratch,
                                  const float* dH, int ld_dh, const float* Q, const float* K,
                                  const float* V, int ld_qkv, const float* A, int d_k, int heads,
                                  int S, int B, int causal) {
    if (d_k <= 0 || heads <= 0 || S <= 0 || B <= 0 || d_k % heads != 0) return -1;
    if (!dQ || !dK || !dV || !dA_scratch || !dH || !Q || !K || !V || !A) return -1;
    if (ld_dqkv < d_k || ld_dh < d_k || ld_qkv < d_k) return -1;
    if (causal < 0 || causal > 2) return -1;
    const int d_h = d_k / heads;
    const long long seq = static_cast<long long>(S) * ld_qkv;
    const long long seq_d = static_cast<long long>(S) * ld_dqkv;
    const long long seq_h = static_cast<long long>(S) * ld_dh;
    const long long blk = static_cast<long long>(S) * S;
    const float scale = 1.0f / sqrtf(static_cast<float>(d_h));
    // dV_i = dH_i * A_i
    int rc = jz::gemm_batched2(dH, A, dV, d_h, S, S, false, false, ld_dh, S, ld_dqkv, seq_h, blk, seq_d, B, d_h,
                               blk * B, d_h, heads, 1.0f, 0.0f);
    if (rc) return rc;
    if (jz::attn_core_ok(d_h, S, heads, B, dQ, dH, K, V, ld_dqkv, ld_dh, ld_qkv)) {
        // dA, dS and dQ in one launch; with causal set the key tiles above the
        // diagonal (exact zeros in A) are skipped
        rc = d_h == 64 ? jz::launch_attn_core<64, true>(dQ, ld_dqkv, const_cast<float*>(A), dA_scratch, nullptr, dH,
                                                        ld_dh, V, K, ld_qkv, heads, S, B, scale, causal)
                       : jz::launch_attn_core<32, true>(dQ, ld_dqkv, const_cast<float*>(A), dA_scratch, nullptr, dH,
                                                        ld_dh, V, K, ld_qkv, heads, S, B, scale, causal);
        if (rc) return rc;
        // dK_i = Q_i * dS_i
        return jz::gemm_batched2(Q, dA_scratch, dK, d_h, S, S, false, false, ld_qkv, S, ld_dqkv, seq, blk, seq_d, B,
                                 d_h, blk * B, d_h, heads, 1.0f, 0.0f);
    }
    // dA_i[q, k] = <dH_i[:, q], V_i[:, k]>
    rc = jz::gemm_batched2(dH, V, dA_scratch, S, S, d_h, true, false, ld_dh, ld_qkv, S, seq_h, seq, blk, B, d_h,
                           d_h, blk * B, heads, 1.0f, 0.0f);
    if (rc) return rc;
    // dS = A .* (dA - rowsum(A .* dA)) * scale, in place
    rc = jzhip_attn_softmax_bwd(dA_scratch, A, dA_scratch, S, B * heads, scale, 0);
    if (rc) return rc;
    // dQ_i = K_i * dS_i^T
    rc = jz::gemm_batched2(K, dA_scratch, dQ, d_h, S, S, false, true, ld_qkv, S, ld_dqkv, seq, blk, seq_d, B, d_h,
                           blk * B, d_h, heads, 1.0f, 0.0f);
    if (rc) return rc;
    // dK_i = Q_i * dS_i
    return jz::gemm_batched2(Q, dA_scratch, dK, d_h, S, S, false, false, ld_qkv, S, ld_dqkv, seq, blk, seq_d, B,
                             d_h, blk * B, d_h, heads, 1.0f, 0.0f);
}

JZ_API int jzhip_attention_bwd(float* dQ, float* dK, float* dV, float* dA_scratch, const float* dH,
                               const float* Q, const float* K, const float* V, const float* A,
                               int d_k, int heads, int S, int B) {
    return jzhip_attention_bwd_ld(dQ, dK, dV, d_k, dA_scratch, dH, d_k, Q, K, V, d_k, A, d_k, heads, S, B, 0);
}

JZ_API int jzhip_attention_flash_fwd(float* H, int ld_h, float* stats, const float* Q, const float* K, const float* V,
                                     int ld_qkv, int d_k, int heads, int S, int B, int causal) {
    if (!H || !stats || !Q || !K || !V) return -1;
    if (!jzhip_attention_flash_supported(d_k, heads, S, B)) return -1;
    if (ld_h < d_k || ld_qkv < d_k || causal < 0 || causal > 1) return -1;
    const int d_h = d_k / heads;
    if (!jz::attn_core_ok(d_h, S, heads, B, H, Q, K, V, ld_h, ld_qkv, ld_qkv)) return -1;
    const float scale = 1.0f / sqrtf(static_cast<float>(d_h));
    if (d_h == 64)
        return jz::launch_attn_core<64, false>(H, ld_h, nullptr, nullptr, stats, Q, ld_qkv, K, V, ld_qkv, heads, S, B,
                                               scale, causal);
    return jz::launch_attn_core<32, false>(H, ld_h, nullptr, nullptr, stats, Q, ld_qkv, K, V, ld_qkv, heads, S, B, scale,
                                           causal);
}
