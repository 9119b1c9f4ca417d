// Matrix-vector products and their few-vector generalisation, the
// bandwidth-bound relatives of the tiled GEMM: y = alpha*op(A)*x + beta*y, and
// C = op(A) op(B) where m or n is at most kThinMax.
#include "common.hpp"

namespace jz {
namespace {

// y[j] = alpha * <A[:,j], x> + beta*y[j]: one wavefront per column of the
// physical m x n matrix (op = transpose).
__global__ __launch_bounds__(kBlock) void gemv_t_kernel(const float* A, const float* x, float* y,
                                                        int m, int n, size_t lda, size_t incx,
                                                        size_t incy, float alpha, float beta) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t wave0 = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
    const size_t nwaves = static_cast<size_t>(gridDim.x) * (kBlock / kWave);
    for (size_t j = wave0; j < static_cast<size_t>(n); j += nwaves) {
        const float* col = A + j * lda;
        float acc = 0.f;
        for (int i = lane; i < m; i += kWave) acc += col[i] * x[i * incx];
        acc = wave_sum(acc);
        if (lane == 0) {
            float r = alpha * acc;
            if (beta != 0.0f) r += beta * y[j * incy];
            y[j * incy] = r;
        }
    }
}

// y[i] = alpha * sum_j A[i,j]*x[j] + beta*y[i] (op = none): lanes along rows,
// the block's waves split the columns, combined through LDS.  Partial results
// over column chunks go to part[chunk*m + i].
__global__ __launch_bounds__(kBlock) void gemv_n_partial_kernel(const float* A, const float* x,
                                                                float* part, int m, int n,
                                                                size_t lda, size_t incx,
                                                                int chunk_len) {
    constexpr int NW = kBlock / kWave;
    __shared__ float red[NW][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int row = blockIdx.x * kWave + lane;
    const int c_begin = blockIdx.y * chunk_len;
    int c_end = c_begin + chunk_len;
    if (c_end > n) c_end = n;
    float acc = 0.f;
    if (row < m)
        for (int c = c_begin + wave; c < c_end; c += NW) acc += A[static_cast<size_t>(c) * lda + row] * x[c * incx];
    red[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && row < m) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) s += red[w][lane];
        part[static_cast<size_t>(blockIdx.y) * m + row] = s;
    }
}

// y[i] = alpha * sum_c part[c*m + i] + beta*y[i]: 64 outputs per workgroup, its
// sixteen waves taking interleaved chunks (four loads in flight each) and
// meeting in LDS; fixed order, so the result is deterministic.
constexpr int kGemvCombineBlock = 1024;
// Output i lives at y[(i % len)*s_in + (i / len)*s_out] (a plain vector has len = m).
__global__ __launch_bounds__(kGemvCombineBlock) void gemv_n_combine_kernel(float* y, const float* part, int m,
                                                                           int chunks, int len, size_t s_in,
                                                                           size_t s_out, float alpha, float beta) {
    constexpr int NW = kGemvCombineBlock / kWave;
    __shared__ float red[NW][kWave];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int i = blockIdx.x * kWave + lane;
    float acc = 0.f;
    if (i < m) {
        const float* p = part + i;
        int c = wave;
        for (; c + 3 * NW < chunks; c += 4 * NW) {
            float x[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) x[u] = p[static_cast<size_t>(c + u * NW) * m];
#pragma unroll
            for (int u = 0; u < 4; ++u) acc += x[u];
        }
        for (; c < chunks; c += NW) acc += p[static_cast<size_t>(c) * m];
    }
    red[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && i < m) {
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) sum += red[w][lane];
        float* dst = y + static_cast<size_t>(i % len) * s_in + static_cast<size_t>(i / len) * s_out;
        float r = alpha * sum;
        if (beta != 0.0f) r += beta * *dst;
        *dst = r;
    }
}

// The same sum for a few chunks and many outputs (a 10 x 12544 gradient in two chunks): one thread per
// output, chunks in order.
__global__ __launch_bounds__(kBlock) void gemv_n_combine_few_kernel(float* y, const float* part, int m, int chunks,
                                                                    int len, size_t s_in, size_t s_out, float alpha,
                                                                    float beta) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= m) return;
    float sum = 0.f;
    for (int c = 0; c < chunks; ++c) sum += part[static_cast<size_t>(c) * m + i];
    float* dst = y + static_cast<size_t>(i % len) * s_in + static_cast<size_t>(i / len) * s_out;
    float r = alpha * sum;
    if (beta != 0.0f) r += beta * *dst;
    *dst = r;
}

void launch_thin_combine(float* y, const float* part, size_t outs, int chunks, int len, size_t s_in, size_t s_out,
                         float alpha, float beta, hipStream_t s) {
    if (chunks <= 8)
        gemv_n_combine_few_kernel<<<static_cast<unsigned>((outs + kBlock - 1) / kBlock), kBlock, 0, s>>>(
            y, part, static_cast<int>(outs), chunks, len, s_in, s_out, alpha, beta);
    else
        gemv_n_combine_kernel<<<static_cast<unsigned>((outs + kWave - 1) / kWave), kGemvCombineBlock, 0, s>>>(
            y, part, static_cast<int>(outs), chunks, len, s_in, s_out, alpha, beta);
}

// ── thin products: one extent of C is at most kThinMax ───────────────────
// C = op(A) op(B) with m or n <= kThinMax (a 3-channel output convolution:
// 3 x 131072 x 576 forward, 576 x 3 x 131072 for its weight gradient; a 10-class
// dense layer: 10 x 128 x 12544) is a handful of matrix-vector products over one big operand: bound by reading
// that operand once, which an MFMA tile padded to 32 rows cannot approach.
// The big operand X is L x K (element (l,k) at X[l*xs_l + k*xs_k], one of the
// strides being 1), the thin one V is T x K (V[t*vs_t + k*vs_k]); output (l,t)
// goes to C[l*cs_l + t*cs_t].
constexpr int kThinMax = 16;
// rows of X a wavefront walks together in the dot form: two with up to four thin
// vectors (measured 55 against 58 us at 3 x 131072 x 576), four with up to eight, where
// each LDS read of V should serve more rows, two again with sixteen (32 sums per lane)
template <int TT> constexpr int kThinRows = TT == 1 ? 4 : (TT <= 4 ? 2 : (TT <= 8 ? 4 : 2));
constexpr int thin_tt(int T) { return T == 1 ? 1 : (T <= 4 ? 4 : (T <= 8 ? 8 : 16)); }   // template width serving T vectors
constexpr int kThinChunkMax = 1024;   // k per workgroup in the other form (V's slice: 32 KB at eight vectors)
constexpr int thin_chunk_max(int tt) { return tt <= 8 ? kThinChunkMax : kThinChunkMax / 2; }
constexpr int kThinDotChunkMax = 512;   // k per workgroup in the chunked dot form: two float4 steps per lane

// Sums NV (a power of two, at most 64) values per lane over the 64 lanes.  On
// return v[0] of lane i holds the total of value i >> log2(64 / NV); the lane
// whose low bits are zero gets that index back, the others -1.
template <int N>
__device__ __forceinline__ void fold_half(float* v, int lane, int mask) {
    const bool upper = (lane & mask) != 0;
#pragma unroll
    for (int i = 0; i < N / 2; ++i) {
        const float keep = upper ? v[i + N / 2] : v[i];
        const float send = upper ? v[i] : v[i + N / 2];
        v[i] = keep + __shfl_xor(send, mask, kWave);
    }
}
template <int NV>
__device__ __forceinline__ int wave_sum_many(float (&v)[NV], int lane) {
    static_assert(NV >= 1 && NV <= kWave && (NV & (NV - 1)) == 0, "power of two");
    int mask = kWave / 2;
    if constexpr (NV >= 64) { fold_half<64>(v, lane, mask); mask >>= 1; }
    if constexpr (NV >= 32) { fold_half<32>(v, lane, mask); mask >>= 1; }
    if constexpr (NV >= 16) { fold_half<16>(v, lane, mask); mask >>= 1; }
    if constexpr (NV >= 8) { fold_half<8>(v, lane, mask); mask >>= 1; }
    if constexpr (NV >= 4) { fold_half<4>(v, lane, mask); mask >>= 1; }
    if constexpr (NV >= 2) { fold_half<2>(v, lane, mask); mask >>= 1; }
    const int rest = 2 * mask;   // lanes that now hold the same value index, a power of two (or 0 when NV == 64)
    for (int m = mask; m >= 1; m >>= 1) v[0] += __shfl_xor(v[0], m, kWave);
    if (rest == 0) return lane;
    return (lane & (rest - 1)) == 0 ? lane / rest : -1;
}

// Stages V's slice [k_begin, k_begin + len) into LDS as [TT][pitch], zeros for t >= T and k >= len.  When the
// thin index is the contiguous one in memory (a 10 x K matrix stored by columns) the threads walk the
// memory order, runs of T floats, instead of gathering one float per 4*vs_k bytes.
template <int TT>
__device__ __forceinline__ void stage_thin(float* __restrict__ vl, const float* __restrict__ V, size_t vs_t, size_t vs_k,
                                           int T, int k_begin, int len, int pitch) {
    // eight independent loads per thread before their LDS stores: a load per iteration behind a store
    // the compiler cannot move it past makes every element a full trip to memory
    constexpr int kBatch = 8;
    const bool by_t = vs_t == 1 && T > 1;
    const int n = T * len;
    const float* block = V + static_cast<size_t>(k_begin) * vs_k;
    if (by_t && vs_k == static_cast<size_t>(T) && n % 4 == 0 && (reinterpret_cast<uintptr_t>(block) & 15u) == 0) {
        // the slice is one contiguous block of T*len floats: 16-byte loads, four in flight per thread
        const float4* b4 = reinterpret_cast<const float4*>(block);
        const int n4 = n / 4;
        for (int i0 = threadIdx.x; i0 < n4; i0 += kBlock * 4) {
            float4 r[4];
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int i = i0 + b * kBlock;
                r[b] = i < n4 ? b4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int i = i0 + b * kBlock;
                if (i < n4) {
                    const float e[4] = {r[b].x, r[b].y, r[b].z, r[b].w};
                    int kk = (4 * i) / T, t = 4 * i - kk * T;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        vl[t * pitch + kk] = e[q];
                        if (++t == T) { t = 0; ++kk; }
                    }
                }
            }
        }
    } else
    for (int i0 = threadIdx.x; i0 < n; i0 += kBlock * kBatch) {
        float r[kBatch];
        int dst[kBatch];
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int i = i0 + b * kBlock;
            dst[b] = -1;
            r[b] = 0.f;
            if (i < n) {
                int t, kk;
                if (by_t) { kk = i / T; t = i - kk * T; }
                else { t = i / len; kk = i - t * len; }
                dst[b] = t * pitch + kk;
                r[b] = V[t * vs_t + static_cast<size_t>(k_begin + kk) * vs_k];
            }
        }
#pragma unroll
        for (int b = 0; b < kBatch; ++b)
            if (dst[b] >= 0) vl[dst[b]] = r[b];
    }
    // the rest: rows past T, columns past len (disjoint from the above, no barrier between)
    for (int i = T * pitch + threadIdx.x; i < TT * pitch; i += kBlock) vl[i] = 0.f;
    if (len < pitch) {
        const int tail = pitch - len;
        for (int i = threadIdx.x; i < T * tail; i += kBlock) {
            const int t = i / tail;
            vl[t * pitch + len + (i - t * tail)] = 0.f;
        }
    }
}

// k contiguous in X: a wavefront takes kThinRows<TT> rows, its lanes stride over k
// in float4 steps against V staged in LDS (each LDS read serves all the rows).
template <int TT, bool NT>
__global__ __launch_bounds__(kBlock) void thin_dot_kernel(const float* __restrict__ X, size_t xs_l,
                                                          const float* __restrict__ V, size_t vs_t, size_t vs_k,
                                                          float* C, size_t cs_l, size_t cs_t, int L, int K, int T,
                                                          float alpha, float beta) {
    extern __shared__ __attribute__((aligned(16))) float vlds[];   // [TT][K]
    stage_thin<TT>(vlds, V, vs_t, vs_k, T, 0, K, K);
    __syncthreads();
    const int lane = threadIdx.x & (kWave - 1);
    const size_t wave0 = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
    const size_t nwaves = static_cast<size_t>(gridDim.x) * (kBlock / kWave);
    const int K4 = K / 4;
    const float4* v4 = reinterpret_cast<const float4*>(vlds);
    constexpr int R = kThinRows<TT>;
    for (size_t l0 = wave0 * R; l0 < static_cast<size_t>(L); l0 += nwaves * R) {
        float acc[R][TT];
#pragma unroll
        for (int u = 0; u < R; ++u)
#pragma unroll
            for (int t = 0; t < TT; ++t) acc[u][t] = 0.f;
        for (int k4 = lane; k4 < K4; k4 += kWave) {
            float4 x[R];
#pragma unroll
            for (int u = 0; u < R; ++u) {
                const size_t l = l0 + u < static_cast<size_t>(L) ? l0 + u : L - 1;   // clamped, dropped at the store
                x[u] = load4<NT>(X + l * xs_l + 4 * static_cast<size_t>(k4));
            }
#pragma unroll
            for (int t = 0; t < TT; ++t) {
                const float4 v = v4[t * K4 + k4];
#pragma unroll
                for (int u = 0; u < R; ++u)
                    acc[u][t] += x[u].x * v.x + x[u].y * v.y + x[u].z * v.z + x[u].w * v.w;
            }
        }
        // R*TT sums over the wavefront at once: each exchange halves the number of
        // values a lane carries (the upper half of the lanes keeps the upper half of
        // the values), so 64 lanes x NV values cost NV - 1 + log2(64 / NV) exchanges
        // instead of 6 per value
        constexpr int NV = R * TT;
        float v[NV];
#pragma unroll
        for (int u = 0; u < R; ++u)
#pragma unroll
            for (int t = 0; t < TT; ++t) v[u * TT + t] = acc[u][t];
        const int idx = wave_sum_many<NV>(v, lane);
        const int u = idx / TT, t = idx - u * TT;
        if (idx >= 0 && l0 + u < static_cast<size_t>(L) && t < T) {
            float* dst = C + (l0 + u) * cs_l + t * cs_t;
            float o = alpha * v[0];
            if (beta != 0.0f) o += beta * *dst;
            *dst = o;
        }
    }
}

// The dot form with K cut into chunks across workgroups: for a short L (a 10 x 128 x 12544
// product has 128 rows of X: whole-K rows would occupy eight workgroups) or a V that does not
// fit LDS whole.  A workgroup stages its chunk's slice of V once and walks rows_per_wg rows of
// X against it, kThinRows<TT> rows per wavefront and pass; the partial sums go to
// part[chunk][t*L + l] for the combine kernel.
template <int TT, bool NT>
__global__ __launch_bounds__(kBlock) void thin_dot_partial_kernel(const float* __restrict__ X, size_t xs_l,
                                                                  const float* __restrict__ V, size_t vs_t,
                                                                  size_t vs_k, float* part, int L, int K, int T,
                                                                  int chunk_len, int rows_per_wg) {
    extern __shared__ __attribute__((aligned(16))) float vlds[];   // [TT][chunk_len], chunk_len % 4 == 0
    const int k_begin = blockIdx.y * chunk_len;
    const int len = (K - k_begin) < chunk_len ? (K - k_begin) : chunk_len;   // a multiple of 4, as K is
    const int lane = threadIdx.x & (kWave - 1);
    constexpr int R = kThinRows<TT>;
    constexpr int NW = kBlock / kWave;
    constexpr int kIter = kThinDotChunkMax / 4 / kWave;   // float4 steps a lane takes through the longest chunk
    const int C4 = chunk_len / 4, len4 = len / 4;
    const size_t row0 = static_cast<size_t>(blockIdx.x) * rows_per_wg + (threadIdx.x / kWave) * R;
    float4 x[kIter][R];
    auto fetch = [&](size_t l0) {
#pragma unroll
        for (int it = 0; it < kIter; ++it) {
            const int k4 = lane + it * kWave;
#pragma unroll
            for (int u = 0; u < R; ++u) {
                const size_t l = l0 + u < static_cast<size_t>(L) ? l0 + u : L - 1;   // clamped, dropped at the store
                x[it][u] = k4 < len4 ? load4<NT>(X + l * xs_l + k_begin + 4 * static_cast<size_t>(k4))
                                     : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
    };
    // the first rows are requested before V is staged, so that the two round trips to memory overlap
    if (row0 < static_cast<size_t>(L)) fetch(row0);
    stage_thin<TT>(vlds, V, vs_t, vs_k, T, k_begin, len, chunk_len);
    __syncthreads();
    const float4* v4 = reinterpret_cast<const float4*>(vlds);
    for (int pass = 0; pass * NW * R < rows_per_wg; ++pass) {
        const size_t l0 = row0 + static_cast<size_t>(pass) * NW * R;
        if (l0 >= static_cast<size_t>(L)) break;
        if (pass > 0) fetch(l0);
        float acc[R][TT];
#pragma unroll
        for (int u = 0; u < R; ++u)
#pragma unroll
            for (int t = 0; t < TT; ++t) acc[u][t] = 0.f;
#pragma unroll
        for (int it = 0; it < kIter; ++it) {
            const int k4 = lane + it * kWave;
            if (k4 < len4) {
#pragma unroll
                for (int t = 0; t < TT; ++t) {
                    const float4 v = v4[t * C4 + k4];
#pragma unroll
                    for (int u = 0; u < R; ++u)
                        acc[u][t] += x[it][u].x * v.x + x[it][u].y * v.y + x[it][u].z * v.z + x[it][u].w * v.w;
                }
            }
        }
        constexpr int NV = R * TT;
        float v[NV];
#pragma unroll
        for (int u = 0; u < R; ++u)
#pragma unroll
            for (int t = 0; t < TT; ++t) v[u * TT + t] = acc[u][t];
        const int idx = wave_sum_many<NV>(v, lane);
        const int u = idx / TT, t = idx - u * TT;
        if (idx >= 0 && l0 + u < static_cast<size_t>(L) && t < T)
            part[(static_cast<size_t>(blockIdx.y) * T + t) * L + l0 + u] = v[0];
    }
}

// l contiguous in X: lanes hold four rows each (a wavefront reads 1 KB of one
// column), the block's waves split the k of a chunk eight at a time, and the
// chunk's slice of V sits in LDS as [t][chunk_len], zero-filled past the end
// of K, read as broadcast float4.  Partial sums go to part[chunk][t*L + l].
template <int TT, bool NT>
__global__ __launch_bounds__(kBlock) void thin_axpy_partial_kernel(const float* __restrict__ X, size_t xs_k,
                                                                   const float* __restrict__ V, size_t vs_t,
                                                                   size_t vs_k, float* part, int L, int K, int T,
                                                                   int chunk_len) {
    constexpr int NW = kBlock / kWave;
    constexpr int U = 8;   // columns in flight per wavefront; chunk_len % U == 0
    extern __shared__ __attribute__((aligned(16))) float vl[];   // [TT][chunk_len]
    __shared__ float4 red[NW][TT < 4 ? TT : 4][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int l = (blockIdx.x * kWave + lane) * 4;
    const bool live = l < L;
    const int k_begin = blockIdx.y * chunk_len;
    const int len = (K - k_begin) < chunk_len ? (K - k_begin) : chunk_len;
    const float* xp = X + (live ? l : 0) + static_cast<size_t>(k_begin) * xs_k;
    auto fetch = [&](float4 (&x)[U], int kk) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int c = kk + u < len ? kk + u : len - 1;   // clamped; its V entry is zero
            x[u] = load4<NT>(xp + static_cast<size_t>(c) * xs_k);
        }
    };
    // the first columns are requested before V is staged, so that the two round trips to memory overlap
    float4 x[U];
    int kk = wave * U;
    if (kk < len) fetch(x, kk);
    stage_thin<TT>(vl, V, vs_t, vs_k, T, k_begin, len, chunk_len);
    __syncthreads();
    float4 acc[TT];
#pragma unroll
    for (int t = 0; t < TT; ++t) acc[t] = make_float4(0.f, 0.f, 0.f, 0.f);
    while (kk < len) {
#pragma unroll
        for (int t = 0; t < TT; ++t) {
#pragma unroll
            for (int q = 0; q < U / 4; ++q) {
                const float4 v = *reinterpret_cast<const float4*>(vl + t * chunk_len + kk + 4 * q);
                const float vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    acc[t].x += x[4 * q + e].x * vv[e]; acc[t].y += x[4 * q + e].y * vv[e];
                    acc[t].z += x[4 * q + e].z * vv[e]; acc[t].w += x[4 * q + e].w * vv[e];
                }
            }
        }
        kk += NW * U;
        if (kk < len) fetch(x, kk);
    }
    // the four waves' sums, four vectors per round: wave w adds vector t0 + w of the four waves in wave order
    constexpr int G = TT < 4 ? TT : 4;
#pragma unroll
    for (int t0 = 0; t0 < TT; t0 += G) {
        if (t0 < T) {   // T is uniform: every thread takes the same barriers
#pragma unroll
            for (int q = 0; q < G; ++q) red[wave][q][lane] = acc[t0 + q];
            __syncthreads();
            const int t = t0 + wave;
            if (wave < G && t < T && live) {
                float4 sum = red[0][wave][lane];
#pragma unroll
                for (int w = 1; w < NW; ++w) {
                    const float4 o = red[w][wave][lane];
                    sum.x += o.x; sum.y += o.y; sum.z += o.z; sum.w += o.w;
                }
                *reinterpret_cast<float4*>(part + (static_cast<size_t>(blockIdx.y) * T + t) * L + l) = sum;
            }
            __syncthreads();
        }
    }
}

}  // namespace

namespace {
int gemv_plain(const float* A, const float* x, float* y, int m, int n, bool trans, size_t lda,
               size_t incx, size_t incy, float alpha, float beta) {
    hipStream_t s = stream();
    if (trans) {
        gemv_t_kernel<<<grid_cover(n, kBlock / kWave), kBlock, 0, s>>>(A, x, y, m, n, lda, incx, incy,
                                                                         alpha, beta);
        return launch_rc();
    }
    const int row_blocks = (m + kWave - 1) / kWave;
    int chunks = static_cast<int>((static_cast<size_t>(num_cus()) * 4 + row_blocks - 1) / row_blocks);
    if (chunks > n / 32) chunks = n / 32;
    if (chunks < 1) chunks = 1;
    if (chunks > 4096) chunks = 4096;
    while (chunks > 1 && static_cast<size_t>(chunks) * m > kWorkspaceFloats) --chunks;
    if (static_cast<size_t>(chunks) * m > kWorkspaceFloats) return -1;
    const int chunk_len = (n + chunks - 1) / chunks;
    chunks = (n + chunk_len - 1) / chunk_len;
    float* part = workspace();
    if (!part) return -2;
    gemv_n_partial_kernel<<<dim3(row_blocks, chunks), kBlock, 0, s>>>(A, x, part, m, n, lda, incx, chunk_len);
    gemv_n_combine_kernel<<<(m + kWave - 1) / kWave, kGemvCombineBlock, 0, s>>>(y, part, m, chunks, m, incy, 0,
                                                                                alpha, beta);
    return launch_rc();
}
}  // namespace

namespace {

struct ThinArgs {
    const float* X; size_t xs_l, xs_k;
    const float* V; size_t vs_t, vs_k;
    float* C; size_t cs_l, cs_t;
    int L, K, T;
    float alpha, beta;
};

// The dot form keeps all of V in LDS and gives a wavefront whole rows when there are rows enough
// to fill the chip; otherwise K is cut into chunks.
bool thin_dot_whole_k(const ThinArgs& a) {
    return a.L >= 256 && static_cast<size_t>(thin_tt(a.T)) * a.K * sizeof(float) <= 64 * 1024;
}
int thin_dot_rows_per_wg(const ThinArgs& a, int tt) {
    const int base = (tt == 1 ? 4 : tt <= 4 ? 2 : tt <= 8 ? 4 : 2) * (kBlock / kWave);   // one pass of the four waves
    const long long chunks_min = (a.K + kThinDotChunkMax - 1) / kThinDotChunkMax;
    int rows = base;
    while (rows < 8 * base && (a.L / (2 * rows)) * chunks_min >= 4ll * num_cus()) rows *= 2;
    return rows;
}
int thin_dot_chunk_len(const ThinArgs& a, int tt, int row_groups) {
    long long chunks = (2ll * num_cus() + row_groups - 1) / row_groups;
    if (chunks > a.K / 64) chunks = a.K / 64;
    if (chunks < 1) chunks = 1;
    int chunk_len = static_cast<int>(((a.K + chunks - 1) / chunks + 3) / 4 * 4);
    (void)tt;   // V's slice of a chunk: at most 16 x 512 floats = 32 KB
    return chunk_len > kThinDotChunkMax ? kThinDotChunkMax : chunk_len;
}

template <int TT>
int thin_launch(const ThinArgs& a) {
    hipStream_t s = stream();
    // the big operand is read once: past the cache size with the streaming hint
    const bool nt = streams_past_cache(static_cast<size_t>(a.L) * a.K * sizeof(float));
    if (a.xs_k == 1 && !thin_dot_whole_k(a)) {
        // K in chunks: enough of them for two workgroups per CU, V's slice within 32 KB; with many rows a
        // workgroup walks up to 64 of them against one staged slice
        const int rows_per_wg = thin_dot_rows_per_wg(a, TT);
        const int row_groups = (a.L + rows_per_wg - 1) / rows_per_wg;
        const int chunk_len = thin_dot_chunk_len(a, TT, row_groups);
        const int chunks = (a.K + chunk_len - 1) / chunk_len;
        const size_t outs = static_cast<size_t>(a.T) * a.L;
        if (outs * chunks > kWorkspaceFloats) return -1;            // thin_ok() rules this out
        float* part = workspace();
        if (!part) return -2;
        const size_t lds = static_cast<size_t>(TT) * chunk_len * sizeof(float);
        if (nt)
            thin_dot_partial_kernel<TT, true><<<dim3(row_groups, chunks), kBlock, lds, s>>>(a.X, a.xs_l, a.V, a.vs_t, a.vs_k,
                                                                                         part, a.L, a.K, a.T, chunk_len, rows_per_wg);
        else
            thin_dot_partial_kernel<TT, false><<<dim3(row_groups, chunks), kBlock, lds, s>>>(a.X, a.xs_l, a.V, a.vs_t, a.vs_k,
                                                                                          part, a.L, a.K, a.T, chunk_len, rows_per_wg);
        launch_thin_combine(a.C, part, outs, chunks, a.L, a.cs_l, a.cs_t, a.alpha, a.beta, s);
        return launch_rc();
    }
    if (a.xs_k == 1) {
        const size_t groups = (static_cast<size_t>(a.L) + kThinRows<TT> - 1) / kThinRows<TT>;
        const unsigned grid = grid_for(groups, kBlock / kWave, 8);
        if (nt)
            thin_dot_kernel<TT, true><<<grid, kBlock, static_cast<size_t>(TT) * a.K * sizeof(float), s>>>(
                a.X, a.xs_l, a.V, a.vs_t, a.vs_k, a.C, a.cs_l, a.cs_t, a.L, a.K, a.T, a.alpha, a.beta);
        else
            thin_dot_kernel<TT, false><<<grid, kBlock, static_cast<size_t>(TT) * a.K * sizeof(float), s>>>(
                a.X, a.xs_l, a.V, a.vs_t, a.vs_k, a.C, a.cs_l, a.cs_t, a.L, a.K, a.T, a.alpha, a.beta);
        return launch_rc();
    }
    const int row_blocks = (a.L / 4 + kWave - 1) / kWave;
    int chunks = static_cast<int>((static_cast<size_t>(num_cus()) * 4 + row_blocks - 1) / row_blocks);
    // chunks of 64 k and more; of 32 where the rows alone give the chip little to do (a 256 x 16 x 4096
    // gradient is one row block)
    const int min_chunk = row_blocks * 8 <= num_cus() ? 32 : 64;
    if (chunks > a.K / min_chunk) chunks = a.K / min_chunk;
    if (chunks < 1) chunks = 1;
    int chunk_len = ((a.K + chunks - 1) / chunks + 7) / 8 * 8;
    if (chunk_len > thin_chunk_max(TT)) chunk_len = thin_chunk_max(TT);   // V's slice of a chunk stays within 32 KB of LDS
    chunks = (a.K + chunk_len - 1) / chunk_len;
    const size_t outs = static_cast<size_t>(a.T) * a.L;
    if (outs * chunks > kWorkspaceFloats) return -1;            // thin_ok() rules this out
    float* part = workspace();
    if (!part) return -2;
    if (nt)
        thin_axpy_partial_kernel<TT, true><<<dim3(row_blocks, chunks), kBlock,
                                             static_cast<size_t>(TT) * chunk_len * sizeof(float), s>>>(
            a.X, a.xs_k, a.V, a.vs_t, a.vs_k, part, a.L, a.K, a.T, chunk_len);
    else
        thin_axpy_partial_kernel<TT, false><<<dim3(row_blocks, chunks), kBlock,
                                              static_cast<size_t>(TT) * chunk_len * sizeof(float), s>>>(
            a.X, a.xs_k, a.V, a.vs_t, a.vs_k, part, a.L, a.K, a.T, chunk_len);
    launch_thin_combine(a.C, part, outs, chunks, a.L, a.cs_l, a.cs_t, a.alpha, a.beta, s);
    return launch_rc();
}

// Whether the thin forms apply: float4 access to X in its contiguous direction,
// V small enough for LDS in the dot form, partial sums that fit the workspace.
bool thin_ok(const ThinArgs& a) {
    if (a.T > kThinMax || !aligned16(a.X)) return false;
    if (a.xs_k == 1) {
        if (!(a.K % 4 == 0 && a.xs_l % 4 == 0 && a.K >= 64)) return false;
        if (thin_dot_whole_k(a)) return true;
        // chunked: at least a wavefront's worth of rows, partial sums within the workspace
        if (a.L < 16) return false;
        const int tt = thin_tt(a.T);
        const int per_wg = thin_dot_rows_per_wg(a, tt);
        const int row_groups = (a.L + per_wg - 1) / per_wg;
        const int chunk_len = thin_dot_chunk_len(a, tt, row_groups);
        const size_t chunks = (static_cast<size_t>(a.K) + chunk_len - 1) / chunk_len;
        return chunks <= 65535 && static_cast<size_t>(a.T) * a.L * chunks <= kWorkspaceFloats;
    }
    if (a.L < 64) return false;
    // partial sums of every chunk must fit the workspace even at the longest chunk
    const size_t min_chunks = (static_cast<size_t>(a.K) + thin_chunk_max(thin_tt(a.T)) - 1) / thin_chunk_max(thin_tt(a.T));
    const size_t row_blocks = (static_cast<size_t>(a.L) / 4 + kWave - 1) / kWave;
    const size_t want = (static_cast<size_t>(num_cus()) * 4 + row_blocks - 1) / row_blocks;
    const size_t chunks = want > min_chunks ? want : min_chunks;
    return a.xs_l == 1 && a.L % 4 == 0 && a.xs_k % 4 == 0 && a.K >= 64 &&
           static_cast<size_t>(a.T) * a.L * (chunks + 1) <= kWorkspaceFloats;
}

int thin_impl(const ThinArgs& a) {
    if (a.T == 1) return thin_launch<1>(a);
    if (a.T <= 4) return thin_launch<4>(a);
    return a.T <= 8 ? thin_launch<8>(a) : thin_launch<16>(a);
}

}  // namespace

namespace {
// y[j] = alpha*<A[:,j], x> + beta*y[j] for long columns (m >= 1024, m % 4 == 0, lda % 4 == 0,
// aligned A and x, incx == 1): a workgroup takes four columns, its four waves a quarter
// of the rows each, eight float4 loads of A in flight per lane; x comes through the caches.
constexpr int kGemvTCols = 4;
template <bool NT>
__global__ __launch_bounds__(kBlock) void gemv_t_split_kernel(const float* __restrict__ A,
                                                              const float* __restrict__ x, float* y, int m,
                                                              int n, size_t lda, size_t incy, float alpha,
                                                              float beta) {
    constexpr int NW = kBlock / kWave;
    __shared__ float red[NW][kGemvTCols];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const size_t j0 = static_cast<size_t>(blockIdx.x) * kGemvTCols;
    const float* col[kGemvTCols];
#pragma unroll
    for (int c = 0; c < kGemvTCols; ++c) {
        const size_t j = j0 + c < static_cast<size_t>(n) ? j0 + c : n - 1;   // clamped, dropped at the store
        col[c] = A + j * lda;
    }
    const float4* x4 = reinterpret_cast<const float4*>(x);
    const int m4 = m / 4;
    float acc[kGemvTCols] = {0.f, 0.f, 0.f, 0.f};
    int i = wave * kWave + lane;
    for (; i + kBlock < m4; i += 2 * kBlock) {
        float4 a[2][kGemvTCols];
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int c = 0; c < kGemvTCols; ++c) a[u][c] = load4<NT>(col[c] + 4 * static_cast<size_t>(i + u * kBlock));
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const float4 xv = x4[i + u * kBlock];
#pragma unroll
            for (int c = 0; c < kGemvTCols; ++c)
                acc[c] += a[u][c].x * xv.x + a[u][c].y * xv.y + a[u][c].z * xv.z + a[u][c].w * xv.w;
        }
    }
    for (; i < m4; i += kBlock) {
        const float4 xv = x4[i];
#pragma unroll
        for (int c = 0; c < kGemvTCols; ++c) {
            const float4 av = load4<NT>(col[c] + 4 * static_cast<size_t>(i));
            acc[c] += av.x * xv.x + av.y * xv.y + av.z * xv.z + av.w * xv.w;
        }
    }
    const int idx = wave_sum_many<kGemvTCols>(acc, lane);
    if (idx >= 0) red[wave][idx] = acc[0];
    __syncthreads();
    if (threadIdx.x < kGemvTCols && j0 + threadIdx.x < static_cast<size_t>(n)) {
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) sum += red[w][threadIdx.x];
        float* dst = y + (j0 + threadIdx.x) * incy;
        float r = alpha * sum;
        if (beta != 0.0f) r += beta * *dst;
        *dst = r;
    }
}
}  // namespace

// y = alpha*op(A)*x + beta*y, A the physical m x n matrix.  A matrix-vector product is the
// thin product with one vector: those kernels keep several float4 loads of A in flight per
// lane, which the plain kernels do not; the plain ones take what the thin forms exclude
// (unaligned or short operands).
int gemv_impl(const float* A, const float* x, float* y, int m, int n, bool trans, size_t lda,
              size_t incx, size_t incy, float alpha, float beta) {
    const ThinArgs t = trans ? ThinArgs{A, lda, 1, x, 0, incx, y, incy, 0, n, m, 1, alpha, beta}
                             : ThinArgs{A, 1, lda, x, 0, incx, y, incy, 0, m, n, 1, alpha, beta};
    if (trans && incx == 1 && m >= 1024 && m % 4 == 0 && lda % 4 == 0 && aligned16(A) && aligned16(x)) {
        const unsigned grid = static_cast<unsigned>((static_cast<size_t>(n) + kGemvTCols - 1) / kGemvTCols);
        if (streams_past_cache(static_cast<size_t>(m) * n * sizeof(float)))
            gemv_t_split_kernel<true><<<grid, kBlock, 0, stream()>>>(A, x, y, m, n, lda, incy, alpha, beta);
        else
            gemv_t_split_kernel<false><<<grid, kBlock, 0, stream()>>>(A, x, y, m, n, lda, incy, alpha, beta);
        return launch_rc();
    }
    if (thin_ok(t)) return thin_impl(t);
    return gemv_plain(A, x, y, m, n, trans, lda, incx, incy, alpha, beta);
}

// C = alpha*op(A)*op(B) + beta*C through the thin forms when they apply;
// *taken says whether they did.
int gemm_thin(const float* A, const float* B, float* C, int m, int n, int k, bool trans_a, bool trans_b, int lda,
              int ldb, int ldc, float alpha, float beta, bool* taken) {
    *taken = false;
    if (n <= kThinMax || m <= kThinMax) {
        const size_t ula = static_cast<size_t>(lda), ulb = static_cast<size_t>(ldb), ulc = static_cast<size_t>(ldc);
        // op(A)(i,p) and op(B)(p,j) as (extent stride, k stride) pairs
        const size_t a_i = trans_a ? ula : 1, a_k = trans_a ? 1 : ula;
        const size_t b_j = trans_b ? 1 : ulb, b_k = trans_b ? ulb : 1;
        const ThinArgs t = n <= m ? ThinArgs{A, a_i, a_k, B, b_j, b_k, C, 1, ulc, m, k, n, alpha, beta}
                                  : ThinArgs{B, b_j, b_k, A, a_i, a_k, C, ulc, 1, n, k, m, alpha, beta};
        if (thin_ok(t)) {
            *taken = true;
            return thin_impl(t);
        }
    }
    return 0;
}

}  // namespace jz

using namespace jz;

JZ_API int jzhip_gemv(const float* A, const float* x, float* y, int m, int n, int trans_a, int lda,
                      int incx, int incy, float alpha, float beta) {
    if (m <= 0 || n <= 0 || lda < m) return -1;
    if (!A || !x || !y) return -1;
    if (incx <= 0 || incy <= 0) return -1;
    return gemv_impl(A, x, y, m, n, trans_a != 0, lda, incx, incy, alpha, beta);
}
