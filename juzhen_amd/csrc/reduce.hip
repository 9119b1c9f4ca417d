// Fixed-function reductions: column / row sums, Frobenius norm, column max
// and argmax.  All are HBM-bound single reads of the operand
// (4*(numrow*numcol + outputs) bytes).  Within a wavefront values are combined
// with DPP row operations, across waves through LDS, and across workgroups
// through a two-phase partial buffer, so results are deterministic (no float
// atomics on global memory).
#include "common.hpp"

#include <atomic>
#include <cmath>

namespace jz {
namespace {

// ── column sums: out[j] = sum_i a[j*ld + i] ──────────────────────────────
// One wavefront per (column, row-chunk).  VEC=4 uses float4 loads and needs
// ld % 4 == 0, a 16-byte aligned base and chunk boundaries that are multiples
// of 4.
template <int VEC, bool NT = false>
__global__ __launch_bounds__(kBlock) void sum_cols_kernel(float* out, const float* a, int numrow,
                                                          int numcol, size_t ld, int chunks,
                                                          int chunk_len) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t wave0 = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
    const size_t nwaves = static_cast<size_t>(gridDim.x) * (kBlock / kWave);
    const size_t items = static_cast<size_t>(numcol) * chunks;
    for (size_t it = wave0; it < items; it += nwaves) {
        const int col = static_cast<int>(it % numcol);
        const int chunk = static_cast<int>(it / numcol);
        const int r_begin = chunk * chunk_len;
        int r_end = r_begin + chunk_len;
        if (r_end > numrow) r_end = numrow;
        const float* p = a + static_cast<size_t>(col) * ld;
        float acc0 = 0.f, acc1 = 0.f;
        if constexpr (VEC == 4) {
            const int v_end = r_begin + ((r_end - r_begin) / 4) * 4;
            int r = r_begin + lane * 4;
            // four float4 loads in flight per lane (4 KB per wave), then two
            float acc2 = 0.f, acc3 = 0.f;
            for (; r + 3 * kWave * 4 < v_end; r += 4 * kWave * 4) {
                const float4 x = load4<NT>(p + r);
                const float4 y = load4<NT>(p + r + kWave * 4);
                const float4 z = load4<NT>(p + r + 2 * kWave * 4);
                const float4 w = load4<NT>(p + r + 3 * kWave * 4);
                acc0 += (x.x + x.y) + (x.z + x.w);
                acc1 += (y.x + y.y) + (y.z + y.w);
                acc2 += (z.x + z.y) + (z.z + z.w);
                acc3 += (w.x + w.y) + (w.z + w.w);
            }
            acc0 += acc2;
            acc1 += acc3;
            for (; r + kWave * 4 < v_end; r += 2 * kWave * 4) {
                const float4 x = load4<NT>(p + r);
                const float4 y = load4<NT>(p + r + kWave * 4);
                acc0 += (x.x + x.y) + (x.z + x.w);
                acc1 += (y.x + y.y) + (y.z + y.w);
            }
            for (; r < v_end; r += kWave * 4) {
                const float4 x = load4<NT>(p + r);
                acc0 += (x.x + x.y) + (x.z + x.w);
            }
            for (int t = v_end + lane; t < r_end; t += kWave) acc1 += p[t];
        } else {
            for (int r = r_begin + lane; r < r_end; r += kWave) acc0 += p[r];
        }
        const float s = wave_sum(acc0 + acc1);
        if (lane == 0) out[static_cast<size_t>(chunk) * numcol + col] = s;
    }
}

// out[i] = sum_{c<chunks} part[c*n + i].  A block owns 64 outputs; its sixteen
// waves take interleaved chunks (lanes stay on consecutive i, so reads are
// coalesced), eight loads in flight each, and are combined through LDS.
constexpr int kCombineBlock = 1024;
__global__ __launch_bounds__(kCombineBlock) void combine_partials_kernel(float* out, const float* part,
                                                                         int n, int chunks) {
    constexpr int NW = kCombineBlock / kWave;
    constexpr int U = 8;
    __shared__ float red[NW][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int i = blockIdx.x * kWave + lane;
    float acc = 0.f;
    if (i < n) {
        const float* p = part + i;
        int c = wave;
        for (; c + (U - 1) * NW < chunks; c += U * NW) {
            float x[U];
#pragma unroll
            for (int u = 0; u < U; ++u) x[u] = p[static_cast<size_t>(c + u * NW) * n];
#pragma unroll
            for (int u = 0; u < U; ++u) acc += x[u];
        }
        for (; c < chunks; c += NW) acc += p[static_cast<size_t>(c) * n];
    }
    red[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && i < n) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) s += red[w][lane];
        out[i] = s;
    }
}

// ── row sums: out[i] = sum_j a[j*ld + i] ─────────────────────────────────
// Lanes run along rows (the contiguous dimension); the four waves of a block
// take interleaved columns of the block's column chunk and are combined
// through LDS.  VEC rows per lane.
template <int VEC, bool NT = false>
__global__ __launch_bounds__(kBlock) void sum_rows_kernel(float* out, const float* a, int numrow,
                                                          int numcol, size_t ld, int chunk_len) {
    constexpr int NW = kBlock / kWave;
    __shared__ float red[NW][kWave * VEC];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int row = (blockIdx.x * kWave + lane) * VEC;
    const int chunk = blockIdx.y;
    const int c_begin = chunk * chunk_len;
    int c_end = c_begin + chunk_len;
    if (c_end > numcol) c_end = numcol;

    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.f;
    if (row < numrow) {
        if constexpr (VEC == 4) {
            // numrow % 4 == 0 is guaranteed by the launcher
            int c = c_begin + wave;
            for (; c + NW < c_end; c += 2 * NW) {
                const float4 x = load4<NT>(a + static_cast<size_t>(c) * ld + row);
                const float4 y =
                    load4<NT>(a + static_cast<size_t>(c + NW) * ld + row);
                acc[0] += x.x; acc[1] += x.y; acc[2] += x.z; acc[3] += x.w;
                acc[0] += y.x; acc[1] += y.y; acc[2] += y.z; acc[3] += y.w;
            }
            for (; c < c_end; c += NW) {
                const float4 x = load4<NT>(a + static_cast<size_t>(c) * ld + row);
                acc[0] += x.x; acc[1] += x.y; acc[2] += x.z; acc[3] += x.w;
            }
        } else {
            for (int c = c_begin + wave; c < c_end; c += NW) acc[0] += a[static_cast<size_t>(c) * ld + row];
        }
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) red[wave][lane * VEC + v] = acc[v];
    __syncthreads();
    if (wave == 0 && row < numrow) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) s += red[w][lane * VEC + v];
            out[static_cast<size_t>(chunk) * numrow + row + v] = s;
        }
    }
}

// Row sums of a short, contiguous matrix (numrow <= 64, ld == numrow): the
// buffer is read as one flat stream; each thread strides by a multiple of
// numrow so it always lands on the same row, then threads of equal row are
// combined through LDS.
__global__ __launch_bounds__(kBlock) void sum_rows_short_kernel(float* part, const float* a,
                                                                int numrow, size_t total,
                                                                int active, size_t span) {
    __shared__ float red[kBlock];
    const int t = threadIdx.x;
    const size_t begin = static_cast<size_t>(blockIdx.x) * span;  // multiple of numrow
    size_t end = begin + span;
    if (end > total) end = total;
    float acc0 = 0.f, acc1 = 0.f;
    if (t < active) {
        size_t i = begin + t;
        for (; i + active < end; i += 2 * static_cast<size_t>(active)) {
            acc0 += a[i];
            acc1 += a[i + active];
        }
        if (i < end) acc0 += a[i];
    }
    red[t] = acc0 + acc1;
    __syncthreads();
    // threads of equal row are numrow apart: halve the number of groups of numrow threads
    // until one is left (with one row a single thread adding 256 values in turn took 9 of
    // the kernel's 11 us)
    for (int groups = active / numrow; groups > 1;) {
        const int half = (groups + 1) / 2;
        if (t < (groups - half) * numrow) red[t] += red[t + half * numrow];
        __syncthreads();
        groups = half;
    }
    if (t < numrow) part[static_cast<size_t>(blockIdx.x) * numrow + t] = red[t];
}

// ── flat sum of squares (norm) ───────────────────────────────────────────
template <bool NT>
__global__ __launch_bounds__(kBlock) void sumsq_partial_kernel(float* part, const float* x, size_t n,
                                                               int vec_ok) {
    __shared__ float red[kBlock / kWave];
    const size_t stride = static_cast<size_t>(gridDim.x) * kBlock;
    const size_t tid = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x;
    float acc0 = 0.f, acc1 = 0.f;
    if (vec_ok) {
        const size_t n4 = n / 4;
        const float4* x4 = reinterpret_cast<const float4*>(x);
        size_t i = tid;
        for (; i + stride < n4; i += 2 * stride) {
            const float4 p = load4<NT>(x + 4 * i), q = load4<NT>(x + 4 * (i + stride));
            acc0 += (p.x * p.x + p.y * p.y) + (p.z * p.z + p.w * p.w);
            acc1 += (q.x * q.x + q.y * q.y) + (q.z * q.z + q.w * q.w);
        }
        if (i < n4) {
            const float4 p = load4<NT>(x + 4 * i);
            acc0 += (p.x * p.x + p.y * p.y) + (p.z * p.z + p.w * p.w);
        }
        for (size_t j = n4 * 4 + tid; j < n; j += stride) acc1 += x[j] * x[j];
    } else {
        for (size_t i = tid; i < n; i += stride) acc0 += x[i] * x[i];
    }
    const float s = block_allreduce<kBlock / kWave>(acc0 + acc1, SumOp{}, red, 0.f);
    if (threadIdx.x == 0) part[blockIdx.x] = s;
}

__global__ __launch_bounds__(kBlock) void sqrt_sum_kernel(float* out, const float* part, int n) {
    __shared__ float red[kBlock / kWave];
    float acc = 0.f;
    for (int i = threadIdx.x; i < n; i += kBlock) acc += part[i];
    const float s = block_allreduce<kBlock / kWave>(acc, SumOp{}, red, 0.f);
    if (threadIdx.x == 0) out[0] = sqrtf(s);
}

// ── mean squared error value: scale * sum((target - pred)^2) ─────────────
// (LossLayer::eval, ml/layer.hpp:223-226: difference, square, two sums and a scaling as five
// matrix operations; here the differences and squares round the same way and the sums run
// over the flat buffer.)  A single workgroup writes the scaled result itself.
template <bool NT>
__global__ __launch_bounds__(kBlock) void sqdiff_partial_kernel(float* part, const float* __restrict__ target,
                                                                const float* __restrict__ pred, size_t n,
                                                                float scale) {
    __shared__ float red[kBlock / kWave];
    const size_t stride = static_cast<size_t>(gridDim.x) * kBlock;
    const size_t tid = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x;
    float acc0 = 0.f, acc1 = 0.f;
    size_t i = tid;
    for (; i + stride < n; i += 2 * stride) {
        const float d0 = load1<NT>(target + i) - load1<NT>(pred + i);
        const float d1 = load1<NT>(target + i + stride) - load1<NT>(pred + i + stride);
        acc0 += d0 * d0;
        acc1 += d1 * d1;
    }
    if (i < n) {
        const float d0 = target[i] - pred[i];
        acc0 += d0 * d0;
    }
    const float s = block_allreduce<kBlock / kWave>(acc0 + acc1, SumOp{}, red, 0.f);
    if (threadIdx.x == 0) part[blockIdx.x] = gridDim.x == 1 ? s * scale : s;
}

__global__ __launch_bounds__(kBlock) void scaled_sum_kernel(float* out, const float* part, int n, float scale) {
    __shared__ float red[kBlock / kWave];
    float acc = 0.f;
    for (int i = threadIdx.x; i < n; i += kBlock) acc += part[i];
    const float s = block_allreduce<kBlock / kWave>(acc, SumOp{}, red, 0.f);
    if (threadIdx.x == 0) out[0] = s * scale;
}

// ── column max / argmax: one wavefront per column ────────────────────────
template <bool ARG, bool NT>
__global__ __launch_bounds__(kBlock) void max_cols_kernel(float* out_val, int32_t* out_idx,
                                                          const float* a, int numrow, int numcol,
                                                          size_t ld) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t wave0 = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
    const size_t nwaves = static_cast<size_t>(gridDim.x) * (kBlock / kWave);
    for (size_t col = wave0; col < static_cast<size_t>(numcol); col += nwaves) {
        const float* p = a + col * ld;
        // std::max_element order: keep the incumbent unless a later element is
        // strictly greater, so the first maximum wins (ml/util.cuh:104-110)
        float best = -INFINITY;
        int bidx = 0x7fffffff;
        if (lane < numrow) {
            best = p[lane];
            bidx = lane;
        }
        int r = lane + kWave;
        // eight loads in flight per lane, visited in row order
        for (; r + 7 * kWave < numrow; r += 8 * kWave) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = load1<NT>(p + r + u * kWave);
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (best < v[u]) {
                    best = v[u];
                    bidx = r + u * kWave;
                }
            }
        }
        for (; r < numrow; r += kWave) {
            const float v = p[r];
            if (best < v) {
                best = v;
                bidx = r;
            }
        }
        if constexpr (ARG) {
            // butterfly on (value, index): larger value wins, ties -> smaller index
#pragma unroll
            for (int off = 1; off < kWave; off <<= 1) {
                const float ov = __shfl_xor(best, off, kWave);
                const int oi = __shfl_xor(bidx, off, kWave);
                if (ov > best || (ov == best && oi < bidx)) {
                    best = ov;
                    bidx = oi;
                }
            }
            if (lane == 0) out_idx[col] = bidx;
        } else {
            const float m = wave_max(best);
            if (lane == 0) out_val[col] = m;
        }
    }
}

// predict_one_hot (ml/util.cuh:258-279) in one launch: the column's maximum as the
// generic chain's functor finds it (strictly-greater updates from the lowest value, so
// NaNs never become the maximum), then x - max > -1e-5 evaluated in double, as the
// chain's element-wise functor does after its float subtraction.  A wave per column;
// the second sweep over the column is served by the cache.
__global__ __launch_bounds__(kBlock) void one_hot_max_cols_kernel(float* out, const float* a, int numrow,
                                                                  int numcol, size_t ld) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t wave0 = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
    const size_t nwaves = static_cast<size_t>(gridDim.x) * (kBlock / kWave);
    for (size_t col = wave0; col < static_cast<size_t>(numcol); col += nwaves) {
        const float* p = a + col * ld;
        float* q = out + col * static_cast<size_t>(numrow);
        float best = -INFINITY;
        int r = lane;
        for (; r + 7 * kWave < numrow; r += 8 * kWave) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = p[r + u * kWave];
#pragma unroll
            for (int u = 0; u < 8; ++u) best = v[u] > best ? v[u] : best;
        }
        for (; r < numrow; r += kWave) {
            const float v = p[r];
            best = v > best ? v : best;
        }
        const float m = wave_max(best);
        for (r = lane; r < numrow; r += kWave) {
            const float d = p[r] - m;
            q[r] = static_cast<double>(d) > -1e-5 ? 1.0f : 0.0f;
        }
    }
}

int pick_chunks(size_t independent, size_t length, size_t min_len) {
    // enough (independent x chunks) work items to give every SIMD a few waves
    const size_t want = static_cast<size_t>(num_cus()) * 16;
    if (independent >= want) return 1;
    size_t chunks = (want + independent - 1) / independent;
    const size_t max_chunks = length / min_len;
    if (chunks > max_chunks) chunks = max_chunks;
    if (chunks < 1) chunks = 1;
    if (chunks > 1024) chunks = 1024;
    return static_cast<int>(chunks);
}

}  // namespace
}  // namespace jz

using namespace jz;

JZ_API int jzhip_sum_cols(float* out, const float* a, int numrow, int numcol, int ld) {
    if (numrow <= 0 || numcol <= 0 || ld < numrow) return -1;
    if (!out || !a) return -1;
    const bool vec = aligned16(a) && (ld % 4 == 0);
    int chunks = pick_chunks(numcol, numrow, 2048);
    while (chunks > 1 && static_cast<size_t>(chunks) * numcol > kWorkspaceFloats) --chunks;
    int chunk_len = (numrow + chunks - 1) / chunks;
    chunk_len = (chunk_len + 3) & ~3;  // keep float4 alignment of chunk starts
    chunks = (numrow + chunk_len - 1) / chunk_len;
    float* dst = out;
    if (chunks > 1) {
        dst = workspace();
        if (!dst) return -2;
    }
    const size_t items = static_cast<size_t>(numcol) * chunks;
    const unsigned grid = grid_cover(items, kBlock / kWave);
    hipStream_t s = stream();
    if (vec && streams_past_cache(static_cast<size_t>(numrow) * numcol * sizeof(float)))
        sum_cols_kernel<4, true><<<grid, kBlock, 0, s>>>(dst, a, numrow, numcol, ld, chunks, chunk_len);
    else if (vec)
        sum_cols_kernel<4><<<grid, kBlock, 0, s>>>(dst, a, numrow, numcol, ld, chunks, chunk_len);
    else
        sum_cols_kernel<1><<<grid, kBlock, 0, s>>>(dst, a, numrow, numcol, ld, chunks, chunk_len);
    if (chunks > 1) {
        combine_partials_kernel<<<(numcol + kWave - 1) / kWave, kCombineBlock, 0, s>>>(out, dst, numcol, chunks);
    }
    return launch_rc();
}

namespace jz {
namespace {

// Row sums with the partial results of the column chunks in `scratch`
// (capacity `cap` floats).  `scratch` is a callable so that the shared
// workspace is only created when a launch really needs partials.
template <class GetScratch>
int sum_rows_impl(float* out, const float* a, int numrow, int numcol, int ld, size_t cap,
                  GetScratch scratch) {
    hipStream_t s = stream();
    if (numrow <= kWave && ld == numrow) {
        // short contiguous matrix: flat stream
        const size_t total = static_cast<size_t>(numrow) * numcol;
        const int active = (kBlock / numrow) * numrow;
        // columns per block so that there are a few blocks per CU
        size_t blocks = (total + static_cast<size_t>(active) * 16 - 1) / (static_cast<size_t>(active) * 16);
        const size_t limit = static_cast<size_t>(num_cus()) * 8;
        if (blocks > limit) blocks = limit;
        if (blocks < 1) blocks = 1;
        while (blocks > 1 && blocks * numrow > cap) blocks /= 2;
        size_t cols_per_block = (numcol + blocks - 1) / blocks;
        blocks = (numcol + cols_per_block - 1) / cols_per_block;
        const size_t span = cols_per_block * numrow;
        float* dst = out;
        if (blocks > 1) {
            dst = scratch();
            if (!dst) return -2;
        }
        sum_rows_short_kernel<<<static_cast<unsigned>(blocks), kBlock, 0, s>>>(dst, a, numrow, total,
                                                                              active, span);
        if (blocks > 1) {
            combine_partials_kernel<<<(numrow + kWave - 1) / kWave, kCombineBlock, 0, s>>>(
                out, dst, numrow, static_cast<int>(blocks));
        }
        return launch_rc();
    }
    const bool vec = aligned16(a) && (ld % 4 == 0) && (numrow % 4 == 0);
    const int rows_per_block = kWave * (vec ? 4 : 1);
    const int row_blocks = (numrow + rows_per_block - 1) / rows_per_block;
    int chunks = pick_chunks(row_blocks * (kBlock / kWave), numcol, 64);
    while (chunks > 1 && static_cast<size_t>(chunks) * numrow > cap) --chunks;
    if (chunks > 65535) chunks = 65535;
    const int chunk_len = (numcol + chunks - 1) / chunks;
    chunks = (numcol + chunk_len - 1) / chunk_len;
    float* dst = out;
    if (chunks > 1) {
        dst = scratch();
        if (!dst) return -2;
    }
    dim3 grid(row_blocks, chunks);
    if (vec && streams_past_cache(static_cast<size_t>(numrow) * numcol * sizeof(float)))
        sum_rows_kernel<4, true><<<grid, kBlock, 0, s>>>(dst, a, numrow, numcol, ld, chunk_len);
    else if (vec)
        sum_rows_kernel<4><<<grid, kBlock, 0, s>>>(dst, a, numrow, numcol, ld, chunk_len);
    else
        sum_rows_kernel<1><<<grid, kBlock, 0, s>>>(dst, a, numrow, numcol, ld, chunk_len);
    if (chunks > 1) {
        combine_partials_kernel<<<(numrow + kWave - 1) / kWave, kCombineBlock, 0, s>>>(out, dst, numrow, chunks);
    }
    return launch_rc();
}

}  // namespace
}  // namespace jz

JZ_API int jzhip_sum_rows(float* out, const float* a, int numrow, int numcol, int ld) {
    if (numrow <= 0 || numcol <= 0 || ld < numrow) return -1;
    if (!out || !a) return -1;
    return sum_rows_impl(out, a, numrow, numcol, ld, kWorkspaceFloats, [] { return workspace(); });
}

JZ_API int jzhip_nrm2(float* out_device, const float* x, size_t count) {
    if (!out_device) return -1;
    if (count == 0) return jzhip_fill(out_device, 1, 0.f);
    if (!x) return -1;
    float* part = workspace();
    if (!part) return -2;
    const unsigned grid = grid_for(count / 4 + 1, static_cast<size_t>(kBlock) * 2, 4);
    hipStream_t s = stream();
    if (streams_past_cache(count * sizeof(float)))
        sumsq_partial_kernel<true><<<grid, kBlock, 0, s>>>(part, x, count, aligned16(x) ? 1 : 0);
    else
        sumsq_partial_kernel<false><<<grid, kBlock, 0, s>>>(part, x, count, aligned16(x) ? 1 : 0);
    sqrt_sum_kernel<<<1, kBlock, 0, s>>>(out_device, part, static_cast<int>(grid));
    return launch_rc();
}

JZ_API int jzhip_mse_loss(float* out_device, const float* target, const float* pred, size_t count, float scale) {
    if (!out_device) return -1;
    if (count == 0) return jzhip_fill(out_device, 1, 0.f);
    if (!target || !pred) return -1;
    hipStream_t s = stream();
    if (count <= static_cast<size_t>(kBlock) * 32) {
        sqdiff_partial_kernel<false><<<1, kBlock, 0, s>>>(out_device, target, pred, count, scale);
        return launch_rc();
    }
    float* part = workspace();
    if (!part) return -2;
    const unsigned grid = grid_for(count, static_cast<size_t>(kBlock) * 2, 4);
    if (streams_past_cache(2 * count * sizeof(float)))
        sqdiff_partial_kernel<true><<<grid, kBlock, 0, s>>>(part, target, pred, count, scale);
    else
        sqdiff_partial_kernel<false><<<grid, kBlock, 0, s>>>(part, target, pred, count, scale);
    if (grid > 1) scaled_sum_kernel<<<1, kBlock, 0, s>>>(out_device, part, static_cast<int>(grid), scale);
    else return jzhip_copy(out_device, part, 1);
    return launch_rc();
}

JZ_API int jzhip_max_cols(float* out, const float* a, int numrow, int numcol, int ld) {
    if (numrow <= 0 || numcol <= 0 || ld < numrow || !out || !a) return -1;
    const unsigned grid = grid_cover(numcol, kBlock / kWave);
    if (streams_past_cache(static_cast<size_t>(numrow) * numcol * sizeof(float)))
        max_cols_kernel<false, true><<<grid, kBlock, 0, stream()>>>(out, nullptr, a, numrow, numcol, ld);
    else
        max_cols_kernel<false, false><<<grid, kBlock, 0, stream()>>>(out, nullptr, a, numrow, numcol, ld);
    return launch_rc();
}

JZ_API int jzhip_predict_one_hot(float* out, const float* a, int numrow, int numcol, int ld) {
    if (numrow <= 0 || numcol <= 0 || ld < numrow || !out || !a) return -1;
    const unsigned grid = grid_cover(numcol, kBlock / kWave);
    one_hot_max_cols_kernel<<<grid, kBlock, 0, stream()>>>(out, a, numrow, numcol, ld);
    return launch_rc();
}

JZ_API int jzhip_argmax_cols(int32_t* out, const float* a, int numrow, int numcol, int ld) {
    if (numrow <= 0 || numcol <= 0 || ld < numrow || !out || !a) return -1;
    const unsigned grid = grid_cover(numcol, kBlock / kWave);
    if (streams_past_cache(static_cast<size_t>(numrow) * numcol * sizeof(float)))
        max_cols_kernel<true, true><<<grid, kBlock, 0, stream()>>>(nullptr, out, a, numrow, numcol, ld);
    else
        max_cols_kernel<true, false><<<grid, kBlock, 0, stream()>>>(nullptr, out, a, numrow, numcol, ld);
    return launch_rc();
}

// ── row sums without any allocation ──────────────────────────────────────
// Callers that may not allocate device memory (code under HIP graph capture,
// serving loops, harnesses that forbid hipMalloc) cannot use the lazily
// created workspace.  This variant keeps the column-chunk partial sums in a
// fixed array that is part of the code object: every GPU the library runs on
// holds its own 4 MiB copy from the first launch until the process ends.
namespace {
constexpr size_t kFixedScratchFloats = size_t(1) << 20;   // 4 MiB
constexpr int kFixedScratchMaxRows = 65536;               // leaves room for >= 16 column chunks
constexpr int kMaxDevices = 64;
static __device__ __align__(256) float scratch[kFixedScratchFloats];
// Device address of `scratch` per device ordinal.  In host code the array's
// name is only a handle for hipGetSymbolAddress, never a pointer a kernel may
// be given.
std::atomic<float*> g_fixed_scratch[kMaxDevices];

int fixed_scratch(float** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int>(e);
    if (dev < 0 || dev >= kMaxDevices) return -1;
    float* p = g_fixed_scratch[dev].load(std::memory_order_acquire);
    if (!p) {
        void* addr = nullptr;
        e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return static_cast<int>(e);
        }
        if (!addr) return -2;
        p = static_cast<float*>(addr);
        g_fixed_scratch[dev].store(p, std::memory_order_release);   // same value from any thread
    }
    *out = p;
    return 0;
}
}  // namespace

JZ_API int jzhip_sum_rows_noalloc(float* out, const float* a, int numrow, int numcol, int ld) {
    if (numrow <= 0 || numcol <= 0 || ld < numrow) return -1;
    if (!out || !a) return -1;
    if (numrow > kFixedScratchMaxRows) return -3;
    float* fixed = nullptr;
    const int rc = fixed_scratch(&fixed);
    if (rc) return rc;
    // Every partial the combine kernel reads is written by the launch before
    // it, so nothing in the array has to start at zero.
    return sum_rows_impl(out, a, numrow, numcol, ld, kFixedScratchFloats, [fixed] { return fixed; });
}
