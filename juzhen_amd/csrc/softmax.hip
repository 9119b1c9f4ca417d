// Single-pass fused softmax kernels.
//
// The reference builds a softmax from ~9 generic matrix ops (max reduce,
// rank-1 broadcast, subtract, exp, ones-GEMV sum, reciprocal, rank-1 broadcast,
// Hadamard: ml/layer.hpp:2344-2358); here each distribution is read once,
// kept in registers, and written once: 8 bytes per element.
//
// Arithmetic follows the reference expression: m = max(x) (floor -1e30f),
// e = exp(x - m) (hardware exp2 with the argument's rounding error folded back in), p = e * (1.0f / (sum(e) + 1e-12f)).
#include "common.hpp"

#include <cmath>

namespace jz {
namespace {

// Optional pre-processing of attention scores: x*scale and the causal mask
// (key index > query index -> -1e9f, ml/layer.hpp:2979-2994).
struct ScoreXform {
    float scale;
    int causal;
    int S;  // block edge; 0 = plain softmax
};

// ── distributions along contiguous columns ───────────────────────────────
// One wavefront per column, NV values per lane held in registers
// (numrow <= 64*NV).
template <int NV>
__global__ __launch_bounds__(kBlock) void softmax_cols_kernel(float* out, const float* in,
                                                              int numrow, size_t numcol, size_t ld,
                                                              ScoreXform xf) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t wave0 = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
    const size_t nwaves = static_cast<size_t>(gridDim.x) * (kBlock / kWave);
    for (size_t col = wave_begin(numcol, wave0, nwaves), col_end = wave_end(numcol, wave0, nwaves); col < col_end; ++col) {
        const float* p = in + col * ld;
        float* q = out + col * ld;
        const int qidx = xf.S ? static_cast<int>(col % xf.S) : 0;  // query index of this column
        float x[NV];
        float m = -1e30f;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int r = lane + v * kWave;
            if (r < numrow) {
                float t = p[r];
                if (xf.S) {
                    t = t * xf.scale;
                    if (xf.causal && r > qidx) t = -1e9f;
                }
                x[v] = t;
                m = m > t ? m : t;
            } else {
                x[v] = -INFINITY;
            }
        }
        m = wave_max(m);
        float s = 0.f;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int r = lane + v * kWave;
            x[v] = (r < numrow) ? exp_neg(x[v] - m) : 0.f;
            s += x[v];
        }
        s = wave_sum(s);
        const float inv = 1.0f / (s + 1e-12f);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int r = lane + v * kWave;
            if (r < numrow) q[r] = x[v] * inv;
        }
    }
}

// Long columns (numrow > 1024): one block per column, three sweeps; the
// second and third hit L2.
__global__ __launch_bounds__(kBlock) void softmax_cols_long_kernel(float* out, const float* in,
                                                                   int numrow, size_t numcol,
                                                                   size_t ld) {
    __shared__ float red[kBlock / kWave];
    for (size_t col = blockIdx.x; col < numcol; col += gridDim.x) {
        const float* p = in + col * ld;
        float* q = out + col * ld;
        float m = -1e30f;
        for (int r = threadIdx.x; r < numrow; r += kBlock) m = m > p[r] ? m : p[r];
        m = block_allreduce<kBlock / kWave>(m, MaxOp{}, red, -1e30f);
        float s = 0.f;
        for (int r = threadIdx.x; r < numrow; r += kBlock) s += exp_neg(p[r] - m);
        s = block_allreduce<kBlock / kWave>(s, SumOp{}, red, 0.f);
        const float inv = 1.0f / (s + 1e-12f);
        for (int r = threadIdx.x; r < numrow; r += kBlock) q[r] = exp_neg(p[r] - m) * inv;
    }
}

// Medium-long columns (1024 < numrow <= 16384): one block per column with the
// column held in registers (NV4 float4 per thread), so it is still one read
// and one write per element.  Columns over 4096 rows take 1024 threads: a
// quarter of the registers per thread, so more columns are in flight per CU.
template <int NV4, int BLOCK, bool NT>
__global__ __launch_bounds__(BLOCK) void softmax_cols_block_kernel(float* out, const float* in,
                                                                    int numrow, size_t numcol,
                                                                    size_t ld) {
    __shared__ float red[BLOCK / kWave];
    for (size_t col = blockIdx.x; col < numcol; col += gridDim.x) {
        const float* p = in + col * ld;
        float* q = out + col * ld;
        float4 x[NV4];
        float m = -1e30f;
#pragma unroll
        for (int v = 0; v < NV4; ++v) {
            const int r = (threadIdx.x + v * BLOCK) * 4;
            if (r < numrow) {   // numrow % 4 == 0 on this path
                x[v] = load4<NT>(p + r);
                const float a = x[v].x > x[v].y ? x[v].x : x[v].y;
                const float b = x[v].z > x[v].w ? x[v].z : x[v].w;
                const float c = a > b ? a : b;
                m = m > c ? m : c;
            }
        }
        m = block_allreduce<BLOCK / kWave>(m, MaxOp{}, red, -1e30f);
        float s = 0.f;
#pragma unroll
        for (int v = 0; v < NV4; ++v) {
            const int r = (threadIdx.x + v * BLOCK) * 4;
            if (r < numrow) {
                x[v].x = exp_neg(x[v].x - m); x[v].y = exp_neg(x[v].y - m);
                x[v].z = exp_neg(x[v].z - m); x[v].w = exp_neg(x[v].w - m);
                s += (x[v].x + x[v].y) + (x[v].z + x[v].w);
            }
        }
        s = block_allreduce<BLOCK / kWave>(s, SumOp{}, red, 0.f);
        const float inv = 1.0f / (s + 1e-12f);
#pragma unroll
        for (int v = 0; v < NV4; ++v) {
            const int r = (threadIdx.x + v * BLOCK) * 4;
            if (r < numrow) {
                x[v].x *= inv; x[v].y *= inv; x[v].z *= inv; x[v].w *= inv;
                store4<NT>(q + r, x[v]);
            }
        }
    }
}

// ── distributions along rows (stride ld) ─────────────────────────────────
// A block owns RPB consecutive rows of one matrix (blockIdx.y selects the
// matrix of a batch); its 256 threads are RPB row lanes x (256/RPB) column
// phases, so global accesses are coalesced along the rows.  Max and sum are
// combined across the column phases through LDS.
template <int RPB>
__global__ __launch_bounds__(kBlock) void softmax_rows_kernel(float* out, const float* in,
                                                              int numrow, int numcol, size_t ld,
                                                              size_t batch_stride, ScoreXform xf) {
    constexpr int CP = kBlock / RPB;
    __shared__ float red[CP][RPB];
    const int rl = threadIdx.x % RPB;
    const int cp = threadIdx.x / RPB;
    const int row = blockIdx.x * RPB + rl;
    const float* p = in + static_cast<size_t>(blockIdx.y) * batch_stride;
    float* q = out + static_cast<size_t>(blockIdx.y) * batch_stride;
    const bool live = row < numrow;
    // with a causal mask only keys <= query (columns <= row) are unmasked;
    // masked entries contribute exp(-1e9 - m) == 0 exactly and are written as 0
    const int c_live = (xf.S && xf.causal) ? (row + 1 < numcol ? row + 1 : numcol) : numcol;

    float m = -1e30f;
    if (live) {
        for (int c = cp; c < c_live; c += CP) {
            float t = p[static_cast<size_t>(c) * ld + row];
            if (xf.S) t = t * xf.scale;
            m = m > t ? m : t;
        }
        if (c_live < numcol) m = m > -1e9f ? m : -1e9f;
    }
    red[cp][rl] = m;
    __syncthreads();
#pragma unroll
    for (int k = 0; k < CP; ++k) m = m > red[k][rl] ? m : red[k][rl];
    __syncthreads();

    float s = 0.f;
    if (live) {
        for (int c = cp; c < c_live; c += CP) {
            float t = p[static_cast<size_t>(c) * ld + row];
            if (xf.S) t = t * xf.scale;
            s += exp_neg(t - m);
        }
    }
    red[cp][rl] = s;
    __syncthreads();
    s = 0.f;
#pragma unroll
    for (int k = 0; k < CP; ++k) s += red[k][rl];
    const float inv = 1.0f / (s + 1e-12f);
    if (live) {
        for (int c = cp; c < numcol; c += CP) {
            float r = 0.f;
            if (c < c_live) {
                float t = p[static_cast<size_t>(c) * ld + row];
                if (xf.S) t = t * xf.scale;
                r = exp_neg(t - m) * inv;
            } else {
                r = exp_neg(-1e9f - m) * inv;
            }
            q[static_cast<size_t>(c) * ld + row] = r;
        }
    }
}

// Row softmax with the whole row held in registers: 64 row lanes x 4 column
// phases, NV columns per thread (numcol <= 4*NV), one read and one write per
// element.  Used for attention score blocks (S <= 256) and other short rows.
template <int NV>
__global__ __launch_bounds__(kBlock) void softmax_rows_reg_kernel(float* out, const float* in,
                                                                  int numrow, int numcol, size_t ld,
                                                                  size_t batch_stride, ScoreXform xf) {
    constexpr int RPB = kWave, CP = kBlock / kWave;
    __shared__ float red[CP][RPB];
    const int rl = threadIdx.x % RPB;
    const int cp = threadIdx.x / RPB;
    const int row = blockIdx.x * RPB + rl;
    const float* p = in + static_cast<size_t>(blockIdx.y) * batch_stride;
    float* q = out + static_cast<size_t>(blockIdx.y) * batch_stride;
    const bool live = row < numrow;
    const bool causal = xf.S && xf.causal;
    float x[NV];
    float m = -1e30f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int c = cp + v * CP;
        float t = -INFINITY;
        if (live && c < numcol) {
            if (causal && c > row) {
                t = -1e9f;  // masked key (ml/layer.hpp:2979-2994); never loaded
            } else {
                t = p[static_cast<size_t>(c) * ld + row];
                if (xf.S) t = t * xf.scale;
            }
            m = m > t ? m : t;
        }
        x[v] = t;
    }
    red[cp][rl] = m;
    __syncthreads();
#pragma unroll
    for (int k = 0; k < CP; ++k) m = m > red[k][rl] ? m : red[k][rl];
    __syncthreads();
    float s = 0.f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int c = cp + v * CP;
        x[v] = (live && c < numcol) ? exp_neg(x[v] - m) : 0.f;
        s += x[v];
    }
    red[cp][rl] = s;
    __syncthreads();
    s = 0.f;
#pragma unroll
    for (int k = 0; k < CP; ++k) s += red[k][rl];
    const float inv = 1.0f / (s + 1e-12f);
    if (live) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int c = cp + v * CP;
            if (c < numcol) q[static_cast<size_t>(c) * ld + row] = x[v] * inv;
        }
    }
}

// Long rows: columns are split into chunks over grid.y.  Pass A leaves one
// (max, sum) pair per (chunk, row) in the workspace (online softmax inside the
// chunk), a small fold kernel turns them into (max, 1/sum) per row, pass B
// writes the result: 12 bytes per element instead of the 16 of a three-sweep
// kernel, and rows x chunks workgroups instead of rows/64.  The column loops
// are unrolled eight deep so that eight loads are in flight per thread.
// part layout: [chunk][2][numrow]; rowstat layout: [2][numrow].
constexpr int kRowUnroll = 8;

template <bool NT>
__global__ __launch_bounds__(kBlock) void softmax_rows_partial_kernel(float* part, const float* in,
                                                                      int numrow, int numcol,
                                                                      size_t ld, int chunk_len) {
    constexpr int RPB = kWave, CP = kBlock / kWave;
    __shared__ float redm[CP][RPB], reds[CP][RPB];
    const int rl = threadIdx.x % RPB, cp = threadIdx.x / RPB;
    const int row = blockIdx.x * RPB + rl;
    const int c0 = blockIdx.y * chunk_len;
    const int c1 = (c0 + chunk_len) < numcol ? (c0 + chunk_len) : numcol;
    float m = -1e30f, s = 0.f;
    if (row < numrow) {
        for (int c = c0 + cp; c < c1; c += CP * kRowUnroll) {
            float t[kRowUnroll];
            float tm = -1e30f;
#pragma unroll
            for (int u = 0; u < kRowUnroll; ++u) {
                const int cc = c + u * CP;
                t[u] = cc < c1 ? load1<NT>(in + static_cast<size_t>(cc) * ld + row) : -1e30f;
                tm = tm > t[u] ? tm : t[u];
            }
            const float mn = m > tm ? m : tm;
            float acc = s * exp_neg(m - mn);
#pragma unroll
            for (int u = 0; u < kRowUnroll; ++u) {
                const int cc = c + u * CP;
                if (cc < c1) acc += exp_neg(t[u] - mn);
            }
            s = acc;
            m = mn;
        }
    }
    redm[cp][rl] = m;
    reds[cp][rl] = s;
    __syncthreads();
    if (cp == 0 && row < numrow) {
        float M = -1e30f;
#pragma unroll
        for (int k = 0; k < CP; ++k) M = M > redm[k][rl] ? M : redm[k][rl];
        float S = 0.f;
#pragma unroll
        for (int k = 0; k < CP; ++k) S += reds[k][rl] * exp_neg(redm[k][rl] - M);
        const size_t o = static_cast<size_t>(blockIdx.y) * 2 * numrow + row;
        part[o] = M;
        part[o + numrow] = S;
    }
}

// (max, sum) pairs of a row over all chunks -> (max, 1/(sum + 1e-12)).
// 64 row lanes x 16 chunk phases per block, four pairs in flight per thread.
constexpr int kFoldThreads = 1024;
__global__ __launch_bounds__(kFoldThreads) void softmax_rows_fold_kernel(float* rowstat, const float* part,
                                                                         int numrow, int chunks) {
    constexpr int RPB = kWave, CP = kFoldThreads / kWave;
    __shared__ float redm[CP][RPB], reds[CP][RPB];
    const int rl = threadIdx.x % RPB, cp = threadIdx.x / RPB;
    const int row = blockIdx.x * RPB + rl;
    float m = -1e30f, s = 0.f;
    if (row < numrow) {
        for (int k = cp; k < chunks; k += CP * 4) {
            float mk[4], sk[4];
            float tm = -1e30f;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int kk = k + u * CP;
                const size_t o = static_cast<size_t>(kk) * 2 * numrow + row;
                mk[u] = kk < chunks ? part[o] : -1e30f;
                sk[u] = kk < chunks ? part[o + numrow] : 0.f;
                tm = tm > mk[u] ? tm : mk[u];
            }
            const float mn = m > tm ? m : tm;
            float acc = s * exp_neg(m - mn);
#pragma unroll
            for (int u = 0; u < 4; ++u) acc += sk[u] * exp_neg(mk[u] - mn);
            s = acc;
            m = mn;
        }
    }
    redm[cp][rl] = m;
    reds[cp][rl] = s;
    __syncthreads();
    if (cp == 0 && row < numrow) {
        float M = -1e30f;
#pragma unroll
        for (int k = 0; k < CP; ++k) M = M > redm[k][rl] ? M : redm[k][rl];
        float S = 0.f;
#pragma unroll
        for (int k = 0; k < CP; ++k) S += reds[k][rl] * exp_neg(redm[k][rl] - M);
        rowstat[row] = M;
        rowstat[numrow + row] = 1.0f / (S + 1e-12f);
    }
}

template <bool NT>
__global__ __launch_bounds__(kBlock) void softmax_rows_apply_kernel(float* out, const float* in,
                                                                    const float* rowstat, int numrow,
                                                                    int numcol, size_t ld,
                                                                    int chunk_len) {
    constexpr int RPB = kWave, CP = kBlock / kWave;
    const int rl = threadIdx.x % RPB, cp = threadIdx.x / RPB;
    const int row = blockIdx.x * RPB + rl;
    if (row >= numrow) return;
    const float M = rowstat[row], inv = rowstat[numrow + row];
    const int c0 = blockIdx.y * chunk_len;
    const int c1 = (c0 + chunk_len) < numcol ? (c0 + chunk_len) : numcol;
    for (int c = c0 + cp; c < c1; c += CP * kRowUnroll) {
        float t[kRowUnroll];
#pragma unroll
        for (int u = 0; u < kRowUnroll; ++u) {
            const int cc = c + u * CP;
            t[u] = cc < c1 ? in[static_cast<size_t>(cc) * ld + row] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < kRowUnroll; ++u) {
            const int cc = c + u * CP;
            if (cc < c1) store1<NT>(out + static_cast<size_t>(cc) * ld + row, exp_neg(t[u] - M) * inv);
        }
    }
}

// Whole rows in the registers of one workgroup, any split of its threads into RL row lanes
// (consecutive rows: the coalesced direction) and THREADS/RL column phases; a thread holds
// the NV columns cp, cp + CP, ... of its row.  One read and one write per element.  Column
// phases that share a wave are combined by lane exchanges, the waves through LDS.
// The split is picked per shape by softmax_rows_single_read below.  What decides it, as
// measured on MI355X: the loads a thread has in flight (16 columns per thread: 6 us at
// 1024 x 1024, 32: 8-9 us, 64: 17-20 us, whatever the run length), then the bytes a wave
// reads contiguously per column (16-byte runs: 10.8 us), then the workgroup count.
template <int THREADS, int RL, int NV>
__global__ __launch_bounds__(THREADS) void softmax_rows_tile_kernel(float* out, const float* in, int numrow,
                                                                    int numcol, size_t ld) {
    constexpr int CP = THREADS / RL;          // column phases
    constexpr int NW = THREADS / kWave;       // waves
    constexpr int PPW = RL >= kWave ? 1 : kWave / RL;   // column phases inside one wave
    constexpr int RPW = RL >= kWave ? kWave : RL;       // distinct rows inside one wave
    constexpr int WPR = RL >= kWave ? RL / kWave : 1;   // waves side by side along the rows
    static_assert(THREADS % kWave == 0 && (RL % kWave == 0 || kWave % RL == 0), "shape");
    __shared__ float red[NW][RPW];
    const int rl = threadIdx.x % RL, cp = threadIdx.x / RL;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int lr = lane % RPW;                // row slot inside the wave
    const int wr = wave % WPR;                // which row group of the workgroup this wave sits in
    const int row = blockIdx.x * RL + rl;
    const bool live = row < numrow;
    const float* p = in + row;
    float x[NV];
    float m = -1e30f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int c = cp + v * CP;
        x[v] = (live && c < numcol) ? p[static_cast<size_t>(c) * ld] : -1e30f;
        m = m > x[v] ? m : x[v];
    }
    auto combine = [&](float val, auto op) {
#pragma unroll
        for (int off = RPW; off < kWave; off <<= 1) val = op(val, __shfl_xor(val, off, kWave));
        if constexpr (NW > WPR) {
            __syncthreads();                  // red may still be read from the previous round
            if (lane < RPW) red[wave][lr] = val;
            __syncthreads();
            val = red[wr][lr];
#pragma unroll
            for (int w = WPR; w < NW; w += WPR) val = op(val, red[wr + w][lr]);
        }
        return val;
    };
    m = combine(m, MaxOp{});
    float s = 0.f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int c = cp + v * CP;
        x[v] = (live && c < numcol) ? exp_neg(x[v] - m) : 0.f;
        s += x[v];
    }
    s = combine(s, SumOp{});
    const float inv = 1.0f / (s + 1e-12f);
    if (live) {
        float* q = out + row;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int c = cp + v * CP;
            if (c < numcol) q[static_cast<size_t>(c) * ld] = x[v] * inv;
        }
    }
}

// The same with four consecutive rows per thread (one float4 per column): a quarter of the
// load and store instructions for the same bytes, and RL4 row lanes cover 4*RL4 rows, so a
// wave reads 16*RL4 contiguous bytes of each column.  Needs numrow % 4 == 0, ld % 4 == 0
// and 16-byte aligned pointers.
template <int THREADS, int RL4, int NV>
__global__ __launch_bounds__(THREADS) void softmax_rows_tile4_kernel(float* out, const float* in, int numrow,
                                                                     int numcol, size_t ld) {
    constexpr int CP = THREADS / RL4;
    constexpr int NW = THREADS / kWave;
    constexpr int RPW = RL4 >= kWave ? kWave : RL4;     // distinct row lanes inside one wave
    constexpr int WPR = RL4 >= kWave ? RL4 / kWave : 1;
    static_assert(THREADS % kWave == 0 && (RL4 % kWave == 0 || kWave % RL4 == 0), "shape");
    __shared__ float4 red[NW][RPW];
    const int rl = threadIdx.x % RL4, cp = threadIdx.x / RL4;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int lr = lane % RPW, wr = wave % WPR;
    const int row = (blockIdx.x * RL4 + rl) * 4;
    const bool live = row < numrow;
    const float* p = in + row;
    float4 x[NV];
    float4 m = make_float4(-1e30f, -1e30f, -1e30f, -1e30f);
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int c = cp + v * CP;
        if (live && c < numcol) x[v] = *reinterpret_cast<const float4*>(p + static_cast<size_t>(c) * ld);
        else x[v] = make_float4(-1e30f, -1e30f, -1e30f, -1e30f);
        m.x = m.x > x[v].x ? m.x : x[v].x; m.y = m.y > x[v].y ? m.y : x[v].y;
        m.z = m.z > x[v].z ? m.z : x[v].z; m.w = m.w > x[v].w ? m.w : x[v].w;
    }
    auto combine = [&](float4 val, auto op) {
#pragma unroll
        for (int off = RPW; off < kWave; off <<= 1) {
            val.x = op(val.x, __shfl_xor(val.x, off, kWave)); val.y = op(val.y, __shfl_xor(val.y, off, kWave));
            val.z = op(val.z, __shfl_xor(val.z, off, kWave)); val.w = op(val.w, __shfl_xor(val.w, off, kWave));
        }
        if constexpr (NW > WPR) {
            __syncthreads();
            if (lane < RPW) red[wave][lr] = val;
            __syncthreads();
            val = red[wr][lr];
#pragma unroll
            for (int w = WPR; w < NW; w += WPR) {
                const float4 o = red[wr + w][lr];
                val.x = op(val.x, o.x); val.y = op(val.y, o.y); val.z = op(val.z, o.z); val.w = op(val.w, o.w);
            }
        }
        return val;
    };
    m = combine(m, MaxOp{});
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int c = cp + v * CP;
        if (live && c < numcol) {
            x[v].x = exp_neg(x[v].x - m.x); x[v].y = exp_neg(x[v].y - m.y);
            x[v].z = exp_neg(x[v].z - m.z); x[v].w = exp_neg(x[v].w - m.w);
        } else {
            x[v] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        s.x += x[v].x; s.y += x[v].y; s.z += x[v].z; s.w += x[v].w;
    }
    s = combine(s, SumOp{});
    const float4 inv = make_float4(1.0f / (s.x + 1e-12f), 1.0f / (s.y + 1e-12f), 1.0f / (s.z + 1e-12f),
                                   1.0f / (s.w + 1e-12f));
    if (live) {
        float* q = out + row;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int c = cp + v * CP;
            if (c < numcol) {
                x[v].x *= inv.x; x[v].y *= inv.y; x[v].z *= inv.z; x[v].w *= inv.w;
                *reinterpret_cast<float4*>(q + static_cast<size_t>(c) * ld) = x[v];
            }
        }
    }
}

// ── softmax backward: dS = A*(dA - sum_keys(A*dA))*scale ─────────────────
template <int NV>
__global__ __launch_bounds__(kBlock) void softmax_bwd_cols_kernel(float* dS, const float* A,
                                                                  const float* dA, int numrow,
                                                                  size_t numcol, float scale) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t wave0 = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
    const size_t nwaves = static_cast<size_t>(gridDim.x) * (kBlock / kWave);
    for (size_t col = wave_begin(numcol, wave0, nwaves), col_end = wave_end(numcol, wave0, nwaves); col < col_end; ++col) {
        const size_t base = col * numrow;
        float a[NV], g[NV];
        float dot = 0.f;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int r = lane + v * kWave;
            a[v] = r < numrow ? A[base + r] : 0.f;
            g[v] = r < numrow ? dA[base + r] : 0.f;
            dot += a[v] * g[v];
        }
        dot = wave_sum(dot);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int r = lane + v * kWave;
            if (r < numrow) dS[base + r] = (a[v] * (g[v] - dot)) * scale;
        }
    }
}

template <int RPB>
__global__ __launch_bounds__(kBlock) void softmax_bwd_rows_kernel(float* dS, const float* A,
                                                                  const float* dA, int S,
                                                                  float scale) {
    constexpr int CP = kBlock / RPB;
    __shared__ float red[CP][RPB];
    const int rl = threadIdx.x % RPB;
    const int cp = threadIdx.x / RPB;
    const int row = blockIdx.x * RPB + rl;
    const size_t off = static_cast<size_t>(blockIdx.y) * S * S;
    const bool live = row < S;
    float dot = 0.f;
    if (live) {
        for (int c = cp; c < S; c += CP) {
            const size_t i = off + static_cast<size_t>(c) * S + row;
            dot += A[i] * dA[i];
        }
    }
    red[cp][rl] = dot;
    __syncthreads();
    dot = 0.f;
#pragma unroll
    for (int k = 0; k < CP; ++k) dot += red[k][rl];
    if (live) {
        for (int c = cp; c < S; c += CP) {
            const size_t i = off + static_cast<size_t>(c) * S + row;
            dS[i] = (A[i] * (dA[i] - dot)) * scale;
        }
    }
}

// ── softmax cross-entropy against integer labels ─────────────────────────
// One wavefront per sample column.  per_sample[n] = x[label] - lse.
// DENSE: the targets are a K x N matrix (leading dimension ld) instead of labels, as
// LogisticLayer holds them: per_sample[n] = sum_k x*y - lse (ml/layer.hpp:281), and the
// gradient subtracts y itself.
template <int NV, bool DENSE>
__global__ __launch_bounds__(kBlock) void xent_cols_kernel(float* per_sample, float* dlogits,
                                                           const float* logits,
                                                           const int32_t* labels, const float* target,
                                                           int K, int N, size_t ld, float inv_n) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t wave0 = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
    const size_t nwaves = static_cast<size_t>(gridDim.x) * (kBlock / kWave);
    for (size_t col = wave_begin(static_cast<size_t>(N), wave0, nwaves), col_end = wave_end(static_cast<size_t>(N), wave0, nwaves); col < col_end; ++col) {
        const float* p = logits + col * ld;
        int label = 0;
        if constexpr (!DENSE) label = labels[col];
        float x[NV];
        float y[DENSE ? NV : 1];
        float m = -1e30f;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int r = lane + v * kWave;
            x[v] = r < K ? p[r] : -INFINITY;
            if constexpr (DENSE) y[v] = r < K ? target[col * ld + r] : 0.f;
            if (r < K) m = m > x[v] ? m : x[v];
        }
        m = wave_max(m);
        float s = 0.f, picked = 0.f;
        float e[NV];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int r = lane + v * kWave;
            e[v] = r < K ? exp_neg(x[v] - m) : 0.f;
            s += e[v];
            if constexpr (DENSE) {
                if (r < K) picked += x[v] * y[v];
            } else {
                if (r == label) picked = x[v];
            }
        }
        s = wave_sum(s);
        picked = wave_sum(picked);
        if (lane == 0) per_sample[col] = picked - (logf(s) + m);
        if (dlogits) {
            // -(y - E/Z)/N with E/Z = e * (float)(1.0/(double)Z)  (ml/layer.hpp:258-261)
            const float invz = static_cast<float>(1.0 / static_cast<double>(s));
            float* d = dlogits + col * ld;
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                const int r = lane + v * kWave;
                if (r < K) {
                    float yv;
                    if constexpr (DENSE) yv = y[v];
                    else yv = (r == label) ? 1.0f : 0.0f;
                    d[r] = -(yv - e[v] * invz) * inv_n;
                }
            }
        }
    }
}

// More than 1024 classes: the same with three sweeps over the column (the second and
// third hit L2) instead of registers.
template <bool DENSE>
__global__ __launch_bounds__(kBlock) void xent_cols_long_kernel(float* per_sample, float* dlogits,
                                                                const float* logits, const int32_t* labels,
                                                                const float* target, int K, int N, size_t ld,
                                                                float inv_n) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t wave0 = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
    const size_t nwaves = static_cast<size_t>(gridDim.x) * (kBlock / kWave);
    for (size_t col = wave_begin(static_cast<size_t>(N), wave0, nwaves), col_end = wave_end(static_cast<size_t>(N), wave0, nwaves); col < col_end; ++col) {
        const float* p = logits + col * ld;
        const float* t = DENSE ? target + col * ld : nullptr;
        int label = 0;
        if constexpr (!DENSE) label = labels[col];
        float m = -1e30f;
        for (int r = lane; r < K; r += kWave) m = m > p[r] ? m : p[r];
        m = wave_max(m);
        float s = 0.f, picked = 0.f;
        for (int r = lane; r < K; r += kWave) {
            const float x = p[r];
            s += exp_neg(x - m);
            if constexpr (DENSE) picked += x * t[r];
            else if (r == label) picked = x;
        }
        s = wave_sum(s);
        picked = wave_sum(picked);
        if (lane == 0) per_sample[col] = picked - (logf(s) + m);
        if (dlogits) {
            const float invz = static_cast<float>(1.0 / static_cast<double>(s));
            float* d = dlogits + col * ld;
            for (int r = lane; r < K; r += kWave) {
                float yv;
                if constexpr (DENSE) yv = t[r];
                else yv = (r == label) ? 1.0f : 0.0f;
                d[r] = -(yv - exp_neg(p[r] - m) * invz) * inv_n;
            }
        }
    }
}

// out = -mean(v): one block of sixteen waves, four independent loads in flight
// per thread (the per-sample losses are few; a serial loop over them costs more
// than the cross-entropy kernel itself)
constexpr int kMeanBlock = 1024;
__global__ __launch_bounds__(kMeanBlock) void neg_mean_kernel(float* out, const float* v, int n,
                                                              float inv_n) {
    __shared__ float red[kMeanBlock / kWave];
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int i = threadIdx.x;
    for (; i + 3 * kMeanBlock < n; i += 4 * kMeanBlock) {
        const float x0 = v[i], x1 = v[i + kMeanBlock], x2 = v[i + 2 * kMeanBlock], x3 = v[i + 3 * kMeanBlock];
        a0 += x0; a1 += x1; a2 += x2; a3 += x3;
    }
    for (; i < n; i += kMeanBlock) a0 += v[i];
    const float s = block_allreduce<kMeanBlock / kWave>((a0 + a1) + (a2 + a3), SumOp{}, red, 0.f);
    if (threadIdx.x == 0) out[0] = -s * inv_n;
}

template <template <int> class Launcher, class... Args>
int dispatch_nv(int numrow, Args... args) {
    if (numrow <= 64) return Launcher<1>::run(args...);
    if (numrow <= 128) return Launcher<2>::run(args...);
    if (numrow <= 256) return Launcher<4>::run(args...);
    if (numrow <= 512) return Launcher<8>::run(args...);
    return Launcher<16>::run(args...);
}

template <int NV>
struct SoftmaxColsL {
    static int run(float* out, const float* in, int numrow, size_t numcol, size_t ld, ScoreXform xf) {
        const unsigned grid = grid_cover(numcol, kBlock / kWave);
        softmax_cols_kernel<NV><<<grid, kBlock, 0, stream()>>>(out, in, numrow, numcol, ld, xf);
        return launch_rc();
    }
};
template <int NV>
struct SoftmaxBwdColsL {
    static int run(float* dS, const float* A, const float* dA, int numrow, size_t numcol, float scale) {
        const unsigned grid = grid_cover(numcol, kBlock / kWave);
        softmax_bwd_cols_kernel<NV><<<grid, kBlock, 0, stream()>>>(dS, A, dA, numrow, numcol, scale);
        return launch_rc();
    }
};
template <int NV>
struct XentL {
    static int run(float* per_sample, float* dlogits, const float* logits, const int32_t* labels,
                   const float* target, int K, int N, size_t ld, float inv_n) {
        const unsigned grid = grid_cover(N, kBlock / kWave);
        if (target)
            xent_cols_kernel<NV, true><<<grid, kBlock, 0, stream()>>>(per_sample, dlogits, logits, nullptr, target,
                                                                      K, N, ld, inv_n);
        else
            xent_cols_kernel<NV, false><<<grid, kBlock, 0, stream()>>>(per_sample, dlogits, logits, labels, nullptr,
                                                                       K, N, ld, inv_n);
        return launch_rc();
    }
};

int xent_impl(float* per_sample, float* dlogits, const float* logits, const int32_t* labels, const float* target,
              int K, int N, size_t ld, float inv_n) {
    if (K <= 1024) return dispatch_nv<XentL>(K, per_sample, dlogits, logits, labels, target, K, N, ld, inv_n);
    const unsigned grid = grid_cover(N, kBlock / kWave);
    if (target)
        xent_cols_long_kernel<true><<<grid, kBlock, 0, stream()>>>(per_sample, dlogits, logits, nullptr, target, K, N,
                                                                   ld, inv_n);
    else
        xent_cols_long_kernel<false><<<grid, kBlock, 0, stream()>>>(per_sample, dlogits, logits, labels, nullptr, K,
                                                                    N, ld, inv_n);
    return launch_rc();
}

int softmax_cols_impl(float* out, const float* in, int numrow, size_t numcol, size_t ld,
                      ScoreXform xf) {
    if (numrow <= 1024) return dispatch_nv<SoftmaxColsL>(numrow, out, in, numrow, numcol, ld, xf);
    if (xf.S) return -1;
    if (numrow % 4 == 0 && ld % 4 == 0 && numrow <= 16 * 1024 && aligned16(in) && aligned16(out) &&
        numcol <= 0x7fffffffull) {
        const unsigned grid = static_cast<unsigned>(numcol);
        hipStream_t st = stream();
        // (2048 x 16384, 0.5 GB: 41 us plain, 43 hinted; 16384^2, 2 GB: 418 -> 372 us)
        const bool nt = streams_past_cache(static_cast<size_t>(numrow) * numcol * sizeof(float));
#define JZ_SOFTMAX_BLOCK(NV4_, BLOCK_)                                                                          \
    do {                                                                                                        \
        if (nt) softmax_cols_block_kernel<NV4_, BLOCK_, true><<<grid, BLOCK_, 0, st>>>(out, in, numrow, numcol, ld);  \
        else softmax_cols_block_kernel<NV4_, BLOCK_, false><<<grid, BLOCK_, 0, st>>>(out, in, numrow, numcol, ld);    \
    } while (0)
        if (numrow <= 2048) JZ_SOFTMAX_BLOCK(2, kBlock);
        else if (numrow <= 4096) JZ_SOFTMAX_BLOCK(4, kBlock);
        else if (numrow <= 8192) JZ_SOFTMAX_BLOCK(2, 1024);
        else JZ_SOFTMAX_BLOCK(4, 1024);
#undef JZ_SOFTMAX_BLOCK
        return launch_rc();
    }
    const unsigned grid = grid_for(numcol, 1, 8);
    softmax_cols_long_kernel<<<grid, kBlock, 0, stream()>>>(out, in, numrow, numcol, ld);
    return launch_rc();
}

// Rows of at most 2048 columns: one read and one write per element, the split of the
// workgroup chosen from the shapes measured (us on MI355X in brackets).
int softmax_rows_single_read(float* out, const float* in, int numrow, int numcol, size_t ld, hipStream_t s) {
#define JZ_ROWS_TILE(T, RL, NV)                                                                              \
    do {                                                                                                     \
        softmax_rows_tile_kernel<T, RL, NV><<<(numrow + RL - 1) / RL, T, 0, s>>>(out, in, numrow, numcol, ld); \
        return launch_rc();                                                                                  \
    } while (0)
#define JZ_ROWS_TILE4(T, RL4, NV)                                                                                      \
    do {                                                                                                               \
        softmax_rows_tile4_kernel<T, RL4, NV><<<(numrow / 4 + RL4 - 1) / RL4, T, 0, s>>>(out, in, numrow, numcol, ld); \
        return launch_rc();                                                                                            \
    } while (0)
    const bool f4 = numrow % 4 == 0 && ld % 4 == 0 && aligned16(in) && aligned16(out);
    if (numcol <= 256) {
        if (f4 && numrow >= 16384) JZ_ROWS_TILE4(256, 16, 16);   // 131072 x 256: 41 us, 6.5 TB/s (64 scalar row lanes: 94)
        if (f4) JZ_ROWS_TILE4(256, 8, 8);                        // 16384 x 128: 5.4 us
        JZ_ROWS_TILE(1024, 64, 16);                              // 131072 x 256: 44 us
    }
    if (numcol <= 512) {
        if (f4 && numrow >= 4096) JZ_ROWS_TILE4(512, 8, 8);      // 16384 x 512: 14.3 us (scalar 16 x 64 split: 22)
        if (numrow >= 4096) JZ_ROWS_TILE(1024, 64, 32);          // 16384 x 512: 15.2 us
        JZ_ROWS_TILE(512, 8, 8);                                 // 512 x 512: 3.9 us, 1024 x 512: 4.1 us
    }
    if (numcol <= 1024) {
        if (f4 && numrow >= 4096) JZ_ROWS_TILE4(1024, 8, 8);     // 4096 x 1024: 11.2 us, 65536 x 1024: 142 us
        if (numrow >= 4096) JZ_ROWS_TILE(1024, 32, 32);          // 4096 x 1024: 11.3 us
        if (numrow >= 2048) JZ_ROWS_TILE(1024, 16, 16);          // 2048 x 1024: 6.7 us
        JZ_ROWS_TILE(512, 8, 16);                                // 1024 x 1024: 5.8 us (column form: 5.7)
    }
    if (f4 && numrow >= 8192) JZ_ROWS_TILE4(512, 8, 32);         // 16384 x 2048: 57 us (16 x 64 split: 80), 65536 x 2048: 292 (411)
    if (f4) JZ_ROWS_TILE4(512, 4, 16);                           // 2048 x 2048: 15.1 us
    if (numrow >= 8192) JZ_ROWS_TILE(1024, 32, 64);              // 16384 x 2048: 68 us
    JZ_ROWS_TILE(1024, 16, 32);                                  // 2048 x 2048: 15.0 us
#undef JZ_ROWS_TILE
#undef JZ_ROWS_TILE4
}

int softmax_rows_impl(float* out, const float* in, int numrow, int numcol, size_t ld, int batch,
                      size_t batch_stride, ScoreXform xf) {
    if (batch > 65535) return -1;
    hipStream_t s = stream();
    const int row_blocks = (numrow + kWave - 1) / kWave;
    if (batch == 1 && !xf.S && numcol <= 2048 && numrow >= 256)
        return softmax_rows_single_read(out, in, numrow, numcol, ld, s);
    if (numcol <= 256) {
        // whole row in registers (batches of score blocks, short matrices)
        dim3 grid(row_blocks, batch);
        if (numcol <= 16)
            softmax_rows_reg_kernel<4><<<grid, kBlock, 0, s>>>(out, in, numrow, numcol, ld, batch_stride, xf);
        else if (numcol <= 64)
            softmax_rows_reg_kernel<16><<<grid, kBlock, 0, s>>>(out, in, numrow, numcol, ld, batch_stride, xf);
        else if (numcol <= 128)
            softmax_rows_reg_kernel<32><<<grid, kBlock, 0, s>>>(out, in, numrow, numcol, ld, batch_stride, xf);
        else
            softmax_rows_reg_kernel<64><<<grid, kBlock, 0, s>>>(out, in, numrow, numcol, ld, batch_stride, xf);
        return launch_rc();
    }
    if (batch == 1 && !xf.S) {
        // long rows: two passes with the columns split over grid.y so that
        // row_blocks x chunks fills the chip.  (Measured and dropped: four rows per lane with
        // float4 loads, 672 against 680 us at 16384 x 16384 and slower below; walking the
        // matrix in 64 MB strips of rows so that the second pass would find its strip in the
        // memory-side cache, 899 us.)
        int chunks = static_cast<int>((static_cast<size_t>(num_cus()) * 8 + row_blocks - 1) / row_blocks);
        if (chunks > numcol / 32) chunks = numcol / 32;
        if (chunks < 1) chunks = 1;
        if (chunks > 512) chunks = 512;   // the fold walks them once per row
        auto need = [&](int ch) { return (static_cast<size_t>(ch) + 1) * numrow * 2; };
        while (chunks > 1 && need(chunks) > kWorkspaceFloats) --chunks;
        const int chunk_len = (numcol + chunks - 1) / chunks;
        chunks = (numcol + chunk_len - 1) / chunk_len;
        if (need(chunks) <= kWorkspaceFloats) {
            float* part = workspace();
            if (!part) return -2;
            float* rowstat = part + static_cast<size_t>(chunks) * numrow * 2;
            dim3 grid(row_blocks, chunks);
            // Loads stay plain in both passes (what the first pass leaves in the memory-side
            // cache serves part of the second); the result is written with the streaming hint
            // from 192 MB up, where it would only push the input out of that cache.  Measured,
            // plain / hinted loads and stores / hinted stores only: 16384 x 4096 175 / 164 / 131 us,
            // 8192 x 8192 180 / 167 / 134, 16384 x 16384 673 / 624 / 603; 2048 x 16384 (134 MB)
            // 70 / 82 / 72, so smaller matrices keep plain stores.
            const bool nt_out = static_cast<size_t>(numrow) * numcol * sizeof(float) >= (size_t(192) << 20);
            softmax_rows_partial_kernel<false><<<grid, kBlock, 0, s>>>(part, in, numrow, numcol, ld, chunk_len);
            softmax_rows_fold_kernel<<<row_blocks, kFoldThreads, 0, s>>>(rowstat, part, numrow, chunks);
            if (nt_out) softmax_rows_apply_kernel<true><<<grid, kBlock, 0, s>>>(out, in, rowstat, numrow, numcol, ld, chunk_len);
            else softmax_rows_apply_kernel<false><<<grid, kBlock, 0, s>>>(out, in, rowstat, numrow, numcol, ld, chunk_len);
            return launch_rc();
        }
    }
    // general fallback: three sweeps per 64-row strip
    dim3 grid(row_blocks, batch);
    softmax_rows_kernel<64><<<grid, kBlock, 0, s>>>(out, in, numrow, numcol, ld, batch_stride, xf);
    return launch_rc();
}

}  // namespace
}  // namespace jz

using namespace jz;

JZ_API int jzhip_softmax_cols(float* out, const float* in, int numrow, int numcol, int ld) {
    if (numrow <= 0 || numcol <= 0 || ld < numrow || !out || !in) return -1;
    return softmax_cols_impl(out, in, numrow, numcol, ld, ScoreXform{1.f, 0, 0});
}

JZ_API int jzhip_softmax_rows(float* out, const float* in, int numrow, int numcol, int ld) {
    if (numrow <= 0 || numcol <= 0 || ld < numrow || !out || !in) return -1;
    return softmax_rows_impl(out, in, numrow, numcol, ld, 1, 0, ScoreXform{1.f, 0, 0});
}

JZ_API int jzhip_attn_softmax(float* out, const float* in, int S, int nblk, float scale,
                              int causal, int keys_along_rows) {
    if (S <= 0 || nblk <= 0 || !out || !in) return -1;
    const ScoreXform xf{scale, causal ? 1 : 0, S};
    if (keys_along_rows) {
        return softmax_cols_impl(out, in, S, static_cast<size_t>(S) * nblk, S, xf);
    }
    // blocks are independent S x S matrices; split the batch over grid.y
    int done = 0;
    while (done < nblk) {
        const int nb = (nblk - done) < 65535 ? (nblk - done) : 65535;
        const size_t off = static_cast<size_t>(done) * S * S;
        int rc = softmax_rows_impl(out + off, in + off, S, S, S, nb, static_cast<size_t>(S) * S, xf);
        if (rc) return rc;
        done += nb;
    }
    return 0;
}

JZ_API int jzhip_attn_softmax_bwd(float* dS, const float* A, const float* dA, int S, int nblk,
                                  float scale, int keys_along_rows) {
    if (S <= 0 || nblk <= 0 || !dS || !A || !dA) return -1;
    if (keys_along_rows) {
        if (S > 1024) return -1;
        return dispatch_nv<SoftmaxBwdColsL>(S, dS, A, dA, S, static_cast<size_t>(S) * nblk, scale);
    }
    int done = 0;
    while (done < nblk) {
        const int nb = (nblk - done) < 65535 ? (nblk - done) : 65535;
        const size_t off = static_cast<size_t>(done) * S * S;
        dim3 grid((S + 63) / 64, nb);
        softmax_bwd_rows_kernel<64><<<grid, kBlock, 0, stream()>>>(dS + off, A + off, dA + off, S, scale);
        int rc = launch_rc();
        if (rc) return rc;
        done += nb;
    }
    return 0;
}

JZ_API int jzhip_softmax_xent(float* loss_out, float* dlogits, const float* logits,
                              const int32_t* labels, int K, int N, int ld) {
    if (K <= 0 || N <= 0 || ld < K || !loss_out || !logits || !labels) return -1;
    if (static_cast<size_t>(N) > kWorkspaceFloats) return -1;
    float* per_sample = workspace();
    if (!per_sample) return -2;
    int rc = xent_impl(per_sample, dlogits, logits, labels, nullptr, K, N, static_cast<size_t>(ld),
                       static_cast<float>(1.0 / N));
    if (rc) return rc;
    neg_mean_kernel<<<1, kMeanBlock, 0, stream()>>>(loss_out, per_sample, N, static_cast<float>(1.0 / N));
    return launch_rc();
}

JZ_API int jzhip_softmax_xent_dense(float* loss_out, float* dlogits, const float* logits, const float* target,
                                    int K, int N, int ld, float inv_nb) {
    if (K <= 0 || N <= 0 || ld < K || !logits || !target || (!loss_out && !dlogits)) return -1;
    if (static_cast<size_t>(N) > kWorkspaceFloats) return -1;
    float* per_sample = workspace();
    if (!per_sample) return -2;
    int rc = xent_impl(per_sample, dlogits, logits, nullptr, target, K, N, static_cast<size_t>(ld), inv_nb);
    if (rc || !loss_out) return rc;
    neg_mean_kernel<<<1, kMeanBlock, 0, stream()>>>(loss_out, per_sample, N, inv_nb);
    return launch_rc();
}
