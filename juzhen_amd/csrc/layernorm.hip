// Fused LayerNorm forward / backward over the columns of a (dim x N)
// column-major activation matrix: one wavefront per token column, the column
// held in registers between the statistics and the normalisation, so x is read
// once and y / xhat written once (the reference's generic formulation is ~12
// matrix ops and four rank-1 GEMMs per call, ml/layer.hpp:2632-2639,2674-2681).
//
// Arithmetic mirrors the generic formulation: mean = sum(x)/dim, centred
// two-pass biased variance, inv = 1.0f/sqrtf(var + 1e-5f).
#include "common.hpp"

#include <cmath>

namespace jz {
namespace {

constexpr float kLnEps = 1e-5f;

// NV float4 per lane: dim <= 256*NV, dim % 4 == 0, 16-byte aligned columns.
// NT: the streaming hint on the column data (launches past the cache size).
template <int NV, bool NT>
__global__ __launch_bounds__(kBlock) void ln_fwd_vec_kernel(float* y, float* xhat, float* inv_std,
                                                            const float* x, const float* gamma,
                                                            const float* beta, int dim, int N) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t wave0 = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
    const size_t nwaves = static_cast<size_t>(gridDim.x) * (kBlock / kWave);
    const float invdim = 1.0f / static_cast<float>(dim);

    float4 g[NV], b[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int r = (lane + v * kWave) * 4;
        if (r < dim) {
            g[v] = *reinterpret_cast<const float4*>(gamma + r);
            b[v] = *reinterpret_cast<const float4*>(beta + r);
        }
    }
    for (size_t col = wave_begin(static_cast<size_t>(N), wave0, nwaves), col_end = wave_end(static_cast<size_t>(N), wave0, nwaves); col < col_end; ++col) {
        const size_t base = col * dim;
        float4 xv[NV];
        float s = 0.f;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int r = (lane + v * kWave) * 4;
            if (r < dim) {
                xv[v] = load4<NT>(x + base + r);
                s += (xv[v].x + xv[v].y) + (xv[v].z + xv[v].w);
            }
        }
        const float mu = wave_sum(s) * invdim;
        float q = 0.f;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int r = (lane + v * kWave) * 4;
            if (r < dim) {
                xv[v].x -= mu; xv[v].y -= mu; xv[v].z -= mu; xv[v].w -= mu;
                q += (xv[v].x * xv[v].x + xv[v].y * xv[v].y) + (xv[v].z * xv[v].z + xv[v].w * xv[v].w);
            }
        }
        const float var = wave_sum(q) * invdim;
        const float inv = 1.0f / sqrtf(var + kLnEps);
        if (lane == 0) inv_std[col] = inv;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int r = (lane + v * kWave) * 4;
            if (r < dim) {
                float4 h, o;
                h.x = xv[v].x * inv; h.y = xv[v].y * inv; h.z = xv[v].z * inv; h.w = xv[v].w * inv;
                o.x = g[v].x * h.x + b[v].x; o.y = g[v].y * h.y + b[v].y;
                o.z = g[v].z * h.z + b[v].z; o.w = g[v].w * h.w + b[v].w;
                store4<NT>(xhat + base + r, h);
                store4<NT>(y + base + r, o);
            }
        }
    }
}

// Any dim / alignment: one wavefront per column, three sweeps (L1/L2 hits).
__global__ __launch_bounds__(kBlock) void ln_fwd_generic_kernel(float* y, float* xhat,
                                                                float* inv_std, const float* x,
                                                                const float* gamma,
                                                                const float* beta, int dim, int N) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t wave0 = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
    const size_t nwaves = static_cast<size_t>(gridDim.x) * (kBlock / kWave);
    const float invdim = 1.0f / static_cast<float>(dim);
    for (size_t col = wave_begin(static_cast<size_t>(N), wave0, nwaves), col_end = wave_end(static_cast<size_t>(N), wave0, nwaves); col < col_end; ++col) {
        const size_t base = col * dim;
        float s = 0.f;
        for (int r = lane; r < dim; r += kWave) s += x[base + r];
        const float mu = wave_sum(s) * invdim;
        float q = 0.f;
        for (int r = lane; r < dim; r += kWave) {
            const float c = x[base + r] - mu;
            q += c * c;
        }
        const float var = wave_sum(q) * invdim;
        const float inv = 1.0f / sqrtf(var + kLnEps);
        if (lane == 0) inv_std[col] = inv;
        for (int r = lane; r < dim; r += kWave) {
            const float h = (x[base + r] - mu) * inv;
            xhat[base + r] = h;
            y[base + r] = gamma[r] * h + beta[r];
        }
    }
}

// JVP = false: dx = P(gamma .* dy) (+ res), the backward pass.  JVP = true:
// out = gamma .* P(dy), the tangent through the same standardisation operator
// P(v) = inv .* (v - mean(v) - xhat .* mean(xhat .* v)) (ml/layer.hpp:2690-2702).
template <int NV, bool JVP, bool NT>
__global__ __launch_bounds__(kBlock) void ln_bwd_vec_kernel(float* dx, const float* dy,
                                                            const float* gamma, const float* xhat,
                                                            const float* inv_std, const float* res,
                                                            int dim, int N) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t wave0 = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
    const size_t nwaves = static_cast<size_t>(gridDim.x) * (kBlock / kWave);
    const float invdim = 1.0f / static_cast<float>(dim);
    float4 g[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int r = (lane + v * kWave) * 4;
        if (r < dim) g[v] = *reinterpret_cast<const float4*>(gamma + r);
    }
    for (size_t col = wave_begin(static_cast<size_t>(N), wave0, nwaves), col_end = wave_end(static_cast<size_t>(N), wave0, nwaves); col < col_end; ++col) {
        const size_t base = col * dim;
        float4 d[NV], h[NV];
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int r = (lane + v * kWave) * 4;
            if (r < dim) {
                d[v] = load4<NT>(dy + base + r);
                h[v] = load4<NT>(xhat + base + r);
                if constexpr (!JVP) { d[v].x *= g[v].x; d[v].y *= g[v].y; d[v].z *= g[v].z; d[v].w *= g[v].w; }
                s1 += (d[v].x + d[v].y) + (d[v].z + d[v].w);
                s2 += (d[v].x * h[v].x + d[v].y * h[v].y) + (d[v].z * h[v].z + d[v].w * h[v].w);
            }
        }
        const float m1 = wave_sum(s1) * invdim;
        const float m2 = wave_sum(s2) * invdim;
        const float inv = inv_std[col];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int r = (lane + v * kWave) * 4;
            if (r < dim) {
                float4 o;
                o.x = inv * (d[v].x - m1 - h[v].x * m2);
                o.y = inv * (d[v].y - m1 - h[v].y * m2);
                o.z = inv * (d[v].z - m1 - h[v].z * m2);
                o.w = inv * (d[v].w - m1 - h[v].w * m2);
                if constexpr (JVP) { o.x *= g[v].x; o.y *= g[v].y; o.z *= g[v].z; o.w *= g[v].w; }
                if (res) {  // dx = LN'(dy) + res, rounded like a separate add
                    const float4 rr = load4<NT>(res + base + r);
                    o.x += rr.x; o.y += rr.y; o.z += rr.z; o.w += rr.w;
                }
                store4<NT>(dx + base + r, o);
            }
        }
    }
}

template <bool JVP>
__global__ __launch_bounds__(kBlock) void ln_bwd_generic_kernel(float* dx, const float* dy,
                                                                const float* gamma,
                                                                const float* xhat,
                                                                const float* inv_std,
                                                                const float* res, int dim, int N) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t wave0 = (static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x) / kWave;
    const size_t nwaves = static_cast<size_t>(gridDim.x) * (kBlock / kWave);
    const float invdim = 1.0f / static_cast<float>(dim);
    for (size_t col = wave_begin(static_cast<size_t>(N), wave0, nwaves), col_end = wave_end(static_cast<size_t>(N), wave0, nwaves); col < col_end; ++col) {
        const size_t base = col * dim;
        float s1 = 0.f, s2 = 0.f;
        for (int r = lane; r < dim; r += kWave) {
            const float d = JVP ? dy[base + r] : dy[base + r] * gamma[r];
            s1 += d;
            s2 += d * xhat[base + r];
        }
        const float m1 = wave_sum(s1) * invdim;
        const float m2 = wave_sum(s2) * invdim;
        const float inv = inv_std[col];
        for (int r = lane; r < dim; r += kWave) {
            const float d = JVP ? dy[base + r] : dy[base + r] * gamma[r];
            float o = inv * (d - m1 - xhat[base + r] * m2);
            if constexpr (JVP) o *= gamma[r];
            if (res) o += res[base + r];
            dx[base + r] = o;
        }
    }
}

// dgamma / dbeta partials: lanes along rows, waves along column phases of the
// block's column chunk.  part layout: [chunk][2][dim].
__global__ __launch_bounds__(kBlock) void ln_param_partial_kernel(float* part, const float* dy,
                                                                  const float* xhat, int dim, int N,
                                                                  int chunk_len) {
    constexpr int NW = kBlock / kWave;
    __shared__ float red[2][NW][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int row = blockIdx.x * kWave + lane;
    const int chunk = blockIdx.y;
    const int c_begin = chunk * chunk_len;
    int c_end = c_begin + chunk_len;
    if (c_end > N) c_end = N;
    float ag = 0.f, ab = 0.f;
    if (row < dim) {
        for (int c = c_begin + wave; c < c_end; c += NW) {
            const size_t i = static_cast<size_t>(c) * dim + row;
            const float d = dy[i];
            ag += d * xhat[i];
            ab += d;
        }
    }
    red[0][wave][lane] = ag;
    red[1][wave][lane] = ab;
    __syncthreads();
    if (wave == 0 && row < dim) {
        float sg = 0.f, sb = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            sg += red[0][w][lane];
            sb += red[1][w][lane];
        }
        part[(static_cast<size_t>(chunk) * 2 + 0) * dim + row] = sg;
        part[(static_cast<size_t>(chunk) * 2 + 1) * dim + row] = sb;
    }
}

// float4 form (dim % 4 == 0, aligned operands): a lane owns four rows, a wave
// 256 rows; each wave walks its columns four at a time, so eight 16-byte loads
// are in flight per lane.
template <bool NT>
__global__ __launch_bounds__(kBlock) void ln_param_partial_vec_kernel(float* part, const float* dy,
                                                                      const float* xhat, int dim, int N,
                                                                      int chunk_len) {
    constexpr int NW = kBlock / kWave;
    __shared__ float4 red[2][NW][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int row = (blockIdx.x * kWave + lane) * 4;
    const int chunk = blockIdx.y;
    const int c_begin = chunk * chunk_len;
    int c_end = c_begin + chunk_len;
    if (c_end > N) c_end = N;
    float4 ag = make_float4(0.f, 0.f, 0.f, 0.f), ab = ag;
    if (row < dim) {
        for (int c = c_begin + wave; c < c_end; c += NW * 4) {
            float4 d[4], h[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int cc = c + u * NW;
                if (cc < c_end) {
                    const size_t i = static_cast<size_t>(cc) * dim + row;
                    d[u] = load4<NT>(dy + i);
                    h[u] = load4<NT>(xhat + i);
                } else {
                    d[u] = make_float4(0.f, 0.f, 0.f, 0.f);
                    h[u] = d[u];
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                ag.x += d[u].x * h[u].x; ag.y += d[u].y * h[u].y; ag.z += d[u].z * h[u].z; ag.w += d[u].w * h[u].w;
                ab.x += d[u].x; ab.y += d[u].y; ab.z += d[u].z; ab.w += d[u].w;
            }
        }
    }
    red[0][wave][lane] = ag;
    red[1][wave][lane] = ab;
    __syncthreads();
    if (wave == 0 && row < dim) {
        float4 sg = make_float4(0.f, 0.f, 0.f, 0.f), sb = sg;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const float4 a = red[0][w][lane], b = red[1][w][lane];
            sg.x += a.x; sg.y += a.y; sg.z += a.z; sg.w += a.w;
            sb.x += b.x; sb.y += b.y; sb.z += b.z; sb.w += b.w;
        }
        *reinterpret_cast<float4*>(part + (static_cast<size_t>(chunk) * 2 + 0) * dim + row) = sg;
        *reinterpret_cast<float4*>(part + (static_cast<size_t>(chunk) * 2 + 1) * dim + row) = sb;
    }
}

// part is [chunk][2*dim]; a block owns 64 of the 2*dim outputs, its waves take
// interleaved chunks and are combined through LDS.
constexpr int kCombineThreads = 1024;
__global__ __launch_bounds__(kCombineThreads) void ln_param_combine_kernel(float* dgamma, float* dbeta,
                                                                           const float* part, int dim,
                                                                           int chunks) {
    constexpr int NW = kCombineThreads / kWave;
    __shared__ float red[NW][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int i = blockIdx.x * kWave + lane;
    const int n = 2 * dim;
    float acc = 0.f;
    if (i < n) {
        int c = wave;
        for (; c + 3 * NW < chunks; c += 4 * NW) {   // four loads in flight
            const float a0 = part[static_cast<size_t>(c) * n + i];
            const float a1 = part[static_cast<size_t>(c + NW) * n + i];
            const float a2 = part[static_cast<size_t>(c + 2 * NW) * n + i];
            const float a3 = part[static_cast<size_t>(c + 3 * NW) * n + i];
            acc += (a0 + a1) + (a2 + a3);
        }
        for (; c < chunks; c += NW) acc += part[static_cast<size_t>(c) * n + i];
    }
    red[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && i < n) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) s += red[w][lane];
        if (i < dim) dgamma[i] = s; else dbeta[i - dim] = s;
    }
}

// The backward pass with everything else that is summed over the tokens in the same sweep:
// dx = P(gamma .* dy) + res as ln_bwd_vec_kernel, and per row the sums over the columns of
// dy .* xhat (dgamma), dy (dbeta), dx and res (the bias gradients of the dense layers on
// either side of the residual add).  A wave keeps its rows and walks a run of columns, so
// the four sums are 4*NV float4 accumulators per lane; the waves of a workgroup meet in LDS
// (wave w adds up sum w in wave order) and leave part[block][4][dim].
template <int NV, bool NT>
__global__ __launch_bounds__(kBlock) void ln_bwd_sums_vec_kernel(float* dx, const float* dy, const float* gamma,
                                                                 const float* xhat, const float* inv_std,
                                                                 const float* res, float* part, int dim, int N) {
    constexpr int NW = kBlock / kWave;
    static_assert(NW == 4, "one wave per sum in the closing step");
    __shared__ float4 red[4][NW][NV][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const size_t wave0 = static_cast<size_t>(blockIdx.x) * NW + wave;
    const size_t nwaves = static_cast<size_t>(gridDim.x) * NW;
    const float invdim = 1.0f / static_cast<float>(dim);
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 g[NV], acc[4][NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int r = (lane + v * kWave) * 4;
        g[v] = r < dim ? *reinterpret_cast<const float4*>(gamma + r) : zero;
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[q][v] = zero;
    }
    // the next column's operands are requested before the current one is worked on
    const size_t col_begin = wave_begin(static_cast<size_t>(N), wave0, nwaves);
    const size_t col_end = wave_end(static_cast<size_t>(N), wave0, nwaves);
    float4 d[NV], h[NV], rr[NV], dn[NV], hn[NV], rn[NV];
    auto fetch = [&](float4 (&fd)[NV], float4 (&fh)[NV], float4 (&fr)[NV], size_t col) {
        const size_t base = col * dim;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int r = (lane + v * kWave) * 4;
            if (r < dim) {
                fd[v] = load4<NT>(dy + base + r);
                fh[v] = load4<NT>(xhat + base + r);
                fr[v] = res ? load4<NT>(res + base + r) : zero;
            } else {
                fd[v] = zero; fh[v] = zero; fr[v] = zero;
            }
        }
    };
    if (col_begin < col_end) fetch(dn, hn, rn, col_begin);
    for (size_t col = col_begin; col < col_end; ++col) {
        const size_t base = col * dim;
#pragma unroll
        for (int v = 0; v < NV; ++v) { d[v] = dn[v]; h[v] = hn[v]; rr[v] = rn[v]; }
        if (col + 1 < col_end) fetch(dn, hn, rn, col + 1);
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int r = (lane + v * kWave) * 4;
            if (r < dim) {
                acc[0][v].x += d[v].x * h[v].x; acc[0][v].y += d[v].y * h[v].y;
                acc[0][v].z += d[v].z * h[v].z; acc[0][v].w += d[v].w * h[v].w;
                acc[1][v].x += d[v].x; acc[1][v].y += d[v].y; acc[1][v].z += d[v].z; acc[1][v].w += d[v].w;
                d[v].x *= g[v].x; d[v].y *= g[v].y; d[v].z *= g[v].z; d[v].w *= g[v].w;
                s1 += (d[v].x + d[v].y) + (d[v].z + d[v].w);
                s2 += (d[v].x * h[v].x + d[v].y * h[v].y) + (d[v].z * h[v].z + d[v].w * h[v].w);
            }
        }
        const float m1 = wave_sum(s1) * invdim;
        const float m2 = wave_sum(s2) * invdim;
        const float inv = inv_std[col];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int r = (lane + v * kWave) * 4;
            if (r < dim) {
                float4 o;
                o.x = inv * (d[v].x - m1 - h[v].x * m2);
                o.y = inv * (d[v].y - m1 - h[v].y * m2);
                o.z = inv * (d[v].z - m1 - h[v].z * m2);
                o.w = inv * (d[v].w - m1 - h[v].w * m2);
                if (res) {  // rounded like a separate add
                    o.x += rr[v].x; o.y += rr[v].y; o.z += rr[v].z; o.w += rr[v].w;
                    acc[3][v].x += rr[v].x; acc[3][v].y += rr[v].y; acc[3][v].z += rr[v].z; acc[3][v].w += rr[v].w;
                }
                acc[2][v].x += o.x; acc[2][v].y += o.y; acc[2][v].z += o.z; acc[2][v].w += o.w;
                store4<NT>(dx + base + r, o);
            }
        }
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int v = 0; v < NV; ++v) red[q][wave][v][lane] = acc[q][v];
    __syncthreads();
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int r = (lane + v * kWave) * 4;
        if (r < dim) {
            float4 sum = red[wave][0][v][lane];
#pragma unroll
            for (int w = 1; w < NW; ++w) {
                const float4 t = red[wave][w][v][lane];
                sum.x += t.x; sum.y += t.y; sum.z += t.z; sum.w += t.w;
            }
            *reinterpret_cast<float4*>(part + (static_cast<size_t>(blockIdx.x) * 4 + wave) * dim + r) = sum;
        }
    }
}

// part is [chunk][4*dim]; a block owns 16 of the 4*dim outputs (128 blocks at dim 512, so that
// the few MB of partial sums are read by half the chip rather than an eighth of it): the four
// 16-lane groups of a wave and the sixteen waves take interleaved chunks, meet by lane exchange
// and through LDS, always in the same order; a sum nobody asked for (null pointer) is skipped.
constexpr int kSumsOutputs = 16;
__global__ __launch_bounds__(kCombineThreads) void ln_sums_combine_kernel(float* s0, float* s1, float* s2, float* s3,
                                                                          const float* part, int dim, int chunks) {
    constexpr int NW = kCombineThreads / kWave;
    constexpr int PH = kWave / kSumsOutputs;      // chunk phases inside a wave
    __shared__ float red[NW][kSumsOutputs];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int o = lane % kSumsOutputs, ph = lane / kSumsOutputs;
    const int i = blockIdx.x * kSumsOutputs + o;
    const int n = 4 * dim;
    const int which = i < n ? i / dim : 0;
    float* dst = which == 0 ? s0 : which == 1 ? s1 : which == 2 ? s2 : s3;
    float acc = 0.f;
    if (i < n && dst) {
        constexpr int STEP = NW * PH;
        int c = wave * PH + ph;
        for (; c + 3 * STEP < chunks; c += 4 * STEP) {   // four loads in flight
            const float a0 = part[static_cast<size_t>(c) * n + i];
            const float a1 = part[static_cast<size_t>(c + STEP) * n + i];
            const float a2 = part[static_cast<size_t>(c + 2 * STEP) * n + i];
            const float a3 = part[static_cast<size_t>(c + 3 * STEP) * n + i];
            acc += (a0 + a1) + (a2 + a3);
        }
        for (; c < chunks; c += STEP) acc += part[static_cast<size_t>(c) * n + i];
    }
    acc += __shfl_xor(acc, 16, kWave);
    acc += __shfl_xor(acc, 32, kWave);
    if (ph == 0) red[wave][o] = acc;
    __syncthreads();
    if (threadIdx.x < kSumsOutputs && i < n && dst) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) s += red[w][o];
        dst[i - which * dim] = s;
    }
}

}  // namespace
}  // namespace jz

using namespace jz;

JZ_API int jzhip_layernorm_fwd(float* y, float* xhat, float* inv_std, const float* x,
                               const float* gamma, const float* beta, int dim, int N) {
    if (dim <= 0 || N <= 0 || !y || !xhat || !inv_std || !x || !gamma || !beta) return -1;
    const bool vec = (dim % 4 == 0) && dim <= 1024 && aligned16(x) && aligned16(y) &&
                     aligned16(xhat) && aligned16(gamma) && aligned16(beta);
    const unsigned grid = grid_cover(N, kBlock / kWave);
    hipStream_t s = stream();
    const bool nt = streams_past_cache(3 * static_cast<size_t>(dim) * N * sizeof(float));
#define JZ_LN_FWD(NV_)                                                                                        \
    do {                                                                                                      \
        if (nt) ln_fwd_vec_kernel<NV_, true><<<grid, kBlock, 0, s>>>(y, xhat, inv_std, x, gamma, beta, dim, N);   \
        else ln_fwd_vec_kernel<NV_, false><<<grid, kBlock, 0, s>>>(y, xhat, inv_std, x, gamma, beta, dim, N);     \
    } while (0)
    if (vec && dim <= 256) JZ_LN_FWD(1);
    else if (vec && dim <= 512) JZ_LN_FWD(2);
    else if (vec) JZ_LN_FWD(4);
#undef JZ_LN_FWD
    else
        ln_fwd_generic_kernel<<<grid, kBlock, 0, s>>>(y, xhat, inv_std, x, gamma, beta, dim, N);
    return launch_rc();
}

namespace {
template <bool JVP>
int launch_ln_bwd(float* dx, const float* dy, const float* gamma, const float* xhat, const float* inv_std,
                  const float* res, int dim, int N) {
    if (dim <= 0 || N <= 0 || !dx || !dy || !gamma || !xhat || !inv_std) return -1;
    const bool vec = (dim % 4 == 0) && dim <= 1024 && aligned16(dx) && aligned16(dy) &&
                     aligned16(xhat) && aligned16(gamma) && (!res || aligned16(res));
    const unsigned grid = grid_cover(N, kBlock / kWave);
    hipStream_t s = stream();
    const bool nt = streams_past_cache((res ? 4 : 3) * static_cast<size_t>(dim) * N * sizeof(float));
#define JZ_LN_BWD(NV_)                                                                                             \
    do {                                                                                                           \
        if (nt) ln_bwd_vec_kernel<NV_, JVP, true><<<grid, kBlock, 0, s>>>(dx, dy, gamma, xhat, inv_std, res, dim, N);  \
        else ln_bwd_vec_kernel<NV_, JVP, false><<<grid, kBlock, 0, s>>>(dx, dy, gamma, xhat, inv_std, res, dim, N);    \
    } while (0)
    if (vec && dim <= 256) JZ_LN_BWD(1);
    else if (vec && dim <= 512) JZ_LN_BWD(2);
    else if (vec) JZ_LN_BWD(4);
#undef JZ_LN_BWD
    else
        ln_bwd_generic_kernel<JVP><<<grid, kBlock, 0, s>>>(dx, dy, gamma, xhat, inv_std, res, dim, N);
    return launch_rc();
}
}  // namespace

JZ_API int jzhip_layernorm_bwd_residual(float* dx, const float* dy, const float* gamma,
                                        const float* xhat, const float* inv_std, const float* res,
                                        int dim, int N) {
    return launch_ln_bwd<false>(dx, dy, gamma, xhat, inv_std, res, dim, N);
}

JZ_API int jzhip_layernorm_bwd_residual_sums(float* dx, const float* dy, const float* gamma, const float* xhat,
                                             const float* inv_std, const float* res, float* dgamma, float* dbeta,
                                             float* sum_dx, float* sum_res, int dim, int N) {
    if (dim <= 0 || N <= 0 || !dx || !dy || !gamma || !xhat || !inv_std || !dgamma || !dbeta) return -1;
    if (sum_res && !res) return -1;
    const bool vec = (dim % 4 == 0) && dim <= 512 && aligned16(dx) && aligned16(dy) && aligned16(xhat) &&
                     aligned16(gamma) && (!res || aligned16(res));
    // workgroups: four per CU, each wave a run of columns; the partial sums are 16*dim bytes per workgroup
    size_t blocks = static_cast<size_t>(num_cus()) * 4;
    const size_t cover = (static_cast<size_t>(N) + kBlock / kWave - 1) / (kBlock / kWave);
    if (blocks > cover) blocks = cover;
    if (vec && N >= 1024 && blocks * 4 * dim <= kWorkspaceFloats) {
        float* part = workspace();
        if (!part) return -2;
        hipStream_t s = stream();
        const bool nt = streams_past_cache((res ? 4 : 3) * static_cast<size_t>(dim) * N * sizeof(float));
        const unsigned grid = static_cast<unsigned>(blocks);
#define JZ_LN_BWD_SUMS(NV_)                                                                                               \
    do {                                                                                                                  \
        if (nt) ln_bwd_sums_vec_kernel<NV_, true><<<grid, kBlock, 0, s>>>(dx, dy, gamma, xhat, inv_std, res, part, dim, N);   \
        else ln_bwd_sums_vec_kernel<NV_, false><<<grid, kBlock, 0, s>>>(dx, dy, gamma, xhat, inv_std, res, part, dim, N);     \
    } while (0)
        if (dim <= 256) JZ_LN_BWD_SUMS(1);
        else JZ_LN_BWD_SUMS(2);
#undef JZ_LN_BWD_SUMS
        ln_sums_combine_kernel<<<(4 * dim + kSumsOutputs - 1) / kSumsOutputs, kCombineThreads, 0, s>>>(dgamma, dbeta, sum_dx, sum_res,
                                                                                         part, dim, static_cast<int>(blocks));
        return launch_rc();
    }
    // other shapes: the separate passes
    int rc = jzhip_layernorm_param_grads(dgamma, dbeta, dy, xhat, dim, N);
    if (rc == 0 && sum_res) rc = jzhip_sum_rows(sum_res, res, dim, N, dim);   // (dx may be res itself)
    if (rc == 0) rc = jzhip_layernorm_bwd_residual(dx, dy, gamma, xhat, inv_std, res, dim, N);
    if (rc == 0 && sum_dx) rc = jzhip_sum_rows(sum_dx, dx, dim, N, dim);
    return rc;
}

JZ_API int jzhip_layernorm_jvp(float* out, const float* dx, const float* gamma, const float* xhat,
                               const float* inv_std, int dim, int N) {
    return launch_ln_bwd<true>(out, dx, gamma, xhat, inv_std, nullptr, dim, N);
}

JZ_API int jzhip_layernorm_bwd(float* dx, const float* dy, const float* gamma, const float* xhat,
                               const float* inv_std, int dim, int N) {
    return jzhip_layernorm_bwd_residual(dx, dy, gamma, xhat, inv_std, nullptr, dim, N);
}

JZ_API int jzhip_layernorm_param_grads(float* dgamma, float* dbeta, const float* dy,
                                       const float* xhat, int dim, int N) {
    if (dim <= 0 || N <= 0 || !dgamma || !dbeta || !dy || !xhat) return -1;
    const bool vec = dim % 4 == 0 && aligned16(dy) && aligned16(xhat);
    const int row_blocks = vec ? (dim / 4 + kWave - 1) / kWave : (dim + kWave - 1) / kWave;
    size_t want = static_cast<size_t>(num_cus()) * 4;
    int chunks = static_cast<int>((want + row_blocks - 1) / row_blocks);
    if (chunks > N / 32) chunks = N / 32;
    if (chunks < 1) chunks = 1;
    if (chunks > 65535) chunks = 65535;
    while (chunks > 1 && static_cast<size_t>(chunks) * 2 * dim > kWorkspaceFloats) --chunks;
    if (static_cast<size_t>(chunks) * 2 * dim > kWorkspaceFloats) return -1;
    const int chunk_len = (N + chunks - 1) / chunks;
    chunks = (N + chunk_len - 1) / chunk_len;
    float* part = workspace();
    if (!part) return -2;
    hipStream_t s = stream();
    dim3 grid(row_blocks, chunks);
    if (vec) {
        if (streams_past_cache(2 * static_cast<size_t>(dim) * N * sizeof(float)))
            ln_param_partial_vec_kernel<true><<<grid, kBlock, 0, s>>>(part, dy, xhat, dim, N, chunk_len);
        else
            ln_param_partial_vec_kernel<false><<<grid, kBlock, 0, s>>>(part, dy, xhat, dim, N, chunk_len);
    } else {
        ln_param_partial_kernel<<<grid, kBlock, 0, s>>>(part, dy, xhat, dim, N, chunk_len);
    }
    ln_param_combine_kernel<<<(2 * dim + kWave - 1) / kWave, kCombineThreads, 0, s>>>(dgamma, dbeta, part, dim, chunks);
    return launch_rc();
}
