// Convolution data movement: im2col, col2im and the channel/space repacking
// kernels of the ROCm ConvLayer / convtransLayer (ml/layer.hpp:1611-1869).
// All index maps are integer-exact restatements of the CPU loops
// (ml/layer.hpp:1897-1999, 2112-2221); values are copied, or summed in the CPU
// loop's order, so results are bit-identical to the oracle.
//
// Three kernels cover the seven entry points:
//   * patch gather  (im2col; convtrans_gather is the same map with the roles
//     of the input and output grids exchanged),
//   * patch scatter-as-gather (col2im; convtrans_scatter is the same map with
//     a bias as the initial value),
//   * batched tile transpose (the four reshape kernels are all
//     (R x C) -> (C x R) per sample, with an optional per-row bias).
#include "common.hpp"

namespace jz {
namespace {

struct PatchGeom {
    int C, H, W;        // image side: channels, height, width
    int kH, kW;
    int pad_h, pad_w, stride_h, stride_w;
    int Hp, Wp;         // patch-grid side (conv output positions)
    int N;
    int K;              // C*kH*kW
    int P;              // Hp*Wp
    FastDiv dK, dP, dWp, dKK, dkW, dCHW, dHW, dW;
};

PatchGeom make_geom(int C, int H, int W, int kH, int kW, int pad_h, int pad_w, int stride_h,
                    int stride_w, int Hp, int Wp, int N) {
    PatchGeom g;
    g.C = C; g.H = H; g.W = W; g.kH = kH; g.kW = kW;
    g.pad_h = pad_h; g.pad_w = pad_w; g.stride_h = stride_h; g.stride_w = stride_w;
    g.Hp = Hp; g.Wp = Wp; g.N = N;
    g.K = C * kH * kW;
    g.P = Hp * Wp;
    g.dK = make_fastdiv(g.K);
    g.dP = make_fastdiv(g.P);
    g.dWp = make_fastdiv(Wp);
    g.dKK = make_fastdiv(kH * kW);
    g.dkW = make_fastdiv(kW);
    g.dCHW = make_fastdiv(C * H * W);
    g.dHW = make_fastdiv(H * W);
    g.dW = make_fastdiv(W);
    return g;
}

// col(K, P*N)[k, c] = image(C*H*W, N)[(ci,ih,iw), n] or 0 in the padding.
// VEC consecutive k per thread (VEC=4 needs K % 4 == 0 and an aligned col).
template <int VEC>
__global__ __launch_bounds__(kBlock) void im2col_kernel(const float* img, float* col, PatchGeom g,
                                                        FastDiv dKv, size_t total_vec) {
    const size_t stride = static_cast<size_t>(gridDim.x) * kBlock;
    const uint32_t kvec = g.K / VEC;
    for (size_t t = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x; t < total_vec; t += stride) {
        // t < 2^31 is guaranteed by the launcher
        const uint32_t tt = static_cast<uint32_t>(t);
        const uint32_t c = fdiv(tt, dKv);
        const uint32_t k0 = (tt - c * kvec) * VEC;
        const uint32_t n = fdiv(c, g.dP);
        const uint32_t p = c - n * g.P;
        const uint32_t ph = fdiv(p, g.dWp);
        const uint32_t pw = p - ph * g.Wp;
        uint32_t ci = fdiv(k0, g.dKK);
        const uint32_t rem = k0 - ci * (g.kH * g.kW);
        uint32_t kh = fdiv(rem, g.dkW);
        uint32_t kw = rem - kh * g.kW;
        const int h0 = static_cast<int>(ph) * g.stride_h - g.pad_h;
        const int w0 = static_cast<int>(pw) * g.stride_w - g.pad_w;
        const float* src = img + static_cast<size_t>(n) * (g.C * g.H * g.W);
        float vals[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            const int ih = h0 + static_cast<int>(kh);
            const int iw = w0 + static_cast<int>(kw);
            float x = 0.0f;
            if (ih >= 0 && ih < g.H && iw >= 0 && iw < g.W)
                x = src[(static_cast<size_t>(ci) * g.H + ih) * g.W + iw];
            vals[v] = x;
            if (++kw == static_cast<uint32_t>(g.kW)) {
                kw = 0;
                if (++kh == static_cast<uint32_t>(g.kH)) {
                    kh = 0;
                    ++ci;
                }
            }
        }
        float* dst = col + static_cast<size_t>(c) * g.K + k0;
        if constexpr (VEC == 4) {
            *reinterpret_cast<float4*>(dst) = make_float4(vals[0], vals[1], vals[2], vals[3]);
        } else {
            dst[0] = vals[0];
        }
    }
}

// image[(ci,ih,iw), n] = init + sum over patch positions (ph asc, pw asc) of
// col[k(ci,kh,kw), c(n,ph,pw)] with ih = ph*stride - pad + kh: the gather form
// of the CPU scatter loop, visiting contributions in the CPU's order
// (ml/layer.hpp:1979-1995: ph ascending, then pw ascending, i.e. kh and kw
// descending).  init = bias[ci] (convtrans forward) or 0 (col2im).
__global__ __launch_bounds__(kBlock) void col2im_kernel(const float* col, float* img,
                                                        const float* bias, PatchGeom g,
                                                        size_t total) {
    const size_t stride = static_cast<size_t>(gridDim.x) * kBlock;
    for (size_t t = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x; t < total; t += stride) {
        const uint32_t tt = static_cast<uint32_t>(t);
        const uint32_t n = fdiv(tt, g.dCHW);
        const uint32_t r = tt - n * (g.C * g.H * g.W);
        const uint32_t ci = fdiv(r, g.dHW);
        const uint32_t rem = r - ci * (g.H * g.W);
        const uint32_t ih = fdiv(rem, g.dW);
        const uint32_t iw = rem - ih * g.W;
        float val = bias ? bias[ci] : 0.0f;
        const float* base = col + static_cast<size_t>(n) * g.P * g.K + static_cast<size_t>(ci) * g.kH * g.kW;
        for (int kh = g.kH - 1; kh >= 0; --kh) {
            const int hn = static_cast<int>(ih) + g.pad_h - kh;
            if (hn < 0) continue;
            const int ph = hn / g.stride_h;
            if (ph * g.stride_h != hn || ph >= g.Hp) continue;
            for (int kw = g.kW - 1; kw >= 0; --kw) {
                const int wn = static_cast<int>(iw) + g.pad_w - kw;
                if (wn < 0) continue;
                const int pw = wn / g.stride_w;
                if (pw * g.stride_w != wn || pw >= g.Wp) continue;
                val += base[static_cast<size_t>(ph * g.Wp + pw) * g.K + kh * g.kW + kw];
            }
        }
        img[t] = val;
    }
}

// dst[b] (C x R, ld = C) = transpose(src[b] (R x C, ld = R)) + bias[r]
constexpr int kT = 32;
__global__ __launch_bounds__(kT * 8) void transpose_batched_kernel(float* dst, const float* src,
                                                                   const float* bias, int R, int C,
                                                                   unsigned tiles_r) {
    __shared__ float tile[kT][kT + 1];
    const size_t boff = static_cast<size_t>(blockIdx.y) * R * C;
    const int r0 = static_cast<int>(blockIdx.x % tiles_r) * kT;
    const int c0 = static_cast<int>(blockIdx.x / tiles_r) * kT;
    const int tx = threadIdx.x % kT, ty = threadIdx.x / kT;
#pragma unroll
    for (int k = 0; k < kT; k += 8) {
        const int r = r0 + tx, c = c0 + ty + k;
        if (r < R && c < C) tile[ty + k][tx] = src[boff + static_cast<size_t>(c) * R + r];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kT; k += 8) {
        const int c = c0 + tx, r = r0 + ty + k;
        if (r < R && c < C) {
            float v = tile[tx][ty + k];
            if (bias) v = v + bias[r];
            dst[boff + static_cast<size_t>(r) * C + c] = v;
        }
    }
}

// float4 form (R, C multiples of 4, aligned buffers): 64x64 tiles, 256 threads
constexpr int kTV = 64;
__global__ __launch_bounds__(kBlock) void transpose_batched_vec_kernel(float* dst, const float* src,
                                                                       const float* bias, int R, int C,
                                                                       unsigned tiles_r) {
    __shared__ float tile[kTV][kTV + 1];
    const size_t boff = static_cast<size_t>(blockIdx.y) * R * C;
    const int r0 = static_cast<int>(blockIdx.x % tiles_r) * kTV;
    const int c0 = static_cast<int>(blockIdx.x / tiles_r) * kTV;
    const int q = threadIdx.x % 16, l = threadIdx.x / 16;
#pragma unroll
    for (int k = 0; k < kTV; k += 16) {
        const int r = r0 + 4 * q, c = c0 + l + k;
        if (r < R && c < C) {
            const float4 v = *reinterpret_cast<const float4*>(src + boff + static_cast<size_t>(c) * R + r);
            float* d = &tile[l + k][4 * q];   // tile[c][r]
            d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
        }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kTV; k += 16) {
        const int c = c0 + 4 * q, r = r0 + l + k;
        if (r < R && c < C) {
            float4 v = make_float4(tile[4 * q][l + k], tile[4 * q + 1][l + k], tile[4 * q + 2][l + k],
                                   tile[4 * q + 3][l + k]);
            if (bias) {
                const float bb = bias[r];
                v.x = v.x + bb; v.y = v.y + bb; v.z = v.z + bb; v.w = v.w + bb;
            }
            *reinterpret_cast<float4*>(dst + boff + static_cast<size_t>(r) * C + c) = v;
        }
    }
}

int transpose_batched(float* dst, const float* src, const float* bias, int R, int C, int batch) {
    if (R <= 0 || C <= 0 || batch <= 0 || !dst || !src) return -1;
    const bool vec = R % 4 == 0 && C % 4 == 0 && aligned16(dst) && aligned16(src);
    if (vec) {
        const unsigned tr = (R + kTV - 1) / kTV, tc = (C + kTV - 1) / kTV;
        int done = 0;
        while (done < batch) {
            const int nb = (batch - done) < 65535 ? (batch - done) : 65535;
            const size_t off = static_cast<size_t>(done) * R * C;
            transpose_batched_vec_kernel<<<dim3(tr * tc, nb), kBlock, 0, stream()>>>(dst + off, src + off, bias, R, C, tr);
            done += nb;
        }
        return launch_rc();
    }
    const unsigned tiles_r = (R + kT - 1) / kT, tiles_c = (C + kT - 1) / kT;
    int done = 0;
    while (done < batch) {
        const int nb = (batch - done) < 65535 ? (batch - done) : 65535;
        const size_t off = static_cast<size_t>(done) * R * C;
        dim3 grid(tiles_r * tiles_c, nb);
        transpose_batched_kernel<<<grid, kT * 8, 0, stream()>>>(dst + off, src + off, bias, R, C, tiles_r);
        done += nb;
    }
    return launch_rc();
}

// ── row-tiled forms for the layer-sized problems ─────────────────────────
// The two kernels above are gather-bound: a thread's reads jump by a column
// (K floats) or a channel plane between neighbours.  The row forms move a
// strip of the image (or of the patch matrix) through LDS so that both the
// HBM reads and the HBM writes are contiguous runs.
constexpr int kPatchChunk = 256;   // k values per workgroup of im2col_rows: one float4 per lane

// Workgroup order of the scatter row kernel.  Work items are (x, yz): x the
// channel chunk, yz = row strip + strips*sample.  Workgroups are dealt round-robin to the 8
// XCDs, so a 1-D grid of 8*per*gx is launched and XCD q takes yz in
// [q*per, (q+1)*per), walking x fastest: the chunks of one strip, which read
// neighbouring pieces of the same cache lines, and the strips above and below,
// which share halo rows, run at the same time on the same L2.
struct RowGrid {
    int gx, gy, nyz, per;
    unsigned blocks() const { return 8u * static_cast<unsigned>(per) * static_cast<unsigned>(gx); }
};
RowGrid make_rowgrid(int gx, int gy, int gz) {
    RowGrid r;
    r.gx = gx; r.gy = gy; r.nyz = gy * gz;
    r.per = (r.nyz + 7) / 8;
    return r;
}
// false: this workgroup is padding of the last XCD's range
__device__ __forceinline__ bool rowgrid_item(const RowGrid& rg, int& x, int& y, int& z) {
    const unsigned id = blockIdx.x;
    const unsigned xcd = id % 8u, j = id / 8u;
    x = static_cast<int>(j % static_cast<unsigned>(rg.gx));
    const int yz = static_cast<int>(xcd) * rg.per + static_cast<int>(j / static_cast<unsigned>(rg.gx));
    if (yz >= rg.nyz) return false;
    y = yz % rg.gy;
    z = yz / rg.gy;
    return true;
}

// One workgroup = a band of `band` rows of the patch grid, one sample n, one chunk of 256
// consecutive k.  The image rows that chunk touches over the band (its channels x
// (band-1)*stride + kH rows, zero-filled where the window hangs over the border) are
// staged in LDS once; then every wave writes whole 1 KB pieces of patch columns: lane l
// owns k = k0+4l..k0+4l+3 for all positions, so its four LDS offsets are computed once.
// (With one patch row per workgroup every image row was staged kH times over: 203 MB
// fetched for a 67 MB input at 3x3; a band of four rows stages it 1.5 times: 145 -> 140 us
// for the 671 MB of patches of 128 x 128 x 32 x 32, which the write side bounds.)
template <int NSUB, bool NT>
__global__ __launch_bounds__(kBlock) void im2col_rows_kernel(const float* __restrict__ img,
                                                             float* __restrict__ col, PatchGeom g,
                                                             int WT, FastDiv dWT, int band, int nr, FastDiv dnr) {
    extern __shared__ float tile[];   // [channels of the chunk][nr][WT]
    const int KK = g.kH * g.kW;
    // (plain dispatch order, chunks of one band spread over the XCDs: the
    // kernel is write-dominated and this order measured faster than the
    // XCD-grouped one the scatter kernel uses)
    // one 256-wide piece per workgroup; with NSUB = 2 the last workgroup also takes
    // the short remainder that would otherwise leave a workgroup mostly idle
    const int k0 = blockIdx.x * kPatchChunk;
    const int k1 = (NSUB == 2 && blockIdx.x == gridDim.x - 1) ? g.K
                                                                : ((k0 + kPatchChunk) < g.K ? (k0 + kPatchChunk) : g.K);
    const int ph0 = blockIdx.y * band, n = blockIdx.z;
    const int c_lo = fdiv(static_cast<uint32_t>(k0), g.dKK);
    const int c_hi = fdiv(static_cast<uint32_t>(k1 - 1), g.dKK);
    const int rows = (c_hi - c_lo + 1) * nr;
    const int h0 = ph0 * g.stride_h - g.pad_h;
    const float* src = img + static_cast<size_t>(n) * (g.C * g.H * g.W) + static_cast<size_t>(c_lo) * g.H * g.W;
    // (eight independent loads in flight per thread, then their LDS stores)
    constexpr int kBatch = 8;
    for (int idx0 = threadIdx.x; idx0 < rows * WT; idx0 += kBlock * kBatch) {
        float v[kBatch];
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int idx = idx0 + b * kBlock;
            v[b] = 0.0f;
            if (idx < rows * WT) {
                const uint32_t r = fdiv(static_cast<uint32_t>(idx), dWT);
                const int w = idx - static_cast<int>(r) * WT;
                const uint32_t chl = fdiv(r, dnr);
                const int rr = static_cast<int>(r - chl * nr);
                const int ih = h0 + rr, iw = w - g.pad_w;
                if (ih >= 0 && ih < g.H && iw >= 0 && iw < g.W)
                    v[b] = src[(static_cast<size_t>(chl) * g.H + ih) * g.W + iw];
            }
        }
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int idx = idx0 + b * kBlock;
            if (idx < rows * WT) tile[idx] = v[b];
        }
    }
    __syncthreads();
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    // lane l owns k = k0 + 256*u + 4l .. +3 of every 256-wide piece u
    int off[NSUB][4];
#pragma unroll
    for (int u = 0; u < NSUB; ++u) {
        const int kq = k0 + u * kPatchChunk + 4 * lane;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            off[u][j] = -1;
            if (kq < k1) {
                const uint32_t k = static_cast<uint32_t>(kq + j);
                const uint32_t ch = fdiv(k, g.dKK);
                const uint32_t rem = k - ch * KK;
                const uint32_t kh = fdiv(rem, g.dkW);
                const uint32_t kw = rem - kh * g.kW;
                off[u][j] = static_cast<int>(((ch - c_lo) * nr + kh) * WT + kw);
            }
        }
    }
    // the band's positions (row p of the band, column pw) dealt to the waves in turn
    const int band_rows = (ph0 + band) <= g.Hp ? band : g.Hp - ph0;
    float* dst = col + (static_cast<size_t>(n) * g.P + static_cast<size_t>(ph0) * g.Wp) * g.K + k0 + 4 * lane;
    const int positions = band_rows * g.Wp;
    int p = 0, pw = wave;
    while (pw >= g.Wp) { pw -= g.Wp; ++p; }
    for (int pos = wave; pos < positions; pos += kBlock / kWave) {
        const int w = p * g.stride_h * WT + pw * g.stride_w;
        float* d = dst + static_cast<size_t>(pos) * g.K;
#pragma unroll
        for (int u = 0; u < NSUB; ++u) {
            if (off[u][0] >= 0) {
                const float4 v = make_float4(tile[off[u][0] + w], tile[off[u][1] + w], tile[off[u][2] + w],
                                             tile[off[u][3] + w]);
                store4<NT>(d + u * kPatchChunk, v);
            }
        }
        pw += kBlock / kWave;
        while (pw >= g.Wp) { pw -= g.Wp; ++p; }
    }
}

// One workgroup = R image rows of CC channels of one sample.  The patch-matrix
// entries those rows collect (the k range of the CC channels, for every pw of
// the ph rows involved) are staged in LDS with contiguous reads; the sums are
// then formed in the CPU's order (kh, kw descending) out of LDS and written as
// whole image rows.  The pitch is odd so that lanes walking along pw hit
// distinct banks.  S, KH, KW > 0 fix stride (both directions) and kernel extent
// at compile time: the collection loop is index arithmetic per tap, and with
// them known the divisions become shifts and the nine or sixteen taps unroll.
template <int S, int KH, int KW>
__global__ __launch_bounds__(kBlock) void col2im_rows_kernel(const float* __restrict__ col,
                                                             float* __restrict__ img,
                                                             const float* __restrict__ bias, PatchGeom g,
                                                             int CC, int R, int pitch, int vec4, FastDiv dL,
                                                             FastDiv dR, FastDiv dsh, FastDiv dsw, RowGrid rg) {
    extern __shared__ float tile[];   // [ph rows][Wp][pitch]
    const int KK = g.kH * g.kW;
    // (the launcher picks CC dividing C and R dividing H, so every workgroup is full)
    int bx, by, n;
    if (!rowgrid_item(rg, bx, by, n)) return;
    const int c0 = bx * CC;
    const int cc = CC;
    const int ih0 = by * R;
    const int rcnt = R;
    // patch rows with ph*stride - pad + kh inside [ih0, ih0 + rcnt)
    int lo = ih0 + g.pad_h - (g.kH - 1);
    lo = lo <= 0 ? 0 : (lo + g.stride_h - 1) / g.stride_h;
    int hi = (ih0 + rcnt - 1 + g.pad_h) / g.stride_h;
    if (hi > g.Hp - 1) hi = g.Hp - 1;
    const int NR = hi - lo + 1;   // may be <= 0: nothing to collect
    const int L = cc * KK;        // contiguous floats per patch column
    if (NR > 0) {
        const size_t col0 = static_cast<size_t>(n) * g.P + static_cast<size_t>(lo) * g.Wp;
        const int ncols = NR * g.Wp;
        const float* base = col + col0 * g.K + static_cast<size_t>(c0) * KK;
        // four independent loads in flight per thread, then their LDS stores (eight
        // cost more in registers, hence resident workgroups, than they hide);
        // float4 loads when the runs are 16-byte aligned (L and K multiples of 4)
        constexpr int kBatch = 4;
        if (vec4) {
            const int L4 = L / 4;
            const int count = ncols * L4;
            for (int idx0 = threadIdx.x; idx0 < count; idx0 += kBlock * kBatch) {
                float4 v[kBatch];
                int dst[kBatch];
#pragma unroll
                for (int b = 0; b < kBatch; ++b) {
                    const int idx = idx0 + b * kBlock;
                    dst[b] = -1;
                    if (idx < count) {
                        const int cidx = static_cast<int>(fdiv(static_cast<uint32_t>(idx), dL));   // dL divides by L/4 here
                        const int kk = (idx - cidx * L4) * 4;
                        dst[b] = cidx * pitch + kk;
                        v[b] = *reinterpret_cast<const float4*>(base + static_cast<size_t>(cidx) * g.K + kk);
                    }
                }
#pragma unroll
                for (int b = 0; b < kBatch; ++b)
                    if (dst[b] >= 0) {
                        float* d = tile + dst[b];
                        d[0] = v[b].x; d[1] = v[b].y; d[2] = v[b].z; d[3] = v[b].w;
                    }
            }
        } else {
            const int count = ncols * L;
            for (int idx0 = threadIdx.x; idx0 < count; idx0 += kBlock * kBatch) {
                float v[kBatch];
                int dst[kBatch];
#pragma unroll
                for (int b = 0; b < kBatch; ++b) {
                    const int idx = idx0 + b * kBlock;
                    dst[b] = -1;
                    if (idx < count) {
                        const int cidx = static_cast<int>(fdiv(static_cast<uint32_t>(idx), dL));
                        const int kk = idx - cidx * L;
                        dst[b] = cidx * pitch + kk;
                        v[b] = base[static_cast<size_t>(cidx) * g.K + kk];
                    }
                }
#pragma unroll
                for (int b = 0; b < kBatch; ++b)
                    if (dst[b] >= 0) tile[dst[b]] = v[b];
            }
        }
    }
    __syncthreads();
    const int total = cc * rcnt * g.W;
    for (int idx = threadIdx.x; idx < total; idx += kBlock) {
        const uint32_t t = fdiv(static_cast<uint32_t>(idx), g.dW);
        const int iw = idx - static_cast<int>(t) * g.W;
        const int cl = static_cast<int>(fdiv(t, dR));
        const int ih = ih0 + (static_cast<int>(t) - cl * rcnt);
        float val = bias ? bias[c0 + cl] : 0.0f;
        if constexpr (S > 0) {
            // Only every S-th kernel row/column can reach this pixel (ih + pad - kh
            // must be a multiple of S): start at the largest such kh, kw and step by
            // S, the patch index going up by one each time; TH x TW taps instead of
            // KH x KW, in the same descending (kh, kw) order.
            constexpr int TH = (KH + S - 1) / S, TW = (KW + S - 1) / S;
            const int hq = ih + g.pad_h, wq = iw + g.pad_w;
            const int kh1 = (KH - 1) - ((KH - 1 - hq % S) + S) % S;   // may be negative: no tap then
            const int kw1 = (KW - 1) - ((KW - 1 - wq % S) + S) % S;
            const int ph1 = (hq - kh1) / S, pw1 = (wq - kw1) / S;      // exact divisions
            const float* p0 = tile + cl * (KH * KW) + ((ph1 - lo) * g.Wp + pw1) * pitch + kh1 * KW + kw1;
#pragma unroll
            for (int a = 0; a < TH; ++a) {
                const int kh = kh1 - a * S, ph = ph1 + a;
                const bool okh = kh >= 0 && ph >= 0 && ph < g.Hp;
                const float* row = p0 + a * (g.Wp * pitch - S * KW);
#pragma unroll
                for (int b = 0; b < TW; ++b) {
                    const int kw = kw1 - b * S, pw = pw1 + b;
                    if (okh && kw >= 0 && pw >= 0 && pw < g.Wp) val += row[b * (pitch - S)];
                }
            }
        } else {
            for (int kh = g.kH - 1; kh >= 0; --kh) {
                const int hn = ih + g.pad_h - kh;
                if (hn < 0) continue;
                const int ph = static_cast<int>(fdiv(static_cast<uint32_t>(hn), dsh));
                if (ph * g.stride_h != hn || ph >= g.Hp) continue;
                const float* row = tile + static_cast<size_t>(ph - lo) * g.Wp * pitch + cl * KK + kh * g.kW;
                for (int kw = g.kW - 1; kw >= 0; --kw) {
                    const int wn = iw + g.pad_w - kw;
                    if (wn < 0) continue;
                    const int pw = static_cast<int>(fdiv(static_cast<uint32_t>(wn), dsw));
                    if (pw * g.stride_w != wn || pw >= g.Wp) continue;
                    val += row[pw * pitch + kw];
                }
            }
        }
        img[static_cast<size_t>(n) * (g.C * g.H * g.W) + (static_cast<size_t>(c0 + cl) * g.H + ih) * g.W + iw] = val;
    }
}

// The streamed form of the kernel above for the fixed-geometry cases: one workgroup = CC
// channels of one sample over `seg` image rows, walking down the patch rows that feed them.
// A ring of TH + 1 patch rows lives in LDS (TH = the patch rows one image row collects
// from).  The first four waves only load: kStreamDepth patch rows are in flight in their
// registers and the oldest enters the ring slot nothing reads; the other four waves sum and
// write the image rows that the newest staged patch row completes.  One barrier per patch
// row joins the two.  (Loads and image stores in one instruction stream share the memory
// counter, and with stores of unknown count between a load and its use the compiler waits
// for everything outstanding: the prefetch then hides nothing.)  Every patch row is fetched
// once per segment, in runs of CC*KH*KW floats; the strip form fetches kH - 1 halo rows for
// every R image rows, 1.5 times the patch matrix at 3x3 with R = 4.
constexpr int kStreamLoads = 4;   // float4 loads per loading thread per patch row
constexpr int kStreamDepth = 2;   // patch rows in flight ahead of the ring
constexpr int kStreamBlock = 2 * kBlock;
constexpr int kStreamOutputs = 4; // (channel, column) pairs per summing thread
template <int S, int KH, int KW>
__global__ __launch_bounds__(kStreamBlock, 8) void col2im_stream_kernel(const float* __restrict__ col,
                                                                        float* __restrict__ img,
                                                                        const float* __restrict__ bias,
                                                                        PatchGeom g, int CC, int seg, int pitch,
                                                                        FastDiv dL4, RowGrid rg) {
    static_assert(KH >= S && KW >= S, "every image row must be reached by some patch row");
    constexpr int TH = (KH + S - 1) / S, TW = (KW + S - 1) / S, RING = TH + 1, KK = KH * KW;
    extern __shared__ float tile[];   // [RING][Wp][pitch], then the bias of the CC channels
    int bx, by, n;
    if (!rowgrid_item(rg, bx, by, n)) return;
    const int c0 = bx * CC;
    const int r0 = by * seg;
    const int r1 = (r0 + seg < g.H ? r0 + seg : g.H) - 1;   // last image row of the segment
    // patch rows with ph*S - pad + kh inside [r0, r1]
    int lo = r0 + g.pad_h - (KH - 1);
    lo = lo <= 0 ? 0 : (lo + S - 1) / S;
    int hi = (r1 + g.pad_h) / S;
    if (hi > g.Hp - 1) hi = g.Hp - 1;
    const int slot = g.Wp * pitch;
    float* bias_l = tile + RING * slot;

    if (threadIdx.x < kBlock) {
        // ── loading waves ──
        const int L4 = CC * KK / 4;          // float4 per patch column of this chunk
        const int count = g.Wp * L4;         // float4 per patch row (<= kStreamLoads * kBlock)
        const float* base = col + static_cast<size_t>(n) * g.P * g.K + static_cast<size_t>(c0) * KK;
        const size_t row_step = static_cast<size_t>(g.Wp) * g.K;
        // Every thread issues all its loads on every patch row (those past the end of the
        // row re-read its first float4), so no branch depends on the lane.
        int src[kStreamLoads], dst[kStreamLoads];
#pragma unroll
        for (int b = 0; b < kStreamLoads; ++b) {
            const int idx = threadIdx.x + b * kBlock;
            src[b] = 0;
            dst[b] = -1;
            if (idx < count) {
                const int cidx = static_cast<int>(fdiv(static_cast<uint32_t>(idx), dL4));
                const int kk = (idx - cidx * L4) * 4;
                src[b] = cidx * g.K + kk;     // < K*P*N < 2^31
                dst[b] = cidx * pitch + kk;
            }
        }
        if (hi < lo) {
            __syncthreads();
            return;
        }
        float4 v[kStreamDepth][kStreamLoads];
        auto fetch = [&](int ph, float4 (&r)[kStreamLoads]) {
            const float* rowp = base + static_cast<size_t>(ph) * row_step;
#pragma unroll
            // (plain loads: with the streaming hint the 604 MB layer ran 160 us instead of 144)
            for (int b = 0; b < kStreamLoads; ++b) r[b] = *reinterpret_cast<const float4*>(rowp + src[b]);
        };
        auto stash = [&](int ph, const float4 (&r)[kStreamLoads]) {
            float* sl = tile + (ph % RING) * slot;
#pragma unroll
            for (int b = 0; b < kStreamLoads; ++b)
                if (dst[b] >= 0) {
                    float* d = sl + dst[b];
                    d[0] = r[b].x; d[1] = r[b].y; d[2] = r[b].z; d[3] = r[b].w;
                }
        };
        // Register set u holds patch row lo + u (+ a multiple of the depth); a set is refilled
        // as soon as its row is in the ring.  Rows past the last one are clamped to it and the
        // loop body has no branch around a load, so the compiler knows how many younger loads
        // are outstanding when a set enters the ring and waits for that set only.  (The
        // clamped rows land in slots nothing reads any more.)
        auto clamped = [&](int ph) { return ph < hi ? ph : hi; };
#pragma unroll
        for (int u = 0; u < kStreamDepth; ++u) fetch(clamped(lo + u), v[u]);
        stash(lo, v[0]);
        fetch(clamped(lo + kStreamDepth), v[0]);
        __syncthreads();
        for (int ph0 = lo; ph0 <= hi; ph0 += kStreamDepth) {
#pragma unroll
            for (int u = 0; u < kStreamDepth; ++u) {
                const int ph = ph0 + u;   // the row the other waves are working from
                stash(ph + 1, v[(u + 1) % kStreamDepth]);
                fetch(clamped(ph + 1 + kStreamDepth), v[(u + 1) % kStreamDepth]);
                if (ph <= hi) __syncthreads();
            }
        }
        return;
    }

    // ── summing waves ──
    // A thread owns up to kStreamOutputs (channel, column) pairs for the whole walk: what
    // depends on them (bias, which kw reach the column, LDS and image offsets) is worked out
    // once, and a step is the taps' LDS reads, the adds in the CPU's order (kh, kw descending)
    // and one store per pair; what depends on the image row is the same for the whole wave.
    const int tid = threadIdx.x - kBlock;
    if (tid < CC) bias_l[tid] = bias ? bias[c0 + tid] : 0.0f;
    const int per_row = CC * g.W;     // <= kStreamOutputs * kBlock
    int woff[kStreamOutputs], ioff[kStreamOutputs];
    unsigned taps[kStreamOutputs];    // bit b: tap kw1 - b*S exists and its patch column is inside
    float init[kStreamOutputs];
#pragma unroll
    for (int j = 0; j < kStreamOutputs; ++j) {
        const int idx = tid + j * kBlock;
        woff[j] = 0; ioff[j] = -1; taps[j] = 0; init[j] = 0.0f;
        if (idx < per_row) {
            const int cl = static_cast<int>(fdiv(static_cast<uint32_t>(idx), g.dW));
            const int iw = idx - cl * g.W;
            const int wq = iw + g.pad_w;
            const int kw1 = (KW - 1) - ((KW - 1 - wq % S) + S) % S;   // largest kw that reaches this column
            const int pw1 = (wq - kw1) / S;                           // exact
#pragma unroll
            for (int b = 0; b < TW; ++b) {
                const int kw = kw1 - b * S, pw = pw1 + b;
                if (kw >= 0 && pw >= 0 && pw < g.Wp) taps[j] |= 1u << b;
            }
            woff[j] = cl * KK + kw1 + pw1 * pitch;
            ioff[j] = (c0 + cl) * g.H * g.W + iw;   // < C*H*W*N < 2^31
        }
    }
    __syncthreads();   // first patch row and the bias are in LDS
#pragma unroll
    for (int j = 0; j < kStreamOutputs; ++j)
        if (ioff[j] >= 0) init[j] = bias_l[(ioff[j] / (g.H * g.W)) - c0];
    float* out = img + static_cast<size_t>(n) * (g.C * g.H * g.W);
    // image rows e0..e1, every patch row they collect from staged (or none existing)
    auto emit = [&](int e0, int e1) {
        for (int ih = e0; ih <= e1; ++ih) {
            const int hq = ih + g.pad_h;
            const int kh1 = (KH - 1) - ((KH - 1 - hq % S) + S) % S;   // largest kh that reaches this row; may be negative
            const int ph1 = (hq - kh1) / S;                           // exact
#pragma unroll
            for (int j = 0; j < kStreamOutputs; ++j) {
                if (j * kBlock < per_row) {
                    float val = init[j];
#pragma unroll
                    for (int a = 0; a < TH; ++a) {
                        const int kh = kh1 - a * S, ph = ph1 + a;
                        if (kh >= 0 && ph >= 0 && ph < g.Hp) {
                            const float* row = tile + (ph % RING) * slot + kh * KW + woff[j];
#pragma unroll
                            for (int b = 0; b < TW; ++b)
                                if (taps[j] >> b & 1u) val += row[b * (pitch - S)];
                        }
                    }
                    if (ioff[j] >= 0) out[ioff[j] + ih * g.W] = val;
                }
            }
        }
    };
    if (hi < lo) {     // no patch row reaches this segment
        emit(r0, r1);
        return;
    }
    for (int ph = lo; ph <= hi; ++ph) {
        // the image rows whose last patch row is ph
        int e0 = ph * S - g.pad_h;
        int e1 = ph == hi ? r1 : e0 + S - 1;
        if (e0 < r0) e0 = r0;
        if (e1 > r1) e1 = r1;
        emit(e0, e1);
        __syncthreads();
    }
}

bool geom_ok(int C, int H, int W, int kH, int kW, int pad_h, int pad_w, int stride_h, int stride_w,
             int Hp, int Wp, int N) {
    return C > 0 && H > 0 && W > 0 && kH > 0 && kW > 0 && pad_h >= 0 && pad_w >= 0 && stride_h > 0 &&
           stride_w > 0 && Hp > 0 && Wp > 0 && N > 0;
}

int gather_patches(const float* img, float* col, const PatchGeom& g) {
    const size_t total = static_cast<size_t>(g.K) * g.P * g.N;
    if (total >= (size_t(1) << 31)) return -1;
    if (static_cast<size_t>(g.C) * g.H * g.W * g.N >= (size_t(1) << 31)) return -1;
    if (g.K % 4 == 0 && g.K >= 64 && aligned16(col) && g.N <= 65535 && g.Hp <= 65535) {
        const int WT = (g.Wp - 1) * g.stride_w + g.kW;
        // a last piece of at most 64 k is folded into the workgroup before it (a
        // workgroup of its own would run with a quarter of its lanes; folding a
        // longer remainder costs more in LDS per workgroup than it saves)
        const int pieces = (g.K + kPatchChunk - 1) / kPatchChunk;
        const bool fold = pieces >= 2 && g.K - (pieces - 1) * kPatchChunk <= kPatchChunk / 4;
        const int nch_max = (fold ? kPatchChunk + kPatchChunk / 4 : kPatchChunk) / (g.kH * g.kW) + 2;
        // rows of the patch grid per workgroup: as many (up to four) as keep the staged rows
        // under 48 KB and leave 16 workgroups per CU to hide the staging phase (with fewer the
        // saved re-reads cost more in idle time: 30 us against 24 us at 128 x 64 x 32 x 32, stride 2)
        int band = 4;
        auto staged_rows = [&](int bd) { return (bd - 1) * g.stride_h + g.kH; };
        auto lds_bytes = [&](int bd) { return static_cast<size_t>(nch_max) * staged_rows(bd) * WT * sizeof(float); };
        auto groups = [&](int bd) {
            return static_cast<size_t>(fold ? pieces - 1 : pieces) * ((g.Hp + bd - 1) / bd) * g.N;
        };
        while (band > 1 && (lds_bytes(band) > 48 * 1024 || band > g.Hp || groups(band) < 4096)) band /= 2;
        const size_t lds = lds_bytes(band);
        const int bands = (g.Hp + band - 1) / band;
        if (lds <= 48 * 1024) {
            dim3 grid(fold ? pieces - 1 : pieces, bands, g.N);
            const int nr = staged_rows(band);
            const FastDiv dWT = make_fastdiv(WT), dnr = make_fastdiv(nr);
            const bool nt = streams_past_cache(total * sizeof(float));   // patches that the cache cannot hold anyway
            if (fold && nt) im2col_rows_kernel<2, true><<<grid, kBlock, lds, stream()>>>(img, col, g, WT, dWT, band, nr, dnr);
            else if (fold) im2col_rows_kernel<2, false><<<grid, kBlock, lds, stream()>>>(img, col, g, WT, dWT, band, nr, dnr);
            else if (nt) im2col_rows_kernel<1, true><<<grid, kBlock, lds, stream()>>>(img, col, g, WT, dWT, band, nr, dnr);
            else im2col_rows_kernel<1, false><<<grid, kBlock, lds, stream()>>>(img, col, g, WT, dWT, band, nr, dnr);
            return launch_rc();
        }
    }
    if (g.K % 4 == 0 && aligned16(col)) {
        const size_t tv = total / 4;
        im2col_kernel<4><<<grid_cover(tv, kBlock), kBlock, 0, stream()>>>(img, col, g, make_fastdiv(g.K / 4), tv);
    } else {
        im2col_kernel<1><<<grid_cover(total, kBlock), kBlock, 0, stream()>>>(img, col, g, g.dK, total);
    }
    return launch_rc();
}

int scatter_patches(const float* col, float* img, const float* bias, const PatchGeom& g) {
    const size_t total = static_cast<size_t>(g.C) * g.H * g.W * g.N;
    if (total >= (size_t(1) << 31)) return -1;
    if (static_cast<size_t>(g.K) * g.P * g.N >= (size_t(1) << 31)) return -1;
    // streamed form: fixed geometry, float4 runs, one patch row of the chunk within
    // kStreamLoads loads per thread and the ring within 40 KB (four workgroups per CU)
    {
        const int KK = g.kH * g.kW;
        const int S = g.stride_h == g.stride_w ? g.stride_h : 0;
        const int form = (S == 1 && g.kH == 3 && g.kW == 3) ? 1 : (S == 2 && g.kH == 3 && g.kW == 3) ? 2
                       : (S == 2 && g.kH == 4 && g.kW == 4) ? 3 : (S == 1 && g.kH == 5 && g.kW == 5) ? 4 : 0;
        const int ring = form ? (g.kH + S - 1) / S + 1 : 0;
        auto fits = [&](int cc) {
            return g.C % cc == 0 && (cc * KK) % 4 == 0 && g.Wp * (cc * KK / 4) <= kStreamLoads * kBlock &&
                   cc * g.W <= kStreamOutputs * kBlock &&
                   static_cast<size_t>(ring) * g.Wp * ((cc * KK) | 1) * sizeof(float) <= 40 * 1024;
        };
        int CC = 16;
        while (CC > 1 && !fits(CC)) CC /= 2;
        // (below 64 MB of patches the strip form is as fast alone and its 256-thread
        // workgroups start sooner behind another kernel: a 29 MB layer ran 3.5 us
        // slower inside a training step with the streamed form)
        const bool large = static_cast<size_t>(g.K) * g.P * g.N * sizeof(float) >= (size_t(64) << 20);
        if (form && large && fits(CC) && g.K % 4 == 0 && aligned16(col)) {
            // whole images per workgroup unless that leaves fewer than 2048 workgroups:
            // then segments of rows, each paying kH - 1 halo patch rows
            int seg = g.H;
            auto groups = [&](int sg) { return static_cast<size_t>(g.C / CC) * ((g.H + sg - 1) / sg) * g.N; };
            while (seg > 8 && groups(seg) < 2048) seg = (seg + 1) / 2;
            const RowGrid rg = make_rowgrid(g.C / CC, (g.H + seg - 1) / seg, g.N);
            const int pitch = (CC * KK) | 1;
            const size_t lds = (static_cast<size_t>(ring) * g.Wp * pitch + CC) * sizeof(float);
            const FastDiv dL4 = make_fastdiv(CC * KK / 4);
#define JZ_COL2IM_STREAM(S_, KH_, KW_)                                                                       \
    col2im_stream_kernel<S_, KH_, KW_><<<rg.blocks(), kStreamBlock, lds, stream()>>>(col, img, bias, g, CC, seg,  \
                                                                               pitch, dL4, rg)
            if (form == 1) JZ_COL2IM_STREAM(1, 3, 3);
            else if (form == 2) JZ_COL2IM_STREAM(2, 3, 3);
            else if (form == 3) JZ_COL2IM_STREAM(2, 4, 4);
            else JZ_COL2IM_STREAM(1, 5, 5);
#undef JZ_COL2IM_STREAM
            return launch_rc();
        }
    }
    if (g.W <= 1024) {
        // channels and image rows per workgroup: as many as keep the staged strip
        // under 40 KB (four workgroups per CU), preferring a channel-chunk count
        // that is a multiple of 8 so that the workgroups sharing patch rows
        // (same chunk, neighbouring rows) meet in one XCD's L2
        const int KK = g.kH * g.kW;
        // (four rows at stride 1, where neighbouring strips share two of six
        // patch rows; two at larger strides, where the smaller strip measured faster)
        int R = g.stride_h >= 2 ? 2 : 4, CC = 16;
        auto bytes = [&](int cc, int r) {
            const int nr = (r - 1 + g.kH - 1) / g.stride_h + 1;
            return static_cast<size_t>(nr) * g.Wp * ((cc * KK) | 1) * sizeof(float);
        };
        while (R > 1 && g.H % R != 0) R /= 2;
        while (CC > 1 && (g.C % CC != 0 || bytes(CC, R) > 40 * 1024)) CC /= 2;
        while (R > 1 && bytes(CC, R) > 40 * 1024) R /= 2;
        if (bytes(CC, R) <= 40 * 1024) {
            // (C/CC * H/R * N <= C*H*W*N < 2^31 workgroups)
            const RowGrid rg = make_rowgrid(g.C / CC, g.H / R, g.N);
            const unsigned grid = rg.blocks();
            const int vec4 = ((CC * KK) % 4 == 0 && g.K % 4 == 0 && aligned16(col)) ? 1 : 0;
            const int S = g.stride_h == g.stride_w ? g.stride_h : 0;
#define JZ_COL2IM(S_, KH_, KW_)                                                                              \
    col2im_rows_kernel<S_, KH_, KW_><<<grid, kBlock, bytes(CC, R), stream()>>>(                              \
        col, img, bias, g, CC, R, (CC * KK) | 1, vec4, make_fastdiv(vec4 ? CC * KK / 4 : CC * KK), make_fastdiv(R), \
        make_fastdiv(g.stride_h), make_fastdiv(g.stride_w), rg)
            if (S == 1 && g.kH == 3 && g.kW == 3) JZ_COL2IM(1, 3, 3);
            else if (S == 2 && g.kH == 3 && g.kW == 3) JZ_COL2IM(2, 3, 3);
            else if (S == 2 && g.kH == 4 && g.kW == 4) JZ_COL2IM(2, 4, 4);
            else if (S == 1 && g.kH == 5 && g.kW == 5) JZ_COL2IM(1, 5, 5);
            else JZ_COL2IM(0, 1, 1);
#undef JZ_COL2IM
            return launch_rc();
        }
    }
    col2im_kernel<<<grid_cover(total, kBlock), kBlock, 0, stream()>>>(col, img, bias, g, total);
    return launch_rc();
}

}  // namespace
}  // namespace jz

using namespace jz;

JZ_API int jzhip_im2col(const float* input, float* col, int C_in, int H_in, int W_in, int kH, int kW,
                        int pad_h, int pad_w, int stride_h, int stride_w, int H_out, int W_out,
                        int N) {
    if (!input || !col || !geom_ok(C_in, H_in, W_in, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N))
        return -1;
    return gather_patches(input, col,
                          make_geom(C_in, H_in, W_in, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N));
}

JZ_API int jzhip_col2im(const float* col, float* dx, int C_in, int H_in, int W_in, int kH, int kW,
                        int pad_h, int pad_w, int stride_h, int stride_w, int H_out, int W_out,
                        int N) {
    if (!col || !dx || !geom_ok(C_in, H_in, W_in, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N))
        return -1;
    return scatter_patches(col, dx, nullptr,
                           make_geom(C_in, H_in, W_in, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N));
}

// y2d(C_out, P*N) -> out(C_out*P, N) + bias[co]   (ml/layer.hpp:1959-1973)
JZ_API int jzhip_conv_forward_reshape_bias(const float* y2d, float* out, const float* bias,
                                           int C_out, int P, int N) {
    return transpose_batched(out, y2d, bias, C_out, P, N);
}

// t(C_out*P, N) -> t2d(C_out, P*N)   (ml/layer.hpp:1942-1957)
JZ_API int jzhip_conv_backward_reshape(const float* t, float* t2d, int C_out, int P, int N) {
    return transpose_batched(t2d, t, nullptr, P, C_out, N);
}

// Transposed convolution: the output image grid (H_out x W_out) is the image
// side and the input grid (H_in x W_in) is the patch side of the same maps
// (oh = ih*stride - pad + kh, ml/layer.hpp:2159-2171,2190-2202).
JZ_API int jzhip_convtrans_scatter(const float* patches, float* out, const float* bias, int C_out,
                                   int H_out, int W_out, int H_in, int W_in, int kH, int kW,
                                   int pad_h, int pad_w, int stride_h, int stride_w, int N) {
    if (!patches || !out || !bias ||
        !geom_ok(C_out, H_out, W_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_in, W_in, N))
        return -1;
    return scatter_patches(patches, out, bias,
                           make_geom(C_out, H_out, W_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_in, W_in, N));
}

JZ_API int jzhip_convtrans_gather(const float* t, float* tp, int C_out, int H_out, int W_out,
                                  int H_in, int W_in, int kH, int kW, int pad_h, int pad_w,
                                  int stride_h, int stride_w, int N) {
    if (!t || !tp || !geom_ok(C_out, H_out, W_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_in, W_in, N))
        return -1;
    return gather_patches(t, tp,
                          make_geom(C_out, H_out, W_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_in, W_in, N));
}

// direction 0: (C*spatial, N) -> (C, spatial*N); direction 1: the inverse
// (ml/layer.hpp:2112-2126,2206-2221).
JZ_API int jzhip_convtrans_reshape(const float* src, float* dst, int C, int spatial, int N,
                                   int direction) {
    if (direction == 0) return transpose_batched(dst, src, nullptr, spatial, C, N);
    if (direction == 1) return transpose_batched(dst, src, nullptr, C, spatial, N);
    return -1;
}
