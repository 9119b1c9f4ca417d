// 3x3, stride-1, pad-1 convolutions with at most four input channels (the first layer of a
// network: a grey or RGB image): forward and weight gradients of ConvLayer
// (ml/layer.hpp:1611-1637, 1679-1696) as plain vector kernels.  With K = C_in*9 <= 36 patch rows
// an MFMA tile of 128 patch rows is mostly padding; the products are bound by writing the
// output (forward) or reading the upstream gradient (weight gradients) once.
//
// A thread owns four consecutive pixels of an image row and keeps their patch window (three
// rows of six columns per channel) in registers.  Forward: for each output channel of the
// workgroup's group the K weights come out of LDS as broadcasts, K x 4 multiply-adds, one
// float4 store.  Weight gradients: for each output channel one float4 of the upstream gradient
// is multiplied into the K patch rows; the sums are added over the wavefront (many values at
// once by halving exchanges), over the workgroup through LDS and over workgroups by the
// split-K reduction from the workspace, always in the same order.
#include "common.hpp"

namespace jz {
void launch_splitk_reduce(float* C, const float* part, int M, int N, size_t ldc, int splits, float alpha,
                          float beta);
namespace {

constexpr int kFewPixels = 4 * kBlock;   // pixels per workgroup pass

// the patch window of four pixels (oh, ow .. ow + 3) of image n: win[c][ky][j] = x(c, oh + ky - 1, ow + j - 1) or 0
template <int CIN>
__device__ __forceinline__ void load_window(float (&win)[CIN][3][6], const float* __restrict__ x, int n, int oh, int ow,
                                            int H, int W) {
    const float* img = x + static_cast<long long>(n) * CIN * H * W;
#pragma unroll
    for (int c = 0; c < CIN; ++c)
#pragma unroll
        for (int ky = 0; ky < 3; ++ky) {
            const int ih = oh + ky - 1;
            const bool row = static_cast<unsigned>(ih) < static_cast<unsigned>(H);
            const float* r = img + (c * H + (row ? ih : 0)) * W + ow;   // ow % 4 == 0, W % 4 == 0: the middle four are one float4
            const float4 mid = row ? *reinterpret_cast<const float4*>(r) : make_float4(0.f, 0.f, 0.f, 0.f);
            win[c][ky][0] = (row && ow > 0) ? r[-1] : 0.0f;
            win[c][ky][1] = mid.x; win[c][ky][2] = mid.y; win[c][ky][3] = mid.z; win[c][ky][4] = mid.w;
            win[c][ky][5] = (row && ow + 4 < W) ? r[4] : 0.0f;
        }
}

// weights of the workgroup's output channels in LDS: ws[g * KP + k], KP = K rounded up to four (so that four
// weights come out as one read), the biases behind them
template <int CIN>
__global__ __launch_bounds__(kBlock) void conv_few_fwd_kernel(const float* __restrict__ x, const float* __restrict__ Wt,
                                                              const float* __restrict__ bias, float* __restrict__ out,
                                                              int H, int W, int Cout, int co_per_wg, long long quads,
                                                              int relu) {
    constexpr int K = CIN * 9, KP = (K + 3) / 4 * 4;
    extern __shared__ __align__(16) float ws[];
    const int co0 = blockIdx.y * co_per_wg;
    const int cg = Cout - co0 < co_per_wg ? Cout - co0 : co_per_wg;
    for (int i = threadIdx.x; i < cg * KP; i += kBlock) {
        const int g = i / KP, k = i - g * KP;
        ws[i] = k < K ? Wt[static_cast<long long>(co0 + g) * K + k] : 0.0f;
    }
    for (int i = threadIdx.x; i < cg; i += kBlock) ws[co_per_wg * KP + i] = bias ? bias[co0 + i] : 0.0f;
    __syncthreads();
    const long long q = static_cast<long long>(blockIdx.x) * kBlock + threadIdx.x;   // pixel quad
    if (q >= quads) return;
    const int W4 = W / 4, P = H * W;
    const int n = static_cast<int>(q / (H * W4));
    const int r = static_cast<int>(q - static_cast<long long>(n) * (H * W4));
    const int oh = r / W4, ow = (r - oh * W4) * 4;
    float win[CIN][3][6];
    load_window<CIN>(win, x, n, oh, ow, H, W);
    float* dst = out + (static_cast<long long>(n) * Cout + co0) * P + oh * W + ow;
    for (int g = 0; g < cg; ++g) {
        const float b = ws[co_per_wg * KP + g];
        float wk[KP];
#pragma unroll
        for (int k = 0; k < KP; k += 4) {
            const float4 w4 = *reinterpret_cast<const float4*>(&ws[g * KP + k]);
            wk[k] = w4.x; wk[k + 1] = w4.y; wk[k + 2] = w4.z; wk[k + 3] = w4.w;
        }
        float4 acc = make_float4(b, b, b, b);
#pragma unroll
        for (int c = 0; c < CIN; ++c)
#pragma unroll
            for (int ky = 0; ky < 3; ++ky)
#pragma unroll
                for (int kx = 0; kx < 3; ++kx) {
                    const float w = wk[(c * 3 + ky) * 3 + kx];
                    acc.x += w * win[c][ky][kx]; acc.y += w * win[c][ky][kx + 1];
                    acc.z += w * win[c][ky][kx + 2]; acc.w += w * win[c][ky][kx + 3];
                }
        if (relu) {
            acc.x = acc.x > 0.f ? acc.x : 0.f; acc.y = acc.y > 0.f ? acc.y : 0.f;
            acc.z = acc.z > 0.f ? acc.z : 0.f; acc.w = acc.w > 0.f ? acc.w : 0.f;
        }
        *reinterpret_cast<float4*>(dst + static_cast<long long>(g) * P) = acc;
    }
}

// sums NV = 16, 32 or 64 values per lane over the wavefront by halving exchanges: afterwards v[0] of lane
// i * (64 / NV) holds the total of value i
template <int N>
__device__ __forceinline__ void few_fold(float* v, int lane, int mask) {
    const bool upper = (lane & mask) != 0;
#pragma unroll
    for (int i = 0; i < N / 2; ++i) {
        const float keep = upper ? v[i + N / 2] : v[i];
        const float send = upper ? v[i] : v[i + N / 2];
        v[i] = keep + __shfl_xor(send, mask, kWave);
    }
}

// part[(chunk * Cout + co) * K + k]: the sums of one workgroup over its pixel quads
template <int CIN, int CG>
__global__ __launch_bounds__(kBlock) void conv_few_dw_kernel(const float* __restrict__ x, const float* __restrict__ t,
                                                             float* __restrict__ part, int H, int W, int Cout,
                                                             long long quads) {
    constexpr int K = CIN * 9;
    constexpr int KP = K <= 16 ? 16 : K <= 32 ? 32 : 64;   // the sums of one output channel, padded to a power of two
    constexpr int NW = kBlock / kWave;
    __shared__ float red[NW][CG][KP];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int co0 = blockIdx.y * CG;
    const int W4 = W / 4, P = H * W;
    float acc[CG][K];
#pragma unroll
    for (int g = 0; g < CG; ++g)
#pragma unroll
        for (int k = 0; k < K; ++k) acc[g][k] = 0.0f;
    for (long long q = static_cast<long long>(blockIdx.x) * kBlock + threadIdx.x; q < quads;
         q += static_cast<long long>(gridDim.x) * kBlock) {
        const int n = static_cast<int>(q / (H * W4));
        const int r = static_cast<int>(q - static_cast<long long>(n) * (H * W4));
        const int oh = r / W4, ow = (r - oh * W4) * 4;
        float win[CIN][3][6];
        load_window<CIN>(win, x, n, oh, ow, H, W);
        const float* tp = t + static_cast<long long>(n) * Cout * P + oh * W + ow;
        float4 tv[CG];
#pragma unroll
        for (int g = 0; g < CG; ++g)
            tv[g] = co0 + g < Cout ? *reinterpret_cast<const float4*>(tp + static_cast<long long>(co0 + g) * P)
                                   : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int g = 0; g < CG; ++g)
#pragma unroll
            for (int c = 0; c < CIN; ++c)
#pragma unroll
                for (int ky = 0; ky < 3; ++ky)
#pragma unroll
                    for (int kx = 0; kx < 3; ++kx)
                        acc[g][(c * 3 + ky) * 3 + kx] += tv[g].x * win[c][ky][kx] + tv[g].y * win[c][ky][kx + 1] +
                                                         tv[g].z * win[c][ky][kx + 2] + tv[g].w * win[c][ky][kx + 3];
    }
    // over the wavefront, one output channel at a time
#pragma unroll
    for (int g = 0; g < CG; ++g) {
        float v[KP];
#pragma unroll
        for (int k = 0; k < KP; ++k) v[k] = k < K ? acc[g][k] : 0.0f;
        int mask = kWave / 2;
        if constexpr (KP >= 64) { few_fold<64>(v, lane, mask); mask >>= 1; }
        if constexpr (KP >= 32) { few_fold<32>(v, lane, mask); mask >>= 1; }
        few_fold<16>(v, lane, mask); mask >>= 1;
        few_fold<8>(v, lane, mask); mask >>= 1;
        few_fold<4>(v, lane, mask); mask >>= 1;
        few_fold<2>(v, lane, mask); mask >>= 1;
        for (int m = mask; m >= 1; m >>= 1) v[0] += __shfl_xor(v[0], m, kWave);
        constexpr int rest = kWave / KP;   // lanes that now hold the same value
        if (lane % rest == 0) red[wave][g][lane / rest] = v[0];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < CG * K; i += kBlock) {
        const int g = i / K, k = i - g * K;
        if (co0 + g < Cout) {
            float s = red[0][g][k];
#pragma unroll
            for (int w = 1; w < NW; ++w) s += red[w][g][k];
            part[(static_cast<long long>(blockIdx.x) * Cout + co0 + g) * K + k] = s;
        }
    }
}

}  // namespace

// Shapes the few-channel kernels take: 3x3, stride 1, padding 1, one to four input channels, rows in
// multiples of four pixels, 16-byte aligned operands.
bool conv_few_ok(const float* x, const float* other, int C, int H, int W, int kH, int kW, int pad_h, int pad_w, int sh,
                 int sw, int Ho, int Wo) {
    return kH == 3 && kW == 3 && pad_h == 1 && pad_w == 1 && sh == 1 && sw == 1 && Ho == H && Wo == W && C >= 1 && C <= 4 &&
           W % 4 == 0 && aligned16(x) && aligned16(other);
}

int launch_conv_few_fwd(const float* x, const float* Wt, const float* bias, float* out, int C, int H, int W, int Cout,
                        int N, int relu) {
    const long long quads = static_cast<long long>(N) * H * (W / 4);
    const long long bx = (quads + kBlock - 1) / kBlock;
    const int KP = (C * 9 + 3) / 4 * 4;
    // output channels per workgroup: all of them when the pixel blocks alone fill the chip (the window is then
    // fetched once), otherwise groups of eight or more so that there are about two workgroups per CU
    const long long want = 2ll * num_cus();
    long long groups = bx >= want ? 1 : (want + bx - 1) / bx;
    int per = static_cast<int>((Cout + groups - 1) / groups);
    per = (per + 7) / 8 * 8;
    const int lds_cap = 32 * 1024 / static_cast<int>(sizeof(float)) / (KP + 1) / 8 * 8;
    if (per > lds_cap) per = lds_cap;
    if (per > Cout) per = Cout;
    const int by = (Cout + per - 1) / per;
    if (bx > 0x7fffffffll || by > 65535) return -1;
    const dim3 grid(static_cast<unsigned>(bx), by);
    const size_t lds = static_cast<size_t>(per) * (KP + 1) * sizeof(float);
    hipStream_t s = stream();
    switch (C) {
        case 1: conv_few_fwd_kernel<1><<<grid, kBlock, lds, s>>>(x, Wt, bias, out, H, W, Cout, per, quads, relu); break;
        case 2: conv_few_fwd_kernel<2><<<grid, kBlock, lds, s>>>(x, Wt, bias, out, H, W, Cout, per, quads, relu); break;
        case 3: conv_few_fwd_kernel<3><<<grid, kBlock, lds, s>>>(x, Wt, bias, out, H, W, Cout, per, quads, relu); break;
        default: conv_few_fwd_kernel<4><<<grid, kBlock, lds, s>>>(x, Wt, bias, out, H, W, Cout, per, quads, relu); break;
    }
    return launch_rc();
}

int launch_conv_few_dw(const float* x, const float* t, float* dW, int C, int H, int W, int Cout, int N) {
    const long long quads = static_cast<long long>(N) * H * (W / 4);
    const int K = C * 9;
    const int CG = C == 1 ? 8 : C == 4 ? 2 : 4;   // K sums per output channel in registers: 72 to 108 per thread
    const int by = (Cout + CG - 1) / CG;
    if (by > 65535) return -1;
    // pixel chunks: channel groups x chunks give every CU a few workgroups; at least one pass of 1024 pixels each
    long long bx = (4ll * num_cus() + by - 1) / by;
    const long long passes = (quads + kBlock - 1) / kBlock;
    if (bx > passes) bx = passes;
    if (bx < 1) bx = 1;
    while (bx > 1 && static_cast<size_t>(bx) * K * Cout > kWorkspaceFloats) --bx;
    if (static_cast<size_t>(bx) * K * Cout > kWorkspaceFloats) return -1;
    float* part = bx > 1 ? workspace() : dW;
    if (!part) return -2;
    const dim3 grid(static_cast<unsigned>(bx), by);
    hipStream_t s = stream();
    switch (C) {
        case 1: conv_few_dw_kernel<1, 8><<<grid, kBlock, 0, s>>>(x, t, part, H, W, Cout, quads); break;
        case 2: conv_few_dw_kernel<2, 4><<<grid, kBlock, 0, s>>>(x, t, part, H, W, Cout, quads); break;
        case 3: conv_few_dw_kernel<3, 4><<<grid, kBlock, 0, s>>>(x, t, part, H, W, Cout, quads); break;
        default: conv_few_dw_kernel<4, 2><<<grid, kBlock, 0, s>>>(x, t, part, H, W, Cout, quads); break;
    }
    if (bx > 1) launch_splitk_reduce(dW, part, K, Cout, static_cast<size_t>(K), static_cast<int>(bx), 1.0f, 0.0f);
    return launch_rc();
}

}  // namespace jz
