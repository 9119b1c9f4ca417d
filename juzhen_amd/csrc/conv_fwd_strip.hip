// Forward product of a 3x3, stride-1, pad-1 convolution from image strips in LDS:
//     out(co, oh, ow; n) = bias(co) + sum over (c, ky, kx) of W((c, ky, kx), co) * x(c, oh + ky - 1, ow + kx - 1; n)   [relu]
// (RocmIm2col + RocmGemm + RocmConvForwardReshapeBias of ConvLayer::eval, ml/layer.hpp:1611-1637;
// with the weights flipped it is also the input gradient of such a layer, :1698-1709).
// The general kernel of conv_gemm.hip builds a patch tile in LDS, one range-checked load per
// patch element.  Here a workgroup stages RT + 2 rows of a few input channels per stage, with a
// zero column on either side and zero rows outside the image, and the patch operand of every
// tap is that strip read at another offset: 32 consecutive pixels are 32 consecutive LDS words,
// so a fragment is one ds_read without any index arithmetic, and a pixel is fetched from memory
// once per stage instead of nine times.  The weights are regrouped beforehand (one small launch,
// or as part of the flip the input-gradient product needs anyway) into the order the stages
// consume: [channel tile][stage][tap][channel pair][parity][output channel], so that a stage's
// weights are one contiguous block copied with 16-byte loads and stores.
//
// Tile: RT rows of one image (64 or 128 pixels) x BN output channels, four waves as two pixel
// halves x two channel halves.  A stage covers 4608 / BN input channels x 9 taps (72 or 36
// steps of the 32x32x2 matrix instruction per wave and pixel block).
#include "common.hpp"
#include "gemm_tile.hpp"

namespace jz {
namespace {

template <int W, int RT, int BN>
struct FwdStrip {
    static constexpr int BMP = W * RT;               // pixels per tile
    static constexpr int PB = BMP / 64;              // 32-pixel blocks per wave
    static constexpr int NB = BN / 64;               // 32-channel blocks per wave
    static constexpr int CB = 512 / BN;              // input channels per stage: 8 or 4
    static constexpr int KSTEPS = 9 * CB / 2;        // matrix-instruction steps per stage
    // Row pitch of the strip.  A fragment reads 32 pixels at once: one row of 32, two rows of 16 or
    // four rows of 8.  With pitch 20 rows four apart, and with pitch 12 rows two apart, start 16
    // (8, 16, 24) banks from each other, so those are the rows a block is made of and its 32 lanes
    // hit 32 banks; consecutive rows at pitch W + 2 would overlap by two banks and take two cycles.
    static constexpr int PITCH = W == 16 ? 20 : W == 8 ? 12 : W + 2;
    static constexpr int ROWS = RT + 2, XCS = ROWS * PITCH;
    static constexpr int XBUF = CB * XCS;
    static constexpr int WBUF = 9 * CB * BN;         // 4608 floats
    static constexpr int XVEC = CB * ROWS * W / 4, XPASS = (XVEC + kBlock - 1) / kBlock;
    static constexpr int WVEC = WBUF / 4, WPASS = (WVEC + kBlock - 1) / kBlock;
    static_assert(BMP == 64 || BMP == 128 || BMP == 256, "a wave takes one, two or four 32-pixel blocks");
    static_assert(32 % W == 0 || W == 32 || W % 32 == 0, "a 32-pixel block is whole rows or part of one");
};

// Packed weights: element ((ct * stages + s) * 9*CB + (tap * CB/2 + m) * 2 + h) * BN + o holds the
// weight of input channel s*CB + 2m + h, tap (ky, kx), output channel ct*BN + o.
// flip = 0: from the layer's stored (K, C_out) matrix, K = C_in*9 (forward product).
// flip = 1: the product's input channels are the layer's output channels and its taps are
//           mirrored (input gradients): W((c = out channel of the product, 2 - ky, 2 - kx), co = in channel).
__global__ __launch_bounds__(kBlock) void conv_strip_pack_kernel(float* __restrict__ packed, const float* __restrict__ Wt,
                                                                 int Cin, int Cout, int BN, int CB, int flip,
                                                                 long long total) {
    const long long e = static_cast<long long>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= total) return;
    const int o = static_cast<int>(e % BN);
    long long r = e / BN;
    const int kk = static_cast<int>(r % (9 * CB));
    r /= 9 * CB;
    const int stages = Cin / CB;
    const int s = static_cast<int>(r % stages), ct = static_cast<int>(r / stages);
    const int h = kk & 1, m = (kk >> 1) % (CB / 2), tap = (kk >> 1) / (CB / 2);
    const int ci = s * CB + 2 * m + h, co = ct * BN + o;
    float v;
    if (!flip) v = Wt[static_cast<long long>(co) * (Cin * 9) + ci * 9 + tap];
    else v = Wt[static_cast<long long>(ci) * (Cout * 9) + co * 9 + (8 - tap)];
    packed[e] = v;
}

template <int W, int RT, int BN>
__global__ __launch_bounds__(kBlock, 2) void conv_fwd_strip_kernel(const float* __restrict__ x,
                                                                   const float* __restrict__ packed,
                                                                   const float* __restrict__ bias,
                                                                   float* __restrict__ out, int C, int H, int Cout,
                                                                   int tiles_co, int relu, unsigned x_bytes) {
    using S = FwdStrip<W, RT, BN>;
    __shared__ __attribute__((aligned(16))) float lds[2 * S::XBUF + 2 * S::WBUF];
    float* const xs = lds + 2 * S::WBUF;   // [2][XBUF]
    float* const ws = lds;                 // [2][WBUF], 16-byte aligned blocks

    // consecutive workgroups share a pixel tile (the same strips) and differ in the channel tile
    const int tile_p = blockIdx.x / tiles_co, ct = blockIdx.x % tiles_co;
    const int per_image = H / RT;
    const int n = tile_p / per_image, oh0 = (tile_p - n * per_image) * RT;
    const int HW = H * W;
    const int stages = C / S::CB;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int wp = wave & 1, wc = wave >> 1;
    const int l32 = lane & 31, h = lane >> 5;

    floatx16 acc[S::PB][S::NB];
#pragma unroll
    for (int a = 0; a < S::PB; ++a)
#pragma unroll
        for (int b = 0; b < S::NB; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.0f;

    // staging assignments, fixed for the whole walk
    unsigned x_src[S::XPASS];
    int x_dst[S::XPASS], x_row[S::XPASS];
#pragma unroll
    for (int b = 0; b < S::XPASS; ++b) {
        const int idx = threadIdx.x + b * kBlock;
        constexpr int per_ch = S::ROWS * W / 4;
        const int ch = idx / per_ch, rem = idx % per_ch;
        const int rr = rem / (W / 4), q = rem % (W / 4);
        x_row[b] = idx < S::XVEC ? rr : -1000000;
        x_src[b] = static_cast<unsigned>(ch * HW + (rr - 1) * W + 4 * q) * 4u;   // + image, first row, channel block
        x_dst[b] = ch * S::XCS + rr * S::PITCH + 1 + 4 * q;
    }
    const __amdgpu_buffer_rsrc_t x_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(x), 0, static_cast<int>(x_bytes), 0x00020000);
    constexpr unsigned kOutside = 0x80000000u;
    const float* wsrc = packed + static_cast<long long>(ct) * stages * S::WBUF + 4 * threadIdx.x;
    unsigned x_stage = static_cast<unsigned>(n * C * HW + oh0 * W) * 4u;
    floatx4 rx[S::XPASS], rw[S::WPASS];
    auto fetch = [&]() {
#pragma unroll
        for (int b = 0; b < S::XPASS; ++b) {
            const bool ok = static_cast<unsigned>(oh0 - 1 + x_row[b]) < static_cast<unsigned>(H);
            rx[b] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, ok ? x_stage + x_src[b] : kOutside, 0, 0));
        }
#pragma unroll
        for (int b = 0; b < S::WPASS; ++b)
            if ((b + 1) * kBlock <= S::WVEC || threadIdx.x + b * kBlock < S::WVEC)
                rw[b] = *reinterpret_cast<const floatx4*>(wsrc + 4 * b * kBlock);
        x_stage += static_cast<unsigned>(S::CB * HW) * 4u;
        wsrc += S::WBUF;
    };
    auto stash = [&](int buf) {
        float* xb = xs + buf * S::XBUF;
        float* wb = ws + buf * S::WBUF + 4 * threadIdx.x;
#pragma unroll
        for (int b = 0; b < S::XPASS; ++b)
            if ((b + 1) * kBlock <= S::XVEC || x_row[b] >= 0) {
                float* d = xb + x_dst[b];
                d[0] = rx[b][0]; d[1] = rx[b][1]; d[2] = rx[b][2]; d[3] = rx[b][3];
            }
#pragma unroll
        for (int b = 0; b < S::WPASS; ++b)
            if ((b + 1) * kBlock <= S::WVEC || threadIdx.x + b * kBlock < S::WVEC)
                *reinterpret_cast<floatx4*>(wb + 4 * b * kBlock) = rw[b];
    };
    // fragment addresses: lane l32 of pixel block pb is pixel (p_row[pb], p_col) of the tile, channel
    // parity h; output channel l32 of block nb
    int p_row[S::PB], p_col, x_lane[S::PB];
#pragma unroll
    for (int pb = 0; pb < S::PB; ++pb) {
        if constexpr (W == 16) {
            static_assert(W != 16 || (RT == 8 && S::PB == 2), "rows b and b + 4 form a block");
            p_row[pb] = 2 * wp + pb + 4 * (l32 / 16);
            p_col = l32 % 16;
        } else if constexpr (W == 8) {
            static_assert(W != 8 || (RT == 8 && S::PB == 1), "rows b, b + 2, b + 4, b + 6 form a block");
            p_row[pb] = wp + 2 * (l32 / 8);
            p_col = l32 % 8;
        } else {
            p_row[pb] = wp * (RT / 2) + pb;
            p_col = l32;
        }
        x_lane[pb] = p_row[pb] * S::PITCH + p_col + h * S::XCS;
    }
    const int w_lane = h * BN + wc * (BN / 2) + l32;
    auto compute = [&](int buf) {
        const float* xb = xs + buf * S::XBUF;
        const float* wb = ws + buf * S::WBUF + w_lane;
#pragma unroll
        for (int tap = 0; tap < 9; ++tap)
#pragma unroll
            for (int m = 0; m < S::CB / 2; ++m) {
                const int ks = tap * (S::CB / 2) + m;
                float a[S::NB], b[S::PB];
#pragma unroll
                for (int nb = 0; nb < S::NB; ++nb) a[nb] = wb[ks * 2 * BN + nb * 32];
#pragma unroll
                for (int pb = 0; pb < S::PB; ++pb)
                    b[pb] = xb[x_lane[pb] + 2 * m * S::XCS + (tap / 3) * S::PITCH + tap % 3];
#pragma unroll
                for (int pb = 0; pb < S::PB; ++pb)
#pragma unroll
                    for (int nb = 0; nb < S::NB; ++nb)
                        acc[pb][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[nb], b[pb], acc[pb][nb], 0, 0, 0);
            }
    };

    for (int i = threadIdx.x; i < 2 * S::XBUF; i += kBlock) xs[i] = 0.0f;   // the zero columns stay
    fetch();
    __syncthreads();
    stash(0);
    __syncthreads();
    int buf = 0;
    for (int s = 0; s < stages; ++s) {
        const bool more = s + 1 < stages;
        if (more) fetch();
        compute(buf);
        if (more) stash(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }

    // register v of lane (l32, h) of a block: output channel 8*(v/4) + 4*h + v%4, pixel l32
    const long long CoP = static_cast<long long>(Cout) * HW;
#pragma unroll
    for (int nb = 0; nb < S::NB; ++nb) {
        const int cbase = ct * BN + wc * (BN / 2) + nb * 32 + 4 * h;
        float bv[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) bv[v] = bias ? bias[cbase + 8 * (v / 4) + v % 4] : 0.0f;
#pragma unroll
        for (int pb = 0; pb < S::PB; ++pb) {
            float* dst = out + n * CoP + (oh0 + p_row[pb]) * W + p_col;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                float r = acc[pb][nb][v] + bv[v];
                if (relu) r = r > 0.0f ? r : 0.0f;
                dst[static_cast<long long>(cbase + 8 * (v / 4) + v % 4) * HW] = r;
            }
        }
    }
}

// the tile shape for a geometry: rows of 32 pixels in tiles of four or eight rows, rows of 16 or 8 in
// tiles of eight (128 / 64 pixels); 0 when the geometry does not fit
int strip_rows(int H, int W) {
    const int rt = W == 32 ? 4 : (W == 16 || W == 8) ? 8 : 0;
    return rt && H % rt == 0 ? rt : 0;
}

}  // namespace

// Shapes the forward strip kernel takes: 3x3, stride 1, padding 1 (the patch grid is the image), rows of
// 8, 16 or 32 pixels in whole tiles, input channels in multiples of 8 and output channels in multiples
// of 64, 16-byte aligned operands of less than 2 GiB, the regrouped weights within the workspace.
bool conv_fwd_strip_ok(const float* x, const float* out, int C, int H, int W, int Cout, int kH, int kW, int pad_h,
                       int pad_w, int sh, int sw, int Ho, int Wo, int N) {
    if (kH != 3 || kW != 3 || pad_h != 1 || pad_w != 1 || sh != 1 || sw != 1 || Ho != H || Wo != W) return false;
    if (!strip_rows(H, W) || C % 8 != 0 || Cout % 64 != 0) return false;
    if (!aligned16(x) || !aligned16(out)) return false;
    const long long hw = static_cast<long long>(H) * W;
    if (hw * C * N >= (1ll << 29) || hw * Cout * N >= (1ll << 29)) return false;
    return static_cast<long long>(C) * 9 * Cout <= static_cast<long long>(kWorkspaceFloats);
}

// weights: the layer's stored matrix; flip = 1 for the input-gradient product (x is then the upstream
// gradient, C its channel count, Cout the layer's input channels)
int launch_conv_fwd_strip(const float* x, const float* weights, const float* bias, float* out, int C, int H, int W,
                          int Cout, int N, int relu, int flip) {
    float* packed = workspace();
    if (!packed) return -2;
    int RT = strip_rows(H, W);
    // rows of 32 pixels: tiles of eight rows (256 pixels: less of the strip is halo, and the weights of a
    // stage feed twice the work) when that still gives every CU two workgroups
    if (W == 32 && H % 8 == 0 && static_cast<long long>(N) * (H / 8) * (Cout / 64) >= 2ll * num_cus()) RT = 8;
    const long long tiles_p = static_cast<long long>(N) * (H / RT);
    // 128 output channels per tile when that still gives every CU two workgroups
    const int BN = (Cout % 128 == 0 && tiles_p * (Cout / 128) >= 2ll * num_cus()) ? 128 : 64;
    const int CB = 512 / BN;
    const int tiles_co = Cout / BN;
    const long long total = static_cast<long long>(C) * 9 * Cout;
    if (tiles_p * tiles_co > 0x7fffffffll) return -1;
    hipStream_t s = stream();
    conv_strip_pack_kernel<<<grid_cover(static_cast<size_t>(total), kBlock), kBlock, 0, s>>>(packed, weights, C, Cout, BN, CB,
                                                                                         flip, total);
    const unsigned grid = static_cast<unsigned>(tiles_p * tiles_co);
    const unsigned xb = static_cast<unsigned>(static_cast<size_t>(N) * C * H * W * sizeof(float));
#define JZ_FWD_STRIP(W_, RT_)                                                                                              \
    do {                                                                                                                   \
        if (BN == 128) conv_fwd_strip_kernel<W_, RT_, 128><<<grid, kBlock, 0, s>>>(x, packed, bias, out, C, H, Cout, tiles_co, relu, xb); \
        else conv_fwd_strip_kernel<W_, RT_, 64><<<grid, kBlock, 0, s>>>(x, packed, bias, out, C, H, Cout, tiles_co, relu, xb);  \
    } while (0)
    if (W == 32 && RT == 8) JZ_FWD_STRIP(32, 8);
    else if (W == 32) JZ_FWD_STRIP(32, 4);
    else if (W == 16) JZ_FWD_STRIP(16, 8);
    else JZ_FWD_STRIP(8, 8);
#undef JZ_FWD_STRIP
    return launch_rc();
}

}  // namespace jz
