// Weight gradients of a 3x3, stride-1, pad-1 convolution from image strips in LDS:
//     dW((c, ky, kx), co) = sum over (n, oh, ow) of x(c, oh + ky - 1, ow + kx - 1; n) * t(co, oh, ow; n)
// (the product col * t2d^T of ConvLayer::backward, ml/layer.hpp:1690-1695, with the patch
// matrix never formed).  The nine taps of a channel read the same pixels shifted by a row
// or a column, so a workgroup stages the rows of 32 input channels once per stage, with a
// zero column on either side and zero rows above and below the image, and every tap's
// operand is the same LDS strip at another offset: no index arithmetic or bounds test per
// element, one global load per pixel instead of nine.
//
// Tile: 32 input channels x 32 output channels x 9 taps = nine 32x32 accumulators per
// wave.  A stage is 64 consecutive output pixels of one image (64/W rows); the four waves
// take 16 pixels each and accumulate the same tile, so an upstream-gradient fragment feeds
// nine matrix instructions.  The image is cut into chunks of stages across workgroups;
// at the end the four waves' sums are added through LDS in a fixed order, the chunk's
// partial tile goes to the workspace in the accumulators' own layout, and a second
// kernel adds the chunks in order and writes the (K, C_out) matrix.
#include "common.hpp"
#include "gemm_tile.hpp"

namespace jz {
namespace {

constexpr int kStagePixels = 64;   // output pixels per stage, 16 per wave
constexpr int kCB = 32;            // channels per tile, both sides
constexpr int kTileFloats = 9 * kCB * kCB;

template <int W>
struct Strip {
    static constexpr int R = kStagePixels / W;          // output rows per stage
    static constexpr int ROWS = R + 2;                   // staged input rows
    static constexpr int PITCH = W + 2;                  // a zero column on either side
    static constexpr int CSTRIDE = (ROWS * PITCH) | 1;   // odd: the 32 channels of a fragment read hit distinct banks
    static constexpr int XBUF = kCB * CSTRIDE;
    static constexpr int TPITCH = kStagePixels + 1;
    static constexpr int TBUF = kCB * TPITCH;
    static constexpr int XVEC = kCB * ROWS * W / 4;      // float4 per stage of x
    static constexpr int XPASS = (XVEC + kBlock - 1) / kBlock;
    static constexpr int TPASS = kCB * kStagePixels / 4 / kBlock;
    static constexpr int kReduce = 4 * 48 * kWave;       // floats the closing sum of the four waves needs
    static constexpr int LDS = 2 * XBUF + 2 * TBUF > kReduce ? 2 * XBUF + 2 * TBUF : kReduce;
    static_assert(kStagePixels % W == 0 && W % 8 == 0, "a wave's half (8 pixels) must lie in one image row");
};

template <int W>
__global__ __launch_bounds__(kBlock, 2) void conv_dw_strip_kernel(const float* __restrict__ x,
                                                                  const float* __restrict__ t,
                                                                  float* __restrict__ part, int C, int H, int Cout,
                                                                  int units, int units_per_chunk, int tiles_co,
                                                                  int tiles, int chunks, unsigned x_bytes,
                                                                  unsigned t_bytes) {
    using S = Strip<W>;
    __shared__ __attribute__((aligned(16))) float lds[S::LDS];
    float* const xs = lds;                   // [2][XBUF]
    float* const ts = lds + 2 * S::XBUF;     // [2][TBUF]

    // the workgroups of a chunk (same pixels, different tiles) are neighbours in one XCD's
    // dispatch order (ids congruent mod 8), so the strips they share meet in that L2
    const int lin = blockIdx.x;
    int chunk, tile;
    if (chunks % 8 == 0) {
        chunk = (lin % 8) + 8 * (lin / (8 * tiles));
        tile = (lin / 8) % tiles;
    } else {
        tile = lin % tiles;
        chunk = lin / tiles;
    }
    const int c0 = (tile / tiles_co) * kCB, co0 = (tile % tiles_co) * kCB;
    const int u_lo = chunk * units_per_chunk;
    const int u_hi = u_lo + units_per_chunk < units ? u_lo + units_per_chunk : units;
    const int per_image = H / S::R;          // stages per image
    const int HW = H * W;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int l32 = lane & 31, h = lane >> 5;

    floatx16 acc[9];
#pragma unroll
    for (int a = 0; a < 9; ++a)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[a][v] = 0.0f;

    // what a thread stages does not depend on the stage: (channel, staged row, float4 of the row) for x,
    // (output channel, float4 of the 64 pixels) for t.  Loads go through buffer resources over the
    // whole of x and of t (at most 2 GiB each): a staged row outside the image gets the offset
    // kOutside, which the hardware range check answers with zeros, so no load sits in a branch.
    unsigned x_src[S::XPASS], t_src[S::TPASS];   // byte offsets inside the image pair (n, first row of the stage)
    int x_dst[S::XPASS], x_row[S::XPASS], t_dst[S::TPASS];
#pragma unroll
    for (int b = 0; b < S::XPASS; ++b) {
        const int idx = threadIdx.x + b * kBlock;
        constexpr int per_ch = S::ROWS * W / 4;
        const int ch = idx / per_ch, rem = idx % per_ch;
        const int rr = rem / (W / 4), q = rem % (W / 4);
        x_row[b] = idx < S::XVEC ? rr : -1000000;          // never a row of the image
        x_src[b] = static_cast<unsigned>((c0 + ch) * HW + (rr - 1) * W + 4 * q) * 4u;   // wraps for rr = 0 of channel 0: masked then
        x_dst[b] = ch * S::CSTRIDE + rr * S::PITCH + 1 + 4 * q;
    }
#pragma unroll
    for (int b = 0; b < S::TPASS; ++b) {
        const int idx = threadIdx.x + b * kBlock;
        const int co = idx / (kStagePixels / 4), q = idx % (kStagePixels / 4);
        t_src[b] = static_cast<unsigned>((co0 + co) * HW + 4 * q) * 4u;
        t_dst[b] = co * S::TPITCH + 4 * q;
    }
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(x), 0, static_cast<int>(x_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t t_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(t), 0, static_cast<int>(t_bytes), 0x00020000);
    constexpr unsigned kOutside = 0x80000000u;
    floatx4 rx[S::XPASS], rt[S::TPASS];
    // the stage being fetched: image fn, first output row foh (stages are visited in order)
    int fn = u_lo / per_image, foh = (u_lo - fn * per_image) * S::R;
    auto fetch = [&]() {
        const unsigned xi = static_cast<unsigned>(fn * C * HW + foh * W) * 4u;
        const unsigned ti = static_cast<unsigned>(fn * Cout * HW + foh * W) * 4u;
#pragma unroll
        for (int b = 0; b < S::XPASS; ++b) {
            const bool ok = static_cast<unsigned>(foh - 1 + x_row[b]) < static_cast<unsigned>(H);
            rx[b] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, ok ? xi + x_src[b] : kOutside, 0, 0));
        }
#pragma unroll
        for (int b = 0; b < S::TPASS; ++b)
            rt[b] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(t_rsrc, ti + t_src[b], 0, 0));
        foh += S::R;
        if (foh == H) {
            foh = 0;
            ++fn;
        }
    };
    auto stash = [&](int buf) {
        float* xb = xs + buf * S::XBUF;
        float* tb = ts + buf * S::TBUF;
#pragma unroll
        for (int b = 0; b < S::XPASS; ++b)
            if ((b + 1) * kBlock <= S::XVEC || x_row[b] >= 0) {   // only a last, partial pass needs the test
                float* d = xb + x_dst[b];
                d[0] = rx[b][0]; d[1] = rx[b][1]; d[2] = rx[b][2]; d[3] = rx[b][3];
            }
#pragma unroll
        for (int b = 0; b < S::TPASS; ++b) {
            float* d = tb + t_dst[b];
            d[0] = rt[b][0]; d[1] = rt[b][1]; d[2] = rt[b][2]; d[3] = rt[b][3];
        }
    };
    // lane (l32, h) of a fragment: channel l32, pixel parity h
    const int x_lane = l32 * S::CSTRIDE + h;
    const int t_lane = l32 * S::TPITCH + h;
    // A stage is four quarters of four pixels (two steps of the matrix instruction) per wave.
    // The fragments of a quarter are read from LDS while the matrix instructions of the
    // quarter before run.
    struct Quarter {
        float xv[3][5];   // padded columns ow + kx (+ h) of the three input rows, ow = 0, 2
        float tv[2];
    };
    auto read_quarter = [&](int buf, int q, Quarter& f) {
        const int p0 = 16 * wave + 4 * q;
        const float* xr = xs + buf * S::XBUF + x_lane + (p0 / W) * S::PITCH + p0 % W;
        const float* tr = ts + buf * S::TBUF + t_lane + p0;
#pragma unroll
        for (int ky = 0; ky < 3; ++ky)
#pragma unroll
            for (int m = 0; m < 5; ++m) f.xv[ky][m] = xr[ky * S::PITCH + m];
        f.tv[0] = tr[0];
        f.tv[1] = tr[2];
    };
    auto mfma_quarter = [&](const Quarter& f) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int ky = 0; ky < 3; ++ky)
#pragma unroll
                for (int kx = 0; kx < 3; ++kx)
                    acc[ky * 3 + kx] =
                        __builtin_amdgcn_mfma_f32_32x32x2f32(f.tv[ks], f.xv[ky][2 * ks + kx], acc[ky * 3 + kx], 0, 0, 0);
    };
    // Stage u: the registers hold stage u + 1, requested a whole stage ago (a request takes
    // longer than half a stage to return when every workgroup asks at once).  They go to the
    // other LDS buffer behind the first quarter's matrix instructions, and stage u + 2 is
    // requested into them.
    auto compute = [&](int buf, bool has1, bool has2) {
        Quarter f0, f1;
        read_quarter(buf, 0, f0);
        read_quarter(buf, 1, f1);
        __builtin_amdgcn_sched_barrier(0);
        mfma_quarter(f0);
        __builtin_amdgcn_sched_barrier(0);
        if (has1) stash(buf ^ 1);
        if (has2) fetch();
        read_quarter(buf, 2, f0);
        __builtin_amdgcn_sched_barrier(0);
        mfma_quarter(f1);
        __builtin_amdgcn_sched_barrier(0);
        read_quarter(buf, 3, f1);
        __builtin_amdgcn_sched_barrier(0);
        mfma_quarter(f0);
        __builtin_amdgcn_sched_barrier(0);
        mfma_quarter(f1);
    };

    // zero columns and the rows a first stage may leave untouched
    for (int i = threadIdx.x; i < 2 * S::XBUF; i += kBlock) xs[i] = 0.0f;
    if (u_lo < u_hi) {
        fetch();
        __syncthreads();
        stash(0);
        if (u_lo + 1 < u_hi) fetch();
        __syncthreads();
        int buf = 0;
        for (int u = u_lo; u < u_hi; ++u) {
            compute(buf, u + 1 < u_hi, u + 2 < u_hi);
            __syncthreads();
            buf ^= 1;
        }
    } else {
        __syncthreads();
    }

    // the four waves' sums, three taps (48 registers) at a time: every wave writes its
    // registers, wave q then adds registers 12q .. 12q + 11 of the four in wave order
    float* out = part + (static_cast<long long>(chunk) * tiles + tile) * kTileFloats;
    float* red = lds;   // [wave][48][64]
#pragma unroll
    for (int ky = 0; ky < 3; ++ky) {
#pragma unroll
        for (int rv = 0; rv < 48; ++rv) red[(wave * 48 + rv) * kWave + lane] = acc[3 * ky + rv / 16][rv % 16];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 12; ++r) {
            const int rv = wave * 12 + r;
            float s = red[(0 * 48 + rv) * kWave + lane];
            s += red[(1 * 48 + rv) * kWave + lane];
            s += red[(2 * 48 + rv) * kWave + lane];
            s += red[(3 * 48 + rv) * kWave + lane];
            out[(3 * ky + rv / 16) * (kCB * kCB) + (rv % 16) * kWave + lane] = s;
        }
        __syncthreads();
    }
}

// dW((c, ky, kx), co) = sum over chunks of the partial tiles.  Element (tap, v, lane) of a
// tile is output channel 8*(v/4) + 4*(lane/32) + v%4 and input channel lane%32 of the tile
// (the accumulator layout of the 32x32 matrix instruction).  A workgroup takes 64
// consecutive elements; wave w adds the chunks of the w-th eighth of the range in order
// (independent loads, eight at a time), and the eight sums are added in wave order.
constexpr int kCombineWaves = 8;
__global__ __launch_bounds__(kCombineWaves* kWave) void conv_dw_strip_combine_kernel(float* __restrict__ dW,
                                                                                     const float* __restrict__ part,
                                                                                     int K, int tiles_co, int tiles,
                                                                                     int chunks) {
    __shared__ float sums[kCombineWaves][kWave];
    const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
    const int e = blockIdx.x * kWave + lane;   // < tiles * kTileFloats, a multiple of 64
    const long long stride = static_cast<long long>(tiles) * kTileFloats;
    const int per = (chunks + kCombineWaves - 1) / kCombineWaves;
    const int lo = w * per, hi = lo + per < chunks ? lo + per : chunks;
    float s = 0.0f;
    int c = lo;
    for (; c + 8 <= hi; c += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = part[(c + u) * stride + e];
#pragma unroll
        for (int u = 0; u < 8; ++u) s += v[u];
    }
    for (; c < hi; ++c) s += part[c * stride + e];
    sums[w][lane] = s;
    __syncthreads();
    if (w != 0) return;
#pragma unroll
    for (int u = 1; u < kCombineWaves; ++u) s += sums[u][lane];
    const int tile = e / kTileFloats, r = e % kTileFloats;
    const int tap = r / (kCB * kCB), v = (r / kWave) % 16;
    const int co = (tile % tiles_co) * kCB + 8 * (v / 4) + 4 * (lane / 32) + v % 4;
    const int ci = (tile / tiles_co) * kCB + lane % 32;
    dW[static_cast<long long>(co) * K + ci * 9 + tap] = s;
}

}  // namespace

// Shapes the strip kernel takes: 3x3, stride 1, padding 1 (the patch grid is the image), rows
// of 8, 16, 32 or 64 pixels with a whole number of 64-pixel stages per image, channel counts in
// multiples of 32 on both sides, 16-byte aligned operands, at least four stages per workgroup.
bool conv_dw_strip_ok(const float* x, const float* t, int C, int H, int W, int Cout, int kH, int kW, int pad_h,
                      int pad_w, int sh, int sw, int Ho, int Wo, int N) {
    if (kH != 3 || kW != 3 || pad_h != 1 || pad_w != 1 || sh != 1 || sw != 1 || Ho != H || Wo != W) return false;
    if (W != 8 && W != 16 && W != 32 && W != 64) return false;
    if (H % (kStagePixels / W) != 0 || C % kCB != 0 || Cout % kCB != 0) return false;
    if (!aligned16(x) || !aligned16(t)) return false;
    const long long hw = static_cast<long long>(H) * W;
    if (hw * C * N >= (1ll << 29) || hw * Cout * N >= (1ll << 29)) return false;   // 2 GiB per buffer resource
    const long long tiles = static_cast<long long>(C / kCB) * (Cout / kCB);
    const long long units = static_cast<long long>(N) * (H / (kStagePixels / W));
    return units >= 4 && tiles * kTileFloats <= static_cast<long long>(kWorkspaceFloats);
}

int launch_conv_dw_strip(const float* x, const float* t, float* dW, int C, int H, int W, int Cout, int N) {
    float* part = workspace();
    if (!part) return -2;
    const int tiles_co = Cout / kCB, tiles = (C / kCB) * tiles_co;
    const int units = N * (H / (kStagePixels / W));
    // two workgroups per CU, chunks in multiples of 8, four stages or more each
    long long chunks = (2ll * num_cus() + tiles - 1) / tiles;
    if (chunks >= 8) chunks = chunks / 8 * 8;
    if (chunks > units / 4) chunks = units / 4;
    while (chunks > 1 && chunks * tiles * kTileFloats > static_cast<long long>(kWorkspaceFloats)) --chunks;
    if (chunks < 1) chunks = 1;
    const int upc = static_cast<int>((units + chunks - 1) / chunks);
    chunks = (units + upc - 1) / upc;
    const unsigned grid = static_cast<unsigned>(chunks * tiles);
    hipStream_t s = stream();
    const int nch = static_cast<int>(chunks);
    const unsigned xb = static_cast<unsigned>(static_cast<size_t>(N) * C * H * W * sizeof(float));
    const unsigned tb = static_cast<unsigned>(static_cast<size_t>(N) * Cout * H * W * sizeof(float));
    if (W == 8) conv_dw_strip_kernel<8><<<grid, kBlock, 0, s>>>(x, t, part, C, H, Cout, units, upc, tiles_co, tiles, nch, xb, tb);
    else if (W == 16) conv_dw_strip_kernel<16><<<grid, kBlock, 0, s>>>(x, t, part, C, H, Cout, units, upc, tiles_co, tiles, nch, xb, tb);
    else if (W == 32) conv_dw_strip_kernel<32><<<grid, kBlock, 0, s>>>(x, t, part, C, H, Cout, units, upc, tiles_co, tiles, nch, xb, tb);
    else conv_dw_strip_kernel<64><<<grid, kBlock, 0, s>>>(x, t, part, C, H, Cout, units, upc, tiles_co, tiles, nch, xb, tb);
    conv_dw_strip_combine_kernel<<<tiles * (kTileFloats / kWave), kCombineWaves * kWave, 0, s>>>(dW, part, C * 9, tiles_co,
                                                                                                 tiles, nch);
    return launch_rc();
}

}  // namespace jz
