// Convolution as an implicit GEMM on the fp32 matrix cores: the patch matrix
// col(K, P*N) of the im2col formulation (ml/layer.hpp:1611-1719) is never
// written.  Its elements are formed while an operand tile is staged into LDS,
//     col(k, j) = input(c, oh*s - pad + ky, ow*s - pad + kx; image n)   or 0 outside,
//     k = (c, ky, kx),  j = n*P + oh*W_out + ow,
// so the three products of a convolution layer read the image (and the upstream
// gradient) directly:
//   forward        out(j, co)  = sum_k col(k, j) W(k, co) + bias(co)  [relu]
//                  stored straight into the layer's (C_out*P, N) layout
//   weight grads   dW(k, co)   = sum_j col(k, j) t(co, j)     (K split across workgroups)
//   input grads    dx = the forward product of t with the flipped weights
//                  (stride 1; strided layers keep the patch-matrix route)
// The tile machinery (LDS layout, fragment reads, software pipeline) is the one
// of gemm.hip; only the global -> register side of the loaders differs.
// HBM traffic per forward call: input + output + weights instead of
// input + 2 * patches + 2 * (C_out x P*N) + output.
#include "common.hpp"
#include "gemm_tile.hpp"

#include <cstdlib>
#include <type_traits>
#include <utility>

namespace jz {
void launch_splitk_reduce(float* C, const float* part, int M, int N, size_t ldc, int splits, float alpha,
                          float beta);
// conv_dw_strip.hip: 3x3 stride-1 weight gradients from image strips in LDS
bool conv_dw_strip_ok(const float* x, const float* t, int C, int H, int W, int Cout, int kH, int kW, int pad_h,
                      int pad_w, int sh, int sw, int Ho, int Wo, int N);
int launch_conv_dw_strip(const float* x, const float* t, float* dW, int C, int H, int W, int Cout, int N);
// conv_fwd_strip.hip: the forward product (and, with flipped weights, the input gradients) of such layers
bool conv_fwd_strip_ok(const float* x, const float* out, int C, int H, int W, int Cout, int kH, int kW, int pad_h,
                       int pad_w, int sh, int sw, int Ho, int Wo, int N);
int launch_conv_fwd_strip(const float* x, const float* weights, const float* bias, float* out, int C, int H, int W,
                          int Cout, int N, int relu, int flip);
// conv_few.hip: 3x3 stride-1 layers with at most four input channels, forward and weight gradients
bool conv_few_ok(const float* x, const float* other, int C, int H, int W, int kH, int kW, int pad_h, int pad_w, int sh,
                 int sw, int Ho, int Wo);
int launch_conv_few_fwd(const float* x, const float* Wt, const float* bias, float* out, int C, int H, int W, int Cout,
                        int N, int relu);
int launch_conv_few_dw(const float* x, const float* t, float* dW, int C, int H, int W, int Cout, int N);
namespace {

struct ConvGeom {
    int C, H, W;          // image the patches are taken from
    int kH, kW, pad_h, pad_w, sh, sw;
    int Ho, Wo;           // patch grid
    int N;                // images
    int Cout;             // columns of the weight matrix
    int K, P, HW, CHW, khw;
    long long J;          // P * N
    FastDiv dP, dWo, dkhw, dkW;
    // Where the forward kernel stores patch-grid position (oh, ow): pixel
    // (oh*out_sh + out_oh0, ow*out_sw + out_ow0) of an out_W-wide image of out_P pixels.
    // A convolution writes its own grid (1, 1, 0, 0, Wo, P); one residue class of a
    // transposed convolution writes every out_sh-th row and out_sw-th column.
    int out_sh, out_sw, out_oh0, out_ow0, out_W, out_P;
    long long w_off;      // this geometry's weights start w_off floats into the weight buffer
};
// The residue classes of a transposed convolution as one launch: blockIdx.y picks the class.
constexpr int kMaxClasses = 4;
struct ConvClasses {
    ConvGeom g[kMaxClasses];
};

ConvGeom make_geom(int C, int H, int W, int kH, int kW, int pad_h, int pad_w, int sh, int sw, int Ho, int Wo, int N,
                   int Cout) {
    ConvGeom g;
    g.C = C; g.H = H; g.W = W; g.kH = kH; g.kW = kW; g.pad_h = pad_h; g.pad_w = pad_w; g.sh = sh; g.sw = sw;
    g.Ho = Ho; g.Wo = Wo; g.N = N; g.Cout = Cout;
    g.khw = kH * kW;
    g.K = C * g.khw;
    g.P = Ho * Wo;
    g.HW = H * W;
    g.CHW = C * g.HW;
    g.J = static_cast<long long>(g.P) * N;
    g.dP = make_fastdiv(g.P);
    g.dWo = make_fastdiv(Wo);
    g.dkhw = make_fastdiv(g.khw);
    g.dkW = make_fastdiv(kW);
    g.out_sh = 1; g.out_sw = 1; g.out_oh0 = 0; g.out_ow0 = 0; g.out_W = Wo; g.out_P = g.P;
    g.w_off = 0;
    return g;
}

// A patch-row index k = (c, ky, kx) as an offset into one image and its tap
struct Tap {
    int off;   // c*H*W + ky*W + kx
    int ky, kx;
};
__device__ __forceinline__ Tap tap_of(int k, const ConvGeom& g) {
    const int c = static_cast<int>(fdiv(static_cast<uint32_t>(k), g.dkhw));
    const int r = k - c * g.khw;
    const int ky = static_cast<int>(fdiv(static_cast<uint32_t>(r), g.dkW));
    const int kx = r - ky * g.kW;
    return Tap{c * g.HW + ky * g.W + kx, ky, kx};
}
__device__ __forceinline__ void tap_next(Tap& t, const ConvGeom& g) {
    ++t.kx;
    ++t.off;
    if (t.kx == g.kW) {
        t.kx = 0;
        ++t.ky;
        t.off += g.W - g.kW;
        if (t.ky == g.kH) {
            t.ky = 0;
            t.off += g.HW - g.kH * g.W;
        }
    }
}
// A patch-column index j = (n, oh, ow): where its patch starts in the input
struct Site {
    long long base;   // n*C*H*W + ih0*W + iw0 (ih0, iw0 may be negative)
    int ih0, iw0;
    int oh, ow;
    int n;
};
__device__ __forceinline__ Site site_of(long long j, const ConvGeom& g) {
    const int n = static_cast<int>(fdiv(static_cast<uint32_t>(j), g.dP));
    const int p = static_cast<int>(j - static_cast<long long>(n) * g.P);
    const int oh = static_cast<int>(fdiv(static_cast<uint32_t>(p), g.dWo));
    const int ow = p - oh * g.Wo;
    Site s;
    s.n = n; s.oh = oh; s.ow = ow;
    s.ih0 = oh * g.sh - g.pad_h;
    s.iw0 = ow * g.sw - g.pad_w;
    s.base = static_cast<long long>(n) * g.CHW + static_cast<long long>(s.ih0) * g.W + s.iw0;
    return s;
}
__device__ __forceinline__ void site_next(Site& s, const ConvGeom& g) {
    ++s.ow;
    s.iw0 += g.sw;
    s.base += g.sw;
    if (s.ow == g.Wo) {
        s.ow = 0;
        ++s.oh;
        s.iw0 = -g.pad_w;
        s.ih0 += g.sh;
        s.base += static_cast<long long>(g.sh) * g.W - static_cast<long long>(g.Wo) * g.sw;
        if (s.oh == g.Ho) {
            s.oh = 0;
            ++s.n;
            s.ih0 = -g.pad_h;
            s.base = static_cast<long long>(s.n) * g.CHW + static_cast<long long>(s.ih0) * g.W + s.iw0;
        }
    }
}
__device__ __forceinline__ float patch_value(const float* __restrict__ in, const Site& s, const Tap& t,
                                             const ConvGeom& g) {
    const bool ok = static_cast<unsigned>(s.ih0 + t.ky) < static_cast<unsigned>(g.H) &&
                    static_cast<unsigned>(s.iw0 + t.kx) < static_cast<unsigned>(g.W);
    return ok ? in[s.base + t.off] : 0.0f;
}

// Bounds-checked loads through a raw buffer resource over the whole input (at most 2 GiB):
// an element that falls in the padding gets the offset kOutside, which the hardware range
// check answers with 0, so a padded element costs a select on the offset instead of a
// branch around the load.
constexpr unsigned kOutside = 0x80000000u;
constexpr long long kBufferMaxBytes = 1ll << 31;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t input_resource(const float* in, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(in), 0, static_cast<int>(bytes), 0x00020000);
}
__device__ __forceinline__ float load_or_zero(__amdgpu_buffer_rsrc_t r, unsigned byte_off) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, byte_off, 0, 0));
}

constexpr int kWGM = 2, kWGN = 2, kTM = 2;   // 128 rows per workgroup tile

// ── forward: out(j, co) = sum_k col(k, j) W(k, co) ───────────────────────────
// Rows of the tile are patch columns j (so that a register of the transposed
// MFMA result holds 32 consecutive output pixels of one channel: the store into
// the (C_out*P, N) layout is coalesced), columns are output channels.
// The A loader takes one j and four consecutive k per thread and pass.
// TAB (kH*kW <= 32 and a table of K entries that fits LDS): the patch-row index k is
// decoded once per workgroup into a table {offset inside an image, one-hot tap bit}, and
// each of a thread's pixels carries a 32-bit mask of the taps that fall inside the image,
// so an element costs a table read, an AND and an address add instead of two divisions
// and four comparisons.
template <int TM, int TN, bool FASTB, bool TAB, bool MULTI = false>
__global__ __launch_bounds__(kBlock, 2) void conv_fwd_kernel(const float* __restrict__ in, const float* __restrict__ Wt,
                                                             const float* __restrict__ bias, float* __restrict__ out,
                                                             std::conditional_t<MULTI, ConvClasses, ConvGeom> geo,
                                                             int relu, int tiles_n, unsigned in_bytes) {
    constexpr int BM = kWGM * TM * 32;
    constexpr int BN = kWGN * TN * 32;
    // MULTI: blockIdx.y selects one of up to four geometries (their weights lie behind each other)
    const ConvGeom& g = [&]() -> const ConvGeom& {
        if constexpr (MULTI) return geo.g[blockIdx.y];
        else return geo;
    }();
    Wt += g.w_off;
    using LA = TileLoader<BM, false, TM>;
    using LB = TileLoader<BN, false, TN>;
    constexpr int LDA_S = LA::LD, LDB_S = LB::LD;
    __shared__ __attribute__((aligned(16))) float As[2][BK * LDA_S];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDB_S];
    extern __shared__ __attribute__((aligned(16))) int2 tap_table[];   // TAB: K rounded up to BK entries

    // consecutive workgroups share a row tile (the same image patches) and differ in
    // the channel tile; the 8 XCDs each take a contiguous run of row tiles
    const int ntiles = gridDim.x;
    int pid = blockIdx.x;
    {
        constexpr int kXcd = 8;
        if (ntiles % kXcd == 0) pid = (pid % kXcd) * (ntiles / kXcd) + pid / kXcd;
    }
    const int tile_m = pid / tiles_n, tile_n = pid % tiles_n;
    const long long m0 = static_cast<long long>(tile_m) * BM;
    const int n0 = tile_n * BN;
    if constexpr (MULTI) {
        if (m0 >= g.J) return;   // the grid is sized for the largest class
    }

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int wm = wave % kWGM, wn = wave / kWGM;
    const int l32 = lane & 31, h = lane >> 5;

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // this thread's patch columns (one per pass), fixed for the whole K walk
    Site site[LA::kPasses];
    bool row_ok[LA::kPasses];
    unsigned tap_ok[LA::kPasses];   // TAB: bit ky*kW + kx set when that tap of the pixel is inside the image
    int kq;   // k offset of this thread inside a stage: 0, 4, 8 or 12
    {
        int x, k;
#pragma unroll
        for (int ps = 0; ps < LA::kPasses; ++ps) {
            LA::coords(ps, x, k);
            const long long j = m0 + x;
            row_ok[ps] = j < g.J;
            site[ps] = site_of(row_ok[ps] ? j : 0, g);
            tap_ok[ps] = 0;
            if constexpr (TAB) {
                if (row_ok[ps]) {
                    for (int ky = 0; ky < g.kH; ++ky)
                        for (int kx = 0; kx < g.kW; ++kx)
                            if (static_cast<unsigned>(site[ps].ih0 + ky) < static_cast<unsigned>(g.H) &&
                                static_cast<unsigned>(site[ps].iw0 + kx) < static_cast<unsigned>(g.W))
                                tap_ok[ps] |= 1u << (ky * g.kW + kx);
                }
            }
        }
        LA::coords(0, x, kq);
    }
    if constexpr (TAB) {
        const int kpad = (g.K + BK - 1) / BK * BK;
        for (int k = threadIdx.x; k < kpad; k += kBlock) {
            int2 e = make_int2(0, 0);   // rows past K match no pixel
            if (k < g.K) {
                const Tap t = tap_of(k, g);
                e = make_int2(t.off * 4, 1 << (t.ky * g.kW + t.kx));   // byte offset inside an image
            }
            tap_table[k] = e;
        }
        // (the barrier after the first stage's LDS stores also publishes the table; the
        // first two stages decode their taps directly)
    }
    floatx4 ra[LA::kPasses], rb[LB::kPasses];
    unsigned offb[LB::kPasses];
    if constexpr (FASTB) LB::offsets(offb, static_cast<unsigned>(g.K));
    // The loads of a stage are issued in pieces between the MFMA steps of the stage two
    // before it (the four taps, then one loader pass per step), so that their index
    // arithmetic runs in the shadow of the matrix pipe instead of in one burst.
    Tap taps[4];
    int kcur = 0;
    auto stage_taps = [&](int k0) {
        kcur = k0 + kq;
        Tap t = tap_of(kcur, g);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            taps[e] = t;
            tap_next(t, g);
        }
    };
    auto load_a = [&](int ps) {
        floatx4 r;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            r[e] = (row_ok[ps] && kcur + e < g.K) ? patch_value(in, site[ps], taps[e], g) : 0.0f;
        ra[ps] = r;
    };
    // table forms, used from the third stage on
    int4 tq[2];   // the thread's four table entries of the stage: {off0, bit0, off1, bit1}, {off2, ...}
    auto stage_taps_tab = [&](int k0) {
        const int4* src = reinterpret_cast<const int4*>(tap_table + k0 + kq);
        tq[0] = src[0];
        tq[1] = src[1];
    };
    const __amdgpu_buffer_rsrc_t in_rsrc = input_resource(in, in_bytes);
    unsigned site_byte[LA::kPasses];   // byte offset of the pixel's patch origin (wraps when the origin is in the padding)
#pragma unroll
    for (int ps = 0; ps < LA::kPasses; ++ps) site_byte[ps] = static_cast<unsigned>(site[ps].base) * 4u;
    auto load_a_tab = [&](int ps) {
        const int off[4] = {tq[0].x, tq[0].z, tq[1].x, tq[1].z};
        const unsigned bit[4] = {static_cast<unsigned>(tq[0].y), static_cast<unsigned>(tq[0].w),
                                 static_cast<unsigned>(tq[1].y), static_cast<unsigned>(tq[1].w)};
        floatx4 r;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            r[e] = load_or_zero(in_rsrc, (tap_ok[ps] & bit[e]) ? site_byte[ps] + static_cast<unsigned>(off[e]) : kOutside);
        ra[ps] = r;
    };
    auto load_b = [&](int k0) {
        if constexpr (FASTB)
            LB::load_fast(rb, LB::origin(Wt, g.K, n0, k0), offb);
        else
            LB::load_checked(rb, Wt, g.K, n0, k0, g.Cout, g.K);
    };
    auto load_stage = [&](int k0) {
        stage_taps(k0);
#pragma unroll
        for (int ps = 0; ps < LA::kPasses; ++ps) load_a(ps);
        load_b(k0);
    };

    const int nk = (g.K + BK - 1) / BK;
    load_stage(0);
    LA::store(ra, As[0]);
    LB::store(rb, Bs[0]);
    __syncthreads();
    if (nk > 1) load_stage(BK);

    constexpr int KS = BK / 2;
    constexpr int kStorePasses = LA::kPasses + LB::kPasses;
    static_assert(kStorePasses <= KS - 2, "staging stores must fit the MFMA steps of a stage");
    Frag<TM> af[2];
    Frag<TN> bf[2];
    const int a_off = wm * LA::kGroup + l32 * TM + h * LDA_S;
    const int b_off = wn * LB::kGroup + l32 * TN + h * LDB_S;
    auto read_frags = [&](int slot, const float* as, const float* bs, int kk) {
        af[slot].read(as + 2 * kk * LDA_S);
        bf[slot].read(bs + 2 * kk * LDB_S);
    };
    auto mfma_step = [&](int slot) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[slot][j], af[slot][i], acc[i][j], 0, 0, 0);
    };
    int cur = 0;
    read_frags(0, As[0] + a_off, Bs[0] + b_off, 0);
    for (int kt = 0; kt < nk; ++kt) {
        const bool more = kt + 1 < nk;
        const float* as = As[cur] + a_off;
        const float* bs = Bs[cur] + b_off;
#pragma unroll
        for (int kk = 0; kk < KS - 1; ++kk) {
            read_frags((kk + 1) & 1, as, bs, kk + 1);
            if (more) {
                if (kk < LA::kPasses) LA::store_pass(ra, As[cur ^ 1], kk);
                else if (kk < kStorePasses) LB::store_pass(rb, Bs[cur ^ 1], kk - LA::kPasses);
            }
            // pass p of the patch operand is requested one step after its registers went to LDS.
            // The requests are unconditional (past the end the last stage is fetched again and
            // dropped): inside a branch they made the wait of the staging store that follows
            // them a wait for all loads in flight, these fresh ones included.
            {
                const int k2 = (kt + 2 < nk ? kt + 2 : nk - 1) * BK;
                if constexpr (TAB) {
                    if (kk == 0) stage_taps_tab(k2);
                    if (kk >= 1 && kk - 1 < LA::kPasses) load_a_tab(kk - 1);
                } else {
                    if (kk == 1) stage_taps(k2);
                    if (kk >= 1 && kk - 1 < LA::kPasses) load_a(kk - 1);
                }
                if (kk == kStorePasses) load_b(k2);
            }
            __builtin_amdgcn_sched_barrier(0);
            mfma_step(kk & 1);
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
        cur ^= 1;
        if (more) read_frags(0, As[cur] + a_off, Bs[cur] + b_off, 0);
        __builtin_amdgcn_sched_barrier(0);
        mfma_step((KS - 1) & 1);
    }

    // store: register v of lane (h, l32) is (row l32, column 8*(v/4) + 4*h + v%4) of a 32x32 tile
    const long long CoP = static_cast<long long>(g.Cout) * g.out_P;
    // the bias values of the wave's output channels, requested together (one load and one
    // wait per stored element made the store loop a chain of round trips)
    float bv[TN][16];
#pragma unroll
    for (int jn = 0; jn < TN; ++jn)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int co = n0 + (wn * TN + jn) * 32 + 4 * h + 8 * (v / 4) + (v % 4);
            bv[jn][v] = (bias && co < g.Cout) ? bias[co] : 0.0f;
        }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const long long j = m0 + (wm * TM + i) * 32 + l32;
        if (j >= g.J) continue;
        const int n = static_cast<int>(fdiv(static_cast<uint32_t>(j), g.dP));
        int p = static_cast<int>(j - static_cast<long long>(n) * g.P);
        if constexpr (MULTI) {
            const int oh = static_cast<int>(fdiv(static_cast<uint32_t>(p), g.dWo));
            const int ow = p - oh * g.Wo;
            p = (oh * g.out_sh + g.out_oh0) * g.out_W + ow * g.out_sw + g.out_ow0;
        }
        float* dst = out + static_cast<long long>(n) * CoP + p;
#pragma unroll
        for (int jn = 0; jn < TN; ++jn) {
            const int cbase = n0 + (wn * TN + jn) * 32 + 4 * h;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int co = cbase + 8 * (v / 4) + (v % 4);
                if (co < g.Cout) {
                    float r = acc[i][jn][v];
                    if (bias) r += bv[jn][v];
                    if (relu) r = r > 0.0f ? r : 0.0f;
                    dst[static_cast<long long>(co) * g.out_P] = r;
                }
            }
        }
    }
}

// ── weight gradients: dW(k, co) = sum_j col(k, j) t(co, j) ───────────────────
// Rows of the tile are patch rows k, columns are output channels, the
// contraction runs over patch columns j and is cut into chunks across
// workgroups (partial results in `part`, summed afterwards in a fixed order).
// t is the upstream gradient in the layer's own (C_out*P, N) layout.  Both
// loaders take four consecutive j per thread: image pixels along a row for the
// patch operand, one float4 of t for the other.
template <int TN, bool QUAD>
__global__ __launch_bounds__(kBlock, 2) void conv_dw_kernel(const float* __restrict__ in, const float* __restrict__ t,
                                                            float* __restrict__ part, ConvGeom g, int tiles_n,
                                                            long long j_chunk, int t_vec, unsigned in_bytes) {
    constexpr int BM = kWGM * kTM * 32;
    constexpr int BN = kWGN * TN * 32;
    using LA = TileLoader<BM, false, kTM>;
    using LB = TileLoader<BN, false, TN>;
    constexpr int LDA_S = LA::LD, LDB_S = LB::LD;
    __shared__ __attribute__((aligned(16))) float As[2][BK * LDA_S];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDB_S];

    // the chunk is the fastest-varying part of the dispatch order: an XCD (ids congruent
    // mod 8) then keeps to its own chunks of the image
    const int splits = gridDim.y;
    const int lin = blockIdx.x + blockIdx.y * gridDim.x;
    const int chunk = lin % splits;
    const int pid = lin / splits;
    const int tile_m = pid / tiles_n, tile_n = pid % tiles_n;
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;
    const long long j_lo = static_cast<long long>(chunk) * j_chunk;
    const long long j_hi = (j_lo + j_chunk) < g.J ? (j_lo + j_chunk) : g.J;
    float* C = part + static_cast<long long>(chunk) * g.K * g.Cout;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int wm = wave % kWGM, wn = wave / kWGM;
    const int l32 = lane & 31, h = lane >> 5;

    floatx16 acc[kTM][TN];
#pragma unroll
    for (int i = 0; i < kTM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // this thread's patch rows (one per pass of the A loader) and channels (B loader)
    Tap tap[LA::kPasses];
    bool k_ok[LA::kPasses];
    int co_b[LB::kPasses];
    int jq;   // j offset of this thread inside a stage: 0, 4, 8 or 12
    {
        int x, k;
#pragma unroll
        for (int ps = 0; ps < LA::kPasses; ++ps) {
            LA::coords(ps, x, k);
            k_ok[ps] = m0 + x < g.K;
            tap[ps] = tap_of(k_ok[ps] ? m0 + x : 0, g);
        }
#pragma unroll
        for (int ps = 0; ps < LB::kPasses; ++ps) {
            LB::coords(ps, x, k);
            co_b[ps] = n0 + x;
        }
        LA::coords(0, x, jq);
    }
    const long long CoP = static_cast<long long>(g.Cout) * g.P;
    floatx4 ra[LA::kPasses], rb[LB::kPasses];
    // The loads of a stage are issued in pieces between the MFMA steps of the stage two
    // before it (stage_sites, then one loader pass per step), so that their index
    // arithmetic runs in the shadow of the matrix pipe instead of in one burst.
    // QUAD (W_out % 4 == 0): the four patch columns of a thread are consecutive pixels of
    // one output row, so one site and one row test serve all four.
    const __amdgpu_buffer_rsrc_t in_rsrc = input_resource(in, in_bytes);   // in_bytes == 0: not used
    Site sites[QUAD ? 1 : 4];
    long long jcur = 0;
    bool quad_live = false;   // QUAD: the thread's four columns are inside this workgroup's chunk
    auto stage_sites = [&](long long jst) {
        jcur = jst + jq;
        if constexpr (QUAD) {
            // stages are visited in order, BK columns apart: the site moves along its row
            // and wraps into the next row or image (J % 4 == 0, so a quad is inside the
            // chunk or outside it as a whole)
            if (jst == j_lo) {
                sites[0] = site_of(jcur < g.J ? jcur : 0, g);
            } else {
                Site& q = sites[0];
                q.ow += BK;
                while (q.ow >= g.Wo) {
                    q.ow -= g.Wo;
                    if (++q.oh == g.Ho) {
                        q.oh = 0;
                        ++q.n;
                    }
                }
                q.ih0 = q.oh * g.sh - g.pad_h;
                q.iw0 = q.ow * g.sw - g.pad_w;
                q.base = static_cast<long long>(q.n) * g.CHW + (q.ih0 * g.W + q.iw0);
            }
            quad_live = jcur < j_hi;
        } else {
            Site s0 = site_of(jcur < g.J ? jcur : 0, g);
            sites[0] = s0;
#pragma unroll
            for (int e = 1; e < 4; ++e) {
                site_next(s0, g);
                sites[e] = s0;
            }
        }
    };
    auto load_a = [&](int ps) {
        floatx4 r;
        if constexpr (QUAD) {
            const Site& s0 = sites[0];
            const bool row = k_ok[ps] && quad_live &&
                             static_cast<unsigned>(s0.ih0 + tap[ps].ky) < static_cast<unsigned>(g.H);
            const int iw = s0.iw0 + tap[ps].kx;
            const unsigned byte0 = (static_cast<unsigned>(s0.base) + static_cast<unsigned>(tap[ps].off)) * 4u;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const bool ok = row && static_cast<unsigned>(iw + e * g.sw) < static_cast<unsigned>(g.W);
                r[e] = load_or_zero(in_rsrc, ok ? byte0 + static_cast<unsigned>(e * g.sw) * 4u : kOutside);
            }
        } else {
            if (in_bytes != 0) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const Site& se = sites[e];
                    const bool ok = k_ok[ps] && jcur + e < j_hi &&
                                    static_cast<unsigned>(se.ih0 + tap[ps].ky) < static_cast<unsigned>(g.H) &&
                                    static_cast<unsigned>(se.iw0 + tap[ps].kx) < static_cast<unsigned>(g.W);
                    r[e] = load_or_zero(in_rsrc, ok ? (static_cast<unsigned>(se.base) + static_cast<unsigned>(tap[ps].off)) * 4u
                                                    : kOutside);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    r[e] = (k_ok[ps] && jcur + e < j_hi) ? patch_value(in, sites[e], tap[ps], g) : 0.0f;
            }
        }
        ra[ps] = r;
    };
    auto load_b = [&](int ps) {
        if (!LB::active(ps)) return;
        floatx4 r = {0.f, 0.f, 0.f, 0.f};
        if (co_b[ps] < g.Cout) {
            if (t_vec && jcur + 3 < j_hi) {
                // P % 4 == 0 and j % 4 == 0: the four pixels are consecutive in one image
                const int p = sites[0].oh * g.Wo + sites[0].ow;
                r = *reinterpret_cast<const floatx4*>(t + sites[0].n * CoP + static_cast<long long>(co_b[ps]) * g.P + p);
            } else {
                Site se = sites[0];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (jcur + e < j_hi) r[e] = t[se.n * CoP + static_cast<long long>(co_b[ps]) * g.P + se.oh * g.Wo + se.ow];
                    site_next(se, g);
                }
            }
        }
        rb[ps] = r;
    };
    auto load_stage = [&](long long jst) {
        stage_sites(jst);
#pragma unroll
        for (int ps = 0; ps < LA::kPasses; ++ps) load_a(ps);
#pragma unroll
        for (int ps = 0; ps < LB::kPasses; ++ps) load_b(ps);
    };

    const int nk = static_cast<int>((j_hi - j_lo + BK - 1) / BK);
    if (nk > 0) {
        load_stage(j_lo);
        LA::store(ra, As[0]);
        LB::store(rb, Bs[0]);
        __syncthreads();
        if (nk > 1) load_stage(j_lo + BK);

        constexpr int KS = BK / 2;
        constexpr int kStorePasses = LA::kPasses + LB::kPasses;
        static_assert(kStorePasses <= KS - 2, "staging stores must fit the MFMA steps of a stage");
        Frag<kTM> af[2];
        Frag<TN> bf[2];
        const int a_off = wm * LA::kGroup + l32 * kTM + h * LDA_S;
        const int b_off = wn * LB::kGroup + l32 * TN + h * LDB_S;
        auto read_frags = [&](int slot, const float* as, const float* bs, int kk) {
            af[slot].read(as + 2 * kk * LDA_S);
            bf[slot].read(bs + 2 * kk * LDB_S);
        };
        auto mfma_step = [&](int slot) {
#pragma unroll
            for (int i = 0; i < kTM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[slot][j], af[slot][i], acc[i][j], 0, 0, 0);
        };
        int cur = 0;
        read_frags(0, As[0] + a_off, Bs[0] + b_off, 0);
        for (int kt = 0; kt < nk; ++kt) {
            const bool more = kt + 1 < nk;
            const float* as = As[cur] + a_off;
            const float* bs = Bs[cur] + b_off;
#pragma unroll
            for (int kk = 0; kk < KS - 1; ++kk) {
                read_frags((kk + 1) & 1, as, bs, kk + 1);
                if (more) {
                    if (kk < LA::kPasses) LA::store_pass(ra, As[cur ^ 1], kk);
                    else if (kk < kStorePasses) LB::store_pass(rb, Bs[cur ^ 1], kk - LA::kPasses);
                }
                // pass p of an operand is requested one step after its registers went to LDS
                // (stage_sites moves the site along from the stage before, so a stage cannot
                // be requested twice: these requests stay behind the test for a further stage)
                if (kt + 2 < nk) {
                    if (kk == 1) stage_sites(j_lo + static_cast<long long>(kt + 2) * BK);
                    if (kk >= 1 && kk - 1 < LA::kPasses) load_a(kk - 1);
                    else if (kk - 1 >= LA::kPasses && kk - 1 < kStorePasses) load_b(kk - 1 - LA::kPasses);
                }
                __builtin_amdgcn_sched_barrier(0);
                mfma_step(kk & 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            __syncthreads();
            cur ^= 1;
            if (more) read_frags(0, As[cur] + a_off, Bs[cur] + b_off, 0);
            __builtin_amdgcn_sched_barrier(0);
            mfma_step((KS - 1) & 1);
        }
    }
#pragma unroll
    for (int i = 0; i < kTM; ++i) {
        const int row = m0 + (wm * kTM + i) * 32 + l32;
#pragma unroll
        for (int jn = 0; jn < TN; ++jn) {
            const int cbase = n0 + (wn * TN + jn) * 32 + 4 * h;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int col = cbase + 8 * (v / 4) + (v % 4);
                if (row < g.K && col < g.Cout) C[static_cast<long long>(col) * g.K + row] = acc[i][jn][v];
            }
        }
    }
}

// flipped weights for the input-gradient product: F(k', c) with k' = (co, ky', kx')
// holds W((c, kH-1-ky', kW-1-kx'), co); F is (C_out*kH*kW) x C_in, column-major
__global__ __launch_bounds__(kBlock) void conv_flip_weights_kernel(float* __restrict__ F, const float* __restrict__ Wt,
                                                                   int C_in, int C_out, int kH, int kW) {
    const int khw = kH * kW;
    const int K = C_in * khw, Kp = C_out * khw;
    const long long total = static_cast<long long>(Kp) * C_in;
    for (long long i = static_cast<long long>(blockIdx.x) * kBlock + threadIdx.x; i < total;
         i += static_cast<long long>(gridDim.x) * kBlock) {
        const int c = static_cast<int>(i / Kp);
        const int kp = static_cast<int>(i - static_cast<long long>(c) * Kp);
        const int co = kp / khw, r = kp - co * khw;
        const int ky = r / kW, kx = r - ky * kW;
        F[i] = Wt[static_cast<long long>(co) * K + c * khw + (kH - 1 - ky) * kW + (kW - 1 - kx)];
    }
}

// ── at most four output channels (the 3-channel output layer of the UNet) ────
// A 64-wide MFMA tile for three channels wastes twenty MFMA columns in twenty-one, and
// the weight gradients took the patch-matrix route (302 MB written and read).  With so few
// channels both products are a stream over the input, so they are plain vector code:
// forward 92 -> 57 us, weight gradients 204 -> 37 us at 64 -> 3 channels, 32 x 32,
// batch 128 (and the input gradients of a 3 -> 64 layer, which are a forward product
// with three output channels, 99 -> 58 us).
constexpr int kThinCout = 4;
constexpr int kThinPixels = 64;   // pixels per workgroup in the forward kernel: one wavefront wide

// Forward: a workgroup takes 64 consecutive output pixels; its four waves take a quarter
// of the input channels each (lanes along the pixels: 256-byte runs of an image row) and
// meet in LDS in a fixed order.  The weights sit in LDS as one float4 per patch row
// (the channels of that row, zero-filled), read as a broadcast.
__global__ __launch_bounds__(kBlock) void conv_thin_fwd_kernel(const float* __restrict__ in,
                                                               const float* __restrict__ Wt,
                                                               const float* __restrict__ bias,
                                                               float* __restrict__ out, ConvGeom g, int relu) {
    extern __shared__ __attribute__((aligned(16))) float thin_lds[];
    floatx4* wl = reinterpret_cast<floatx4*>(thin_lds);                 // [K]
    floatx4* red = wl + g.K;                                            // [3][64]
    for (int k = threadIdx.x; k < g.K; k += kBlock) {
        floatx4 w = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int co = 0; co < kThinCout; ++co)
            if (co < g.Cout) w[co] = Wt[static_cast<long long>(co) * g.K + k];
        wl[k] = w;
    }
    __syncthreads();
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const long long j = static_cast<long long>(blockIdx.x) * kThinPixels + lane;
    const bool live = j < g.J;
    const Site s = site_of(live ? j : 0, g);
    constexpr int NW = kBlock / kWave;
    const int c_per = (g.C + NW - 1) / NW;
    const int c_lo = wave * c_per, c_hi = (c_lo + c_per) < g.C ? (c_lo + c_per) : g.C;
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
    if (live) {
        for (int c = c_lo; c < c_hi; ++c) {
            const float* plane = in + s.base + static_cast<long long>(c) * g.HW;
            const floatx4* wc = wl + c * g.khw;
            for (int ky = 0; ky < g.kH; ++ky) {
                const bool row = static_cast<unsigned>(s.ih0 + ky) < static_cast<unsigned>(g.H);
                for (int kx = 0; kx < g.kW; ++kx) {
                    const bool ok = row && static_cast<unsigned>(s.iw0 + kx) < static_cast<unsigned>(g.W);
                    const float v = ok ? plane[ky * g.W + kx] : 0.0f;
                    const floatx4 w = wc[ky * g.kW + kx];
                    acc[0] += v * w[0]; acc[1] += v * w[1]; acc[2] += v * w[2]; acc[3] += v * w[3];
                }
            }
        }
    }
    if (wave > 0) red[(wave - 1) * kWave + lane] = acc;
    __syncthreads();
    if (wave == 0 && live) {
#pragma unroll
        for (int w = 0; w < NW - 1; ++w) {
            const floatx4 o = red[w * kWave + lane];
            acc[0] += o[0]; acc[1] += o[1]; acc[2] += o[2]; acc[3] += o[3];
        }
        const int p = s.oh * g.Wo + s.ow;
        float* dst = out + static_cast<long long>(s.n) * g.Cout * g.P + p;
#pragma unroll
        for (int co = 0; co < kThinCout; ++co) {
            if (co < g.Cout) {
                float r = acc[co];
                if (bias) r += bias[co];
                if (relu) r = r > 0.0f ? r : 0.0f;
                dst[static_cast<long long>(co) * g.P] = r;
            }
        }
    }
}

// Weight gradients for a KH x KW kernel: a workgroup takes one input channel and a
// chunk of the patch columns; a thread walks its pixels and keeps KH*KW*4 sums
// (tap x channel), which the workgroup adds up at the end; one partial result per
// chunk, summed afterwards in a fixed order.
template <int KH, int KW>
__global__ __launch_bounds__(kBlock) void conv_thin_dw_kernel(const float* __restrict__ in,
                                                              const float* __restrict__ t,
                                                              float* __restrict__ part, ConvGeom g,
                                                              long long j_chunk) {
    constexpr int KHW = KH * KW;
    constexpr int NW = kBlock / kWave;
    __shared__ float red[NW][KHW * kThinCout];
    const int c = blockIdx.x;
    const long long j_lo = static_cast<long long>(blockIdx.y) * j_chunk;
    const long long j_hi = (j_lo + j_chunk) < g.J ? (j_lo + j_chunk) : g.J;
    const long long CoP = static_cast<long long>(g.Cout) * g.P;
    float acc[KHW][kThinCout];
#pragma unroll
    for (int a = 0; a < KHW; ++a)
#pragma unroll
        for (int co = 0; co < kThinCout; ++co) acc[a][co] = 0.0f;
    for (long long j = j_lo + threadIdx.x; j < j_hi; j += kBlock) {
        const Site s = site_of(j, g);
        const float* tp = t + s.n * CoP + s.oh * g.Wo + s.ow;
        float tv[kThinCout];
#pragma unroll
        for (int co = 0; co < kThinCout; ++co) tv[co] = co < g.Cout ? tp[static_cast<long long>(co) * g.P] : 0.0f;
        const float* plane = in + s.base + static_cast<long long>(c) * g.HW;
#pragma unroll
        for (int ky = 0; ky < KH; ++ky) {
            const bool row = static_cast<unsigned>(s.ih0 + ky) < static_cast<unsigned>(g.H);
#pragma unroll
            for (int kx = 0; kx < KW; ++kx) {
                const bool ok = row && static_cast<unsigned>(s.iw0 + kx) < static_cast<unsigned>(g.W);
                const float v = ok ? plane[ky * g.W + kx] : 0.0f;
#pragma unroll
                for (int co = 0; co < kThinCout; ++co) acc[ky * KW + kx][co] += v * tv[co];
            }
        }
    }
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
    for (int a = 0; a < KHW; ++a)
#pragma unroll
        for (int co = 0; co < kThinCout; ++co) {
            const float v = wave_sum(acc[a][co]);
            if (lane == 0) red[wave][a * kThinCout + co] = v;
        }
    __syncthreads();
    if (threadIdx.x < KHW * kThinCout) {
        const int a = threadIdx.x / kThinCout, co = threadIdx.x % kThinCout;
        if (co < g.Cout) {
            float sum = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) sum += red[w][threadIdx.x];
            // partial result of this chunk: (K, C_out) column-major, row k = c*KHW + a
            part[static_cast<long long>(blockIdx.y) * g.K * g.Cout + static_cast<long long>(co) * g.K + c * KHW + a] = sum;
        }
    }
}

bool dims_ok(int C_in, int H_in, int W_in, int C_out, int kH, int kW, int pad_h, int pad_w, int sh, int sw, int H_out,
             int W_out, int N) {
    if (C_in <= 0 || H_in <= 0 || W_in <= 0 || C_out <= 0 || kH <= 0 || kW <= 0 || pad_h < 0 || pad_w < 0 || sh <= 0 ||
        sw <= 0 || H_out <= 0 || W_out <= 0 || N <= 0)
        return false;
    // every index product must stay inside the 32-bit arithmetic the kernels use per image
    const long long chw = static_cast<long long>(C_in) * H_in * W_in, cop = static_cast<long long>(C_out) * H_out * W_out;
    const long long j = static_cast<long long>(H_out) * W_out * N, k = static_cast<long long>(C_in) * kH * kW;
    if (!(chw < (1ll << 30) && cop < (1ll << 30) && j < (1ll << 31) && k < (1ll << 24))) return false;
    // the patch grid must be the one the geometry implies (or smaller): out, t and dx are sized
    // from it by the caller, and a larger grid would be written past their end
    const long long span_h = static_cast<long long>(H_in) + 2ll * pad_h - kH, span_w = static_cast<long long>(W_in) + 2ll * pad_w - kW;
    if (span_h < 0 || span_w < 0) return false;
    return H_out <= span_h / sh + 1 && W_out <= span_w / sw + 1;
}

// What jzhip_conv2d_backward_data needs beyond dims_ok: stride 1, the padding of a "full"
// correlation non-negative, the input grid exactly the one a stride-1 layer maps to the
// output grid, and the flipped weights small enough for the workspace.
bool data_grad_ok(int C_in, int H_in, int W_in, int C_out, int kH, int kW, int pad_h, int pad_w, int sh, int sw,
                  int H_out, int W_out) {
    if (sh != 1 || sw != 1) return false;
    if (pad_h > kH - 1 || pad_w > kW - 1) return false;
    if (H_in != H_out + kH - 1 - 2 * pad_h || W_in != W_out + kW - 1 - 2 * pad_w) return false;
    return static_cast<size_t>(C_out) * kH * kW * C_in <= kWorkspaceFloats;
}

// JZHIP_CONV_FWD_STRIP=0 keeps the general forward kernel for every shape (for comparisons)
// JZHIP_CONV_FEW=0 keeps the general kernels for layers with few input channels (for comparisons)
bool few_enabled() {
    static const bool on = [] {
        const char* e = std::getenv("JZHIP_CONV_FEW");
        return !(e && e[0] == '0');
    }();
    return on;
}

bool fwd_strip_enabled() {
    static const bool on = [] {
        const char* e = std::getenv("JZHIP_CONV_FWD_STRIP");
        return !(e && e[0] == '0');
    }();
    return on;
}

int launch_fwd(const float* in, const float* Wt, const float* bias, float* out, const ConvGeom& g, int relu) {
    if (g.Cout <= kThinCout && g.C >= 8) {
        const size_t lds = (static_cast<size_t>(g.K) + 3 * kWave) * sizeof(floatx4);
        const long long blocks = (g.J + kThinPixels - 1) / kThinPixels;
        if (lds <= 48 * 1024 && blocks <= 0x7fffffffll) {
            conv_thin_fwd_kernel<<<static_cast<unsigned>(blocks), kBlock, lds, stream()>>>(in, Wt, bias, out, g, relu);
            return launch_rc();
        }
    }
    // the largest tile that still gives every CU two workgroups; 64-row tiles for layers
    // with few output pixels (8x8 grids), 64-channel tiles when that is not enough
    const long long want = 2ll * num_cus();
    auto tiles = [&](int bm, int bn) { return ((g.J + bm - 1) / bm) * ((g.Cout + bn - 1) / bn); };
    int TM = 2, TN = g.Cout > 64 ? 2 : 1;
    if (tiles(64 * TM, 64 * TN) < want) TM = 1;
    if (tiles(64 * TM, 64 * TN) < want) TN = 1;
    const int BM = 64 * TM, BN = 64 * TN;
    const int tiles_n = (g.Cout + BN - 1) / BN;
    const long long total = tiles(BM, BN);
    if (total > 0x7fffffffll) return -1;
    const bool fastb = g.K % BK == 0 && g.Cout % BN == 0 && aligned16(Wt);
    const unsigned grid = static_cast<unsigned>(total);
    hipStream_t s = stream();
    // tap table: kH*kW one-hot bits in a word, K (rounded up to a stage) entries of 8 bytes in LDS
    const size_t tab_bytes = static_cast<size_t>((g.K + BK - 1) / BK * BK) * sizeof(int2);
    const long long in_bytes = static_cast<long long>(g.N) * g.CHW * static_cast<long long>(sizeof(float));
    const bool tab = g.khw <= 32 && tab_bytes <= 24 * 1024 && g.K > 2 * BK && in_bytes <= kBufferMaxBytes;
    const unsigned in_b = tab ? static_cast<unsigned>(in_bytes) : 0u;
#define JZ_CONV_FWD_T(TMV, TNV, FB)                                                                              \
    do {                                                                                                         \
        if (tab) conv_fwd_kernel<TMV, TNV, FB, true><<<grid, kBlock, tab_bytes, s>>>(in, Wt, bias, out, g, relu, tiles_n, in_b); \
        else conv_fwd_kernel<TMV, TNV, FB, false><<<grid, kBlock, 0, s>>>(in, Wt, bias, out, g, relu, tiles_n, in_b);  \
    } while (0)
#define JZ_CONV_FWD(TMV, TNV)                \
    do {                                     \
        if (fastb) JZ_CONV_FWD_T(TMV, TNV, true); \
        else JZ_CONV_FWD_T(TMV, TNV, false); \
    } while (0)
    if (TM == 2 && TN == 2) JZ_CONV_FWD(2, 2);
    else if (TM == 2) JZ_CONV_FWD(2, 1);
    else if (TN == 2) JZ_CONV_FWD(1, 2);
    else JZ_CONV_FWD(1, 1);
#undef JZ_CONV_FWD_T
#undef JZ_CONV_FWD
    return launch_rc();
}

// ── transposed convolution as stride-1 convolutions, one per residue class ───
// out(co, oy, ox) = bias(co) + sum over (ci, ky, kx) with (oy + pad - ky) divisible by the
// stride of x(ci, (oy + pad - ky)/s, (ox + pad - kx)/s) * W((co, ky, kx), ci).
// Output rows with the same residue (oy + pad) mod s use the same taps ky = r, r + s, ...
// and consecutive input rows: for those rows the sum is a stride-1 convolution of x with
// the sub-kernel made of these taps (in reversed order), on a patch grid that maps to every
// s-th output row.  The s_h * s_w classes partition both the output pixels and the taps,
// so together they do exactly the multiply-adds of the scatter formulation
// (ml/layer.hpp:1770-1790, 2112-2160) and write every output pixel once.
struct ClassAxis {
    int o0;      // first output index of the class
    int taps;    // sub-kernel extent
    int r;       // first tap: k = r + s*m
    int pad;     // padding of the stride-1 sub-convolution (may be negative)
    int count;   // output indices in the class
};
ClassAxis class_axis(int o0, int k, int s, int pad, int out) {
    ClassAxis a;
    a.o0 = o0;
    a.r = (o0 + pad) % s;
    a.taps = a.r < k ? (k - a.r + s - 1) / s : 0;
    const int q0 = (o0 + pad) / s;           // input index of tap m = 0 for the class's first output
    a.pad = (a.taps - 1) - q0;
    a.count = o0 < out ? (out - o0 + s - 1) / s : 0;
    return a;
}

// Wsub of class (cy, cx): (K_sub, C_out) column-major, row (ci, ky2, kx2) holds the tap
// ky = ry + sh*(ty - 1 - ky2), kx likewise; classes behind each other in (cy, cx) order.
__global__ __launch_bounds__(kBlock) void convtrans_pack_kernel(float* __restrict__ packed, const float* __restrict__ W,
                                                                int C_in, int C_out, int kH, int kW, int sh, int sw,
                                                                int pad_h, int pad_w, long long total) {
    const long long e = static_cast<long long>(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= total) return;
    // source element ((co, ky, kx), ci) of the (C_out*kH*kW, C_in) column-major matrix
    const int rows = C_out * kH * kW;
    const int ci = static_cast<int>(e / rows);
    int r = static_cast<int>(e - static_cast<long long>(ci) * rows);
    const int kx = r % kW;
    r /= kW;
    const int ky = r % kH;
    const int co = r / kH;
    // the class whose first tap has this residue, and the classes before it
    long long off = 0;
    int ty = 0, tx = 0;
    for (int cy = 0; cy < sh; ++cy)
        for (int cx = 0; cx < sw; ++cx) {
            const int ry = (cy + pad_h) % sh, rx = (cx + pad_w) % sw;
            const int ny = ry < kH ? (kH - ry + sh - 1) / sh : 0, nx = rx < kW ? (kW - rx + sw - 1) / sw : 0;
            if (ry == ky % sh && rx == kx % sw) {
                ty = ny;
                tx = nx;
                cy = sh;     // leave both loops
                break;
            }
            off += static_cast<long long>(C_in) * ny * nx * C_out;
        }
    const int ky2 = ty - 1 - ky / sh, kx2 = tx - 1 - kx / sw;
    const long long Ksub = static_cast<long long>(C_in) * ty * tx;
    packed[off + static_cast<long long>(co) * Ksub + (static_cast<long long>(ci) * ty + ky2) * tx + kx2] = W[e];
}

bool transposed_ok(int C_in, int H_in, int W_in, int C_out, int kH, int kW, int pad_h, int pad_w, int sh, int sw, int H_out,
                   int W_out, int N) {
    if (C_in <= 0 || H_in <= 0 || W_in <= 0 || C_out <= 0 || kH <= 0 || kW <= 0 || pad_h < 0 || pad_w < 0 || sh <= 0 ||
        sw <= 0 || H_out <= 0 || W_out <= 0 || N <= 0)
        return false;
    if (sh * sw > kMaxClasses) return false;
    const long long chw = static_cast<long long>(C_in) * H_in * W_in, cop = static_cast<long long>(C_out) * H_out * W_out;
    const long long j = static_cast<long long>(H_in + kH) * (W_in + kW) * N, k = static_cast<long long>(C_in) * kH * kW;
    if (!(chw < (1ll << 30) && cop < (1ll << 30) && j < (1ll << 31) && k < (1ll << 24))) return false;
    if (static_cast<size_t>(k) * C_out > kWorkspaceFloats) return false;
    // the output may be the natural extent (H_in-1)*s - 2*pad + kH or up to s-1 rows more (the
    // input gradient of a strided convolution whose last rows no patch reached from below)
    const long long nat_h = static_cast<long long>(H_in - 1) * sh - 2ll * pad_h + kH;
    const long long nat_w = static_cast<long long>(W_in - 1) * sw - 2ll * pad_w + kW;
    if (!(H_out <= nat_h + sh - 1 && W_out <= nat_w + sw - 1)) return false;
    return kH >= sh && kW >= sw;   // every residue class needs at least one tap
}

int launch_transposed(const float* x, const float* W, const float* bias, float* out, int C_in, int H_in, int W_in,
                      int C_out, int kH, int kW, int pad_h, int pad_w, int sh, int sw, int H_out, int W_out, int N,
                      int relu) {
    float* packed = workspace();
    if (!packed) return -2;
    hipStream_t s = stream();
    const long long wcount = static_cast<long long>(C_in) * kH * kW * C_out;
    convtrans_pack_kernel<<<grid_cover(static_cast<size_t>(wcount), kBlock), kBlock, 0, s>>>(packed, W, C_in, C_out, kH, kW,
                                                                                         sh, sw, pad_h, pad_w, wcount);
    ConvClasses cls;
    int ncls = 0;
    long long off = 0, max_j = 0;
    int max_k = 0, max_khw = 0;
    bool k_aligned = true, k_long = true;
    for (int cy = 0; cy < sh; ++cy)
        for (int cx = 0; cx < sw; ++cx) {
            const ClassAxis ay = class_axis(cy, kH, sh, pad_h, H_out), ax = class_axis(cx, kW, sw, pad_w, W_out);
            if (ay.taps <= 0 || ax.taps <= 0) return -1;   // kernel extent below the stride: refused by the entry point
            // a class without output pixels (an output narrower than the stride) keeps its weights' place and runs no tile
            ConvGeom g = make_geom(C_in, H_in, W_in, ay.taps, ax.taps, ay.pad, ax.pad, 1, 1, ay.count > 0 ? ay.count : 1,
                                   ax.count > 0 ? ax.count : 1, N, C_out);
            g.w_off = off;
            off += static_cast<long long>(C_in) * ay.taps * ax.taps * C_out;
            if (ay.count <= 0 || ax.count <= 0) g.J = 0;
            g.out_sh = sh; g.out_sw = sw; g.out_oh0 = cy; g.out_ow0 = cx; g.out_W = W_out; g.out_P = H_out * W_out;
            cls.g[ncls++] = g;
            if (g.J > max_j) max_j = g.J;
            if (g.K > max_k) max_k = g.K;
            if (g.khw > max_khw) max_khw = g.khw;
            k_aligned = k_aligned && g.K % BK == 0 && g.w_off % 4 == 0;
            k_long = k_long && g.K > 2 * BK;
        }
    // classes with more taps first: the workgroups of the longest K walks start earliest
    for (int a = 1; a < ncls; ++a)
        for (int b = a; b > 0 && cls.g[b].K > cls.g[b - 1].K; --b) std::swap(cls.g[b], cls.g[b - 1]);
    for (int c = ncls; c < kMaxClasses; ++c) cls.g[c] = cls.g[0];
    // tile choice as in launch_fwd, over all classes together
    const long long want = 2ll * num_cus();
    auto tiles = [&](int bm, int bn) { return ((max_j + bm - 1) / bm) * ((C_out + bn - 1) / bn) * ncls; };
    int TM = 2, TN = C_out > 64 ? 2 : 1;
    if (tiles(64 * TM, 64 * TN) < want) TM = 1;
    if (tiles(64 * TM, 64 * TN) < want) TN = 1;
    const int BM = 64 * TM, BN = 64 * TN;
    const int tiles_n = (C_out + BN - 1) / BN;
    const long long per_class = ((max_j + BM - 1) / BM) * tiles_n;
    if (per_class > 0x7fffffffll) return -1;
    const bool fastb = k_aligned && C_out % BN == 0 && aligned16(packed);
    const size_t tab_bytes = static_cast<size_t>((max_k + BK - 1) / BK * BK) * sizeof(int2);
    const long long in_bytes = static_cast<long long>(N) * C_in * H_in * W_in * static_cast<long long>(sizeof(float));
    const bool tab = max_khw <= 32 && tab_bytes <= 24 * 1024 && k_long && in_bytes <= kBufferMaxBytes;
    const unsigned in_b = tab ? static_cast<unsigned>(in_bytes) : 0u;
    const dim3 grid(static_cast<unsigned>(per_class), ncls);
#define JZ_CONVT_T(TMV, TNV, FB)                                                                                   \
    do {                                                                                                           \
        if (tab) conv_fwd_kernel<TMV, TNV, FB, true, true><<<grid, kBlock, tab_bytes, s>>>(x, packed, bias, out, cls, relu, tiles_n, in_b); \
        else conv_fwd_kernel<TMV, TNV, FB, false, true><<<grid, kBlock, 0, s>>>(x, packed, bias, out, cls, relu, tiles_n, in_b);  \
    } while (0)
#define JZ_CONVT(TMV, TNV)                   \
    do {                                     \
        if (fastb) JZ_CONVT_T(TMV, TNV, true); \
        else JZ_CONVT_T(TMV, TNV, false);    \
    } while (0)
    if (TM == 2 && TN == 2) JZ_CONVT(2, 2);
    else if (TM == 2) JZ_CONVT(2, 1);
    else if (TN == 2) JZ_CONVT(1, 2);
    else JZ_CONVT(1, 1);
#undef JZ_CONVT_T
#undef JZ_CONVT
    return launch_rc();
}

}  // namespace
}  // namespace jz

using namespace jz;

JZ_API int jzhip_conv2d_transposed(const float* x, const float* weights, const float* bias, float* out, int C_in,
                                   int H_in, int W_in, int C_out, int kH, int kW, int pad_h, int pad_w, int stride_h,
                                   int stride_w, int H_out, int W_out, int N, int relu) {
    if (!x || !weights || !out) return -1;
    if (!transposed_ok(C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N)) return -1;
    return launch_transposed(x, weights, bias, out, C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w,
                             H_out, W_out, N, relu ? 1 : 0);
}

JZ_API int jzhip_conv2d_forward(const float* input, const float* weights, const float* bias, float* out, int C_in,
                                int H_in, int W_in, int C_out, int kH, int kW, int pad_h, int pad_w, int stride_h,
                                int stride_w, int H_out, int W_out, int N, int relu) {
    if (!input || !weights || !out) return -1;
    if (!dims_ok(C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N)) return -1;
    if (fwd_strip_enabled() &&
        conv_fwd_strip_ok(input, out, C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N))
        return launch_conv_fwd_strip(input, weights, bias, out, C_in, H_in, W_in, C_out, N, relu ? 1 : 0, 0);
    if (few_enabled() && C_out >= 8 &&
        conv_few_ok(input, out, C_in, H_in, W_in, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out))
        return launch_conv_few_fwd(input, weights, bias, out, C_in, H_in, W_in, C_out, N, relu ? 1 : 0);
    const ConvGeom g = make_geom(C_in, H_in, W_in, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N, C_out);
    return launch_fwd(input, weights, bias, out, g, relu ? 1 : 0);
}

JZ_API int jzhip_conv2d_backward_weights(const float* input, const float* t, float* dW, int C_in, int H_in, int W_in,
                                         int C_out, int kH, int kW, int pad_h, int pad_w, int stride_h, int stride_w,
                                         int H_out, int W_out, int N) {
    if (!input || !t || !dW) return -1;
    if (!dims_ok(C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N)) return -1;
    if (few_enabled() && C_out >= 8 &&
        conv_few_ok(input, t, C_in, H_in, W_in, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out))
        return launch_conv_few_dw(input, t, dW, C_in, H_in, W_in, C_out, N);
    const ConvGeom g = make_geom(C_in, H_in, W_in, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N, C_out);
    if (C_out <= kThinCout && kH == 3 && kW == 3 && C_in <= 65535) {
        // chunks of the patch columns so that channels x chunks gives every CU several workgroups
        const long long cus = num_cus();
        long long chunks = (8 * cus + C_in - 1) / C_in;
        if (chunks > g.J / 1024) chunks = g.J / 1024;
        if (chunks < 1) chunks = 1;
        const long long per = static_cast<long long>(g.K) * C_out;
        while (chunks > 1 && per * chunks > static_cast<long long>(kWorkspaceFloats)) --chunks;
        const long long j_chunk = (g.J + chunks - 1) / chunks;
        chunks = (g.J + j_chunk - 1) / j_chunk;
        if (chunks <= 65535) {
            float* part = dW;
            if (chunks > 1) {
                part = workspace();
                if (!part) return -2;
            }
            conv_thin_dw_kernel<3, 3><<<dim3(C_in, static_cast<unsigned>(chunks)), kBlock, 0, stream()>>>(input, t, part, g,
                                                                                                           j_chunk);
            if (chunks > 1)
                launch_splitk_reduce(dW, part, g.K, C_out, static_cast<size_t>(g.K), static_cast<int>(chunks), 1.0f, 0.0f);
            return launch_rc();
        }
    }
    {
        // JZHIP_CONV_DW_STRIP=0 keeps the general kernel for every shape (for comparisons)
        static const bool strip_on = [] {
            const char* e = std::getenv("JZHIP_CONV_DW_STRIP");
            return !(e && e[0] == '0');
        }();
        if (strip_on && conv_dw_strip_ok(input, t, C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out,
                                         W_out, N))
            return launch_conv_dw_strip(input, t, dW, C_in, H_in, W_in, C_out, N);
    }
    const bool wide = C_out > 64;
    const int BN = wide ? 128 : 64;
    const int tiles_n = (C_out + BN - 1) / BN, tiles_m = (g.K + 127) / 128;
    const long long tiles = static_cast<long long>(tiles_m) * tiles_n;
    // chunks of the patch-column range: enough workgroups for two to four per CU, a multiple of 8
    // so that an XCD keeps to its own chunks, at least 16 stages each
    const long long cus = num_cus();
    // (four per CU while the partial results stay small: 167 against 202 us at 576 x 64;
    // with larger outputs the extra partial sums cost more than the occupancy gains)
    const long long per_cu = static_cast<long long>(g.K) * C_out <= 100000 ? 4 : 2;
    long long splits = (per_cu * cus + tiles - 1) / tiles;
    splits = splits <= 2 ? splits : splits <= 4 ? 4 : (splits + 7) / 8 * 8;
    const long long per = static_cast<long long>(g.K) * C_out;
    // at least 16 stages per chunk, 6 where a partial tile set is small (288 x 64: 42 -> 31 us with
    // the sum of the partial results included; 576 x 128 loses with anything below 16)
    const int min_stages = per <= 20000 ? 6 : 16;
    while (splits > 1 && (g.J / splits < min_stages * BK || per * splits > static_cast<long long>(kWorkspaceFloats)))
        splits = splits > 8 ? splits - 8 : splits / 2;
    if (splits < 1) splits = 1;
    long long j_chunk = ((g.J + splits - 1) / splits + BK - 1) / BK * BK;
    splits = (g.J + j_chunk - 1) / j_chunk;
    if (splits > 65535 || tiles > 0x7fffffffll) return -1;
    float* part = dW;
    if (splits > 1) {
        part = workspace();
        if (!part) return -2;
    }
    const int t_vec = (g.P % 4 == 0) && aligned16(t);
    dim3 grid(static_cast<unsigned>(tiles), static_cast<unsigned>(splits));
    hipStream_t s = stream();
    const long long in_bytes = static_cast<long long>(N) * g.CHW * static_cast<long long>(sizeof(float));
    // inputs of up to 2 GiB are read through a buffer resource (padding by the range check);
    // larger ones take the loaders with a branch per element
    const unsigned in_b = in_bytes <= kBufferMaxBytes ? static_cast<unsigned>(in_bytes) : 0u;
    const bool quad = W_out % 4 == 0 && in_b != 0;
    if (wide && quad) conv_dw_kernel<2, true><<<grid, kBlock, 0, s>>>(input, t, part, g, tiles_n, j_chunk, t_vec, in_b);
    else if (wide) conv_dw_kernel<2, false><<<grid, kBlock, 0, s>>>(input, t, part, g, tiles_n, j_chunk, t_vec, in_b);
    else if (quad) conv_dw_kernel<1, true><<<grid, kBlock, 0, s>>>(input, t, part, g, tiles_n, j_chunk, t_vec, in_b);
    else conv_dw_kernel<1, false><<<grid, kBlock, 0, s>>>(input, t, part, g, tiles_n, j_chunk, t_vec, in_b);
    if (splits > 1) launch_splitk_reduce(dW, part, g.K, C_out, static_cast<size_t>(g.K), static_cast<int>(splits), 1.0f, 0.0f);
    return launch_rc();
}

JZ_API int jzhip_conv2d_backward_data(const float* t, const float* weights, float* dx, int C_in, int H_in, int W_in,
                                      int C_out, int kH, int kW, int pad_h, int pad_w, int stride_h, int stride_w,
                                      int H_out, int W_out, int N) {
    if (!t || !weights || !dx) return -1;
    if (!dims_ok(C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N)) return -1;
    if (!data_grad_ok(C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out)) return -1;
    // the product: t (C_out channels on the H_out x W_out grid) against the mirrored taps, padding k-1-pad
    if (fwd_strip_enabled() && conv_fwd_strip_ok(t, dx, C_out, H_out, W_out, C_in, kH, kW, kH - 1 - pad_h, kW - 1 - pad_w, 1, 1,
                                                 H_in, W_in, N))
        return launch_conv_fwd_strip(t, weights, nullptr, dx, C_out, H_out, W_out, C_in, N, 0, 1);
    const size_t wcount = static_cast<size_t>(C_out) * kH * kW * C_in;
    float* flipped = workspace();
    if (!flipped) return -2;
    hipStream_t s = stream();
    conv_flip_weights_kernel<<<grid_for(wcount, kBlock, 4), kBlock, 0, s>>>(flipped, weights, C_in, C_out, kH, kW);
    // a stride-1 convolution of t (C_out channels on the H_out x W_out grid) with the
    // flipped taps and padding k-1-pad lands on the H_in x W_in grid
    const ConvGeom g = make_geom(C_out, H_out, W_out, kH, kW, kH - 1 - pad_h, kW - 1 - pad_w, 1, 1, H_in, W_in, N, C_in);
    return launch_fwd(t, flipped, nullptr, dx, g, 0);
}

JZ_API int jzhip_conv2d_check(int which, int C_in, int H_in, int W_in, int C_out, int kH, int kW, int pad_h, int pad_w,
                              int stride_h, int stride_w, int H_out, int W_out, int N) {
    if (which == 3)
        return transposed_ok(C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N) ? 0 : -1;
    if (which == 4) {
        // backward_weights with the strip kernel (operands assumed 16-byte aligned)
        const float* aligned = reinterpret_cast<const float*>(uintptr_t(256));
        return dims_ok(C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N) &&
                       conv_dw_strip_ok(aligned, aligned, C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w,
                                        H_out, W_out, N)
                   ? 0
                   : -1;
    }
    if (which == 5 || which == 6) {
        // forward (5) / backward_data (6) with the kernel that stages image strips
        const float* aligned = reinterpret_cast<const float*>(uintptr_t(256));
        if (!dims_ok(C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N)) return -1;
        if (which == 5)
            return conv_fwd_strip_ok(aligned, aligned, C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out,
                                     W_out, N)
                       ? 0
                       : -1;
        return data_grad_ok(C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out) &&
                       conv_fwd_strip_ok(aligned, aligned, C_out, H_out, W_out, C_in, kH, kW, kH - 1 - pad_h, kW - 1 - pad_w, 1, 1,
                                         H_in, W_in, N)
                   ? 0
                   : -1;
    }
    if (which < 0 || which > 2) return -1;
    if (!dims_ok(C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N)) return -1;
    if (which == 2 && !data_grad_ok(C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out))
        return -1;
    return 0;
}
