// Two-dimensional elementwise kernels that honour per-operand transpose
// flags and leading dimensions: the logical-index semantics of the CPU oracle
// (cpp/core.hpp:414-449, cpp/matrix.hpp:93-150,428-474, cpp/core.hpp:353-373).
//
// Everything is expressed in the *output's physical frame*: the output is an
// R x C column-major block with leading dimension ldo; an operand whose
// transpose flag differs from the output's is "relatively transposed" and its
// element (r,c) lives at x[r*ldx + c].  Such operands are staged through a
// padded LDS tile so that both the global read and the global write are
// coalesced along the contiguous dimension of their own buffer.
#include "common.hpp"

namespace jz {
namespace {

constexpr int kTile = 32;
constexpr int kRowsPerPass = 8;  // block = 32 x 8 threads, 4 passes per tile

enum : int { kOpCopy = 0, kOpAxpby = 1, kOpHadamard = 2 };

template <int OP>
__global__ __launch_bounds__(kTile* kRowsPerPass) void ew2d_kernel(
    float* out, size_t ldo, const float* a, size_t lda, int rel_a, const float* b, size_t ldb,
    int rel_b, size_t R, size_t C, unsigned tiles_r, float s1, float s2) {
    __shared__ float ta[kTile][kTile + 1];
    __shared__ float tb[kTile][kTile + 1];
    const unsigned tile = blockIdx.x;
    const size_t r0 = static_cast<size_t>(tile % tiles_r) * kTile;
    const size_t c0 = static_cast<size_t>(tile / tiles_r) * kTile;
    const int tx = threadIdx.x % kTile;
    const int ty = threadIdx.x / kTile;

    if (rel_a) {
#pragma unroll
        for (int k = 0; k < kTile; k += kRowsPerPass) {
            const size_t r = r0 + ty + k, c = c0 + tx;
            if (r < R && c < C) ta[ty + k][tx] = a[r * lda + c];
        }
    }
    if (OP != kOpCopy && rel_b) {
#pragma unroll
        for (int k = 0; k < kTile; k += kRowsPerPass) {
            const size_t r = r0 + ty + k, c = c0 + tx;
            if (r < R && c < C) tb[ty + k][tx] = b[r * ldb + c];
        }
    }
    if (rel_a || (OP != kOpCopy && rel_b)) __syncthreads();

#pragma unroll
    for (int k = 0; k < kTile; k += kRowsPerPass) {
        const int cl = ty + k;
        const size_t r = r0 + tx, c = c0 + cl;
        if (r < R && c < C) {
            const float va = rel_a ? ta[tx][cl] : a[c * lda + r];
            float res;
            if constexpr (OP == kOpCopy) {
                res = va;
            } else {
                const float vb = rel_b ? tb[tx][cl] : b[c * ldb + r];
                res = (OP == kOpAxpby) ? (s1 * va + s2 * vb) : (va * vb);
            }
            out[c * ldo + r] = res;
        }
    }
}

// float4 form of the kernel above for 16-byte aligned operands whose extents and
// leading dimensions are multiples of 4: 64x64 tiles, every global access a
// float4, relatively transposed operands turned in LDS (pitch 65).
constexpr int kTileV = 64;
template <int OP, bool NT>
__global__ __launch_bounds__(kBlock) void ew2d_vec_kernel(
    float* out, size_t ldo, const float* a, size_t lda, int rel_a, const float* b, size_t ldb,
    int rel_b, size_t R, size_t C, unsigned tiles_r, float s1, float s2) {
    __shared__ float ta[kTileV][kTileV + 1];
    __shared__ float tb[OP == kOpCopy ? 1 : kTileV][kTileV + 1];
    // Diagonal tile order: consecutive workgroups step along the rows and the
    // columns at once.  With a power-of-two leading dimension, tiles that differ
    // in one index only are a multiple of 2 MB apart in the transposed operand
    // and land on the same memory channels.
    const unsigned tile = blockIdx.x;
    const unsigned ti = tile % tiles_r, tj0 = tile / tiles_r;
    const unsigned tiles_c = gridDim.x / tiles_r;
    const size_t r0 = static_cast<size_t>(ti) * kTileV;
    const size_t c0 = static_cast<size_t>((tj0 + ti) % tiles_c) * kTileV;
    const int q = threadIdx.x % 16;    // float4 slot along the contiguous index
    const int l = threadIdx.x / 16;    // line inside a pass of 16
    auto stage = [&](float (*t)[kTileV + 1], const float* x, size_t ldx) {
#pragma unroll
        for (int k = 0; k < kTileV; k += 16) {
            const size_t r = r0 + l + k, c = c0 + 4 * q;
            if (r < R && c < C) {
                const float4 v = load4<NT>(x + r * ldx + c);
                float* d = &t[l + k][4 * q];
                d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
            }
        }
    };
    if (rel_a) stage(ta, a, lda);
    if constexpr (OP != kOpCopy) {
        if (rel_b) stage(tb, b, ldb);
    }
    if (rel_a || (OP != kOpCopy && rel_b)) __syncthreads();
#pragma unroll
    for (int k = 0; k < kTileV; k += 16) {
        const int cl = l + k;
        const size_t r = r0 + 4 * q, c = c0 + cl;
        if (r < R && c < C) {
            float4 va;
            if (rel_a) va = make_float4(ta[4 * q][cl], ta[4 * q + 1][cl], ta[4 * q + 2][cl], ta[4 * q + 3][cl]);
            else va = load4<NT>(a + c * lda + r);
            float4 res = va;
            if constexpr (OP != kOpCopy) {
                float4 vb;
                if (rel_b) vb = make_float4(tb[4 * q][cl], tb[4 * q + 1][cl], tb[4 * q + 2][cl], tb[4 * q + 3][cl]);
                else vb = load4<NT>(b + c * ldb + r);
                if constexpr (OP == kOpAxpby) {
                    res.x = s1 * va.x + s2 * vb.x; res.y = s1 * va.y + s2 * vb.y;
                    res.z = s1 * va.z + s2 * vb.z; res.w = s1 * va.w + s2 * vb.w;
                } else {
                    res.x = va.x * vb.x; res.y = va.y * vb.y; res.z = va.z * vb.z; res.w = va.w * vb.w;
                }
            }
            store4<NT>(out + c * ldo + r, res);
        }
    }
}

// No operand is transposed relative to the output (a row block of a vstack, a slice, an
// addition of two sub-blocks): nothing has to be turned, so a wavefront takes 256
// consecutive rows of one column (1 KB runs on every operand instead of the 256 B runs of
// the 64 x 64 tile) and a workgroup 256 rows x 16 columns.
constexpr int kStripRows = 256, kStripCols = 16;
template <int OP, bool NT>
__global__ __launch_bounds__(kBlock) void ew2d_strip_kernel(float* out, size_t ldo, const float* a, size_t lda,
                                                            const float* b, size_t ldb, size_t R, size_t C,
                                                            unsigned strips_r, float s1, float s2) {
    const unsigned sr = blockIdx.x % strips_r, sc = blockIdx.x / strips_r;
    const size_t r = static_cast<size_t>(sr) * kStripRows + 4 * (threadIdx.x % kWave);
    if (r >= R) return;
    const size_t c0 = static_cast<size_t>(sc) * kStripCols + threadIdx.x / kWave;
#pragma unroll
    for (int k = 0; k < kStripCols; k += kBlock / kWave) {
        const size_t c = c0 + k;
        if (c < C) {
            const float4 va = load4<NT>(a + c * lda + r);
            float4 res = va;
            if constexpr (OP != kOpCopy) {
                const float4 vb = load4<NT>(b + c * ldb + r);
                if constexpr (OP == kOpAxpby) {
                    res.x = s1 * va.x + s2 * vb.x; res.y = s1 * va.y + s2 * vb.y;
                    res.z = s1 * va.z + s2 * vb.z; res.w = s1 * va.w + s2 * vb.w;
                } else {
                    res.x = va.x * vb.x; res.y = va.y * vb.y; res.z = va.z * vb.z; res.w = va.w * vb.w;
                }
            }
            store4<NT>(out + c * ldo + r, res);
        }
    }
}

template <int OP>
int launch2d(float* out, size_t ldo, const float* a, size_t lda, int rel_a, const float* b,
             size_t ldb, int rel_b, size_t R, size_t C, float s1, float s2) {
    if (R == 0 || C == 0) return 0;
    const bool vec = R % 4 == 0 && C % 4 == 0 && ldo % 4 == 0 && lda % 4 == 0 && aligned16(out) && aligned16(a) &&
                     (OP == kOpCopy || (ldb % 4 == 0 && aligned16(b)));
    const bool past_cache = streams_past_cache((OP == kOpCopy ? 2 : 3) * R * C * sizeof(float));
    if (vec && !rel_a && (OP == kOpCopy || !rel_b) && R >= 128) {
        const size_t sr = (R + kStripRows - 1) / kStripRows, sc = (C + kStripCols - 1) / kStripCols;
        if (sr * sc <= 0x7fffffffull) {
            if (past_cache)
                ew2d_strip_kernel<OP, true><<<static_cast<unsigned>(sr * sc), kBlock, 0, stream()>>>(
                    out, ldo, a, lda, b, ldb, R, C, static_cast<unsigned>(sr), s1, s2);
            else
                ew2d_strip_kernel<OP, false><<<static_cast<unsigned>(sr * sc), kBlock, 0, stream()>>>(
                    out, ldo, a, lda, b, ldb, R, C, static_cast<unsigned>(sr), s1, s2);
            return launch_rc();
        }
    }
    if (vec) {
        const size_t tr = (R + kTileV - 1) / kTileV, tc = (C + kTileV - 1) / kTileV;
        if (tr * tc > 0x7fffffffull) return -1;
        if (past_cache)
            ew2d_vec_kernel<OP, true><<<static_cast<unsigned>(tr * tc), kBlock, 0, stream()>>>(
                out, ldo, a, lda, rel_a, b, ldb, rel_b, R, C, static_cast<unsigned>(tr), s1, s2);
        else
            ew2d_vec_kernel<OP, false><<<static_cast<unsigned>(tr * tc), kBlock, 0, stream()>>>(
                out, ldo, a, lda, rel_a, b, ldb, rel_b, R, C, static_cast<unsigned>(tr), s1, s2);
        return launch_rc();
    }
    const size_t tiles_r = (R + kTile - 1) / kTile;
    const size_t tiles_c = (C + kTile - 1) / kTile;
    if (tiles_r * tiles_c > 0x7fffffffull) return -1;
    ew2d_kernel<OP><<<static_cast<unsigned>(tiles_r * tiles_c), kTile * kRowsPerPass, 0, stream()>>>(
        out, ldo, a, lda, rel_a, b, ldb, rel_b, R, C, static_cast<unsigned>(tiles_r), s1, s2);
    return launch_rc();
}

// Shared front end of axpby2d / hadamard2d.  rows/cols are logical.
template <int OP>
int binary2d(float* out, int ldo, int trans_o, const float* a, int lda, int trans_a,
             const float* b, int ldb, int trans_b, int rows, int cols, float s1, float s2) {
    if (rows < 0 || cols < 0) return -1;
    if (rows == 0 || cols == 0) return 0;
    if (!out || !a || !b) return -1;
    // physical extent of the output block
    const size_t R = trans_o ? cols : rows;
    const size_t C = trans_o ? rows : cols;
    if (ldo < static_cast<int>(R)) return -1;
    const int rel_a = (trans_a != 0) != (trans_o != 0);
    const int rel_b = (trans_b != 0) != (trans_o != 0);
    if (lda < static_cast<int>(rel_a ? C : R) || ldb < static_cast<int>(rel_b ? C : R)) return -1;
    // contiguous, identically laid out operands: flat vectorised kernel
    if (!rel_a && !rel_b && static_cast<size_t>(ldo) == R && static_cast<size_t>(lda) == R &&
        static_cast<size_t>(ldb) == R) {
        return OP == kOpAxpby ? jzhip_axpby(out, a, b, R * C, s1, s2) : jzhip_hadamard(out, a, b, R * C);
    }
    return launch2d<OP>(out, ldo, a, lda, rel_a, b, ldb, rel_b, R, C, s1, s2);
}

}  // namespace
}  // namespace jz

using namespace jz;

JZ_API int jzhip_axpby2d(float* out, int ldo, int trans_o, const float* a, int lda, int trans_a,
                         const float* b, int ldb, int trans_b, int rows, int cols, float s1,
                         float s2) {
    return binary2d<kOpAxpby>(out, ldo, trans_o, a, lda, trans_a, b, ldb, trans_b, rows, cols, s1, s2);
}

JZ_API int jzhip_hadamard2d(float* out, int ldo, int trans_o, const float* a, int lda, int trans_a,
                            const float* b, int ldb, int trans_b, int rows, int cols) {
    return binary2d<kOpHadamard>(out, ldo, trans_o, a, lda, trans_a, b, ldb, trans_b, rows, cols, 1.f,
                                 1.f);
}

JZ_API int jzhip_copy2d(float* dst, int ldd, int trans_d, size_t dr0, size_t dc0, const float* src,
                        int lds, int trans_s, size_t sr0, size_t sc0, size_t rows, size_t cols) {
    if (rows == 0 || cols == 0) return 0;
    if (!dst || !src || ldd <= 0 || lds <= 0) return -1;
    // move to the destination's physical frame
    const size_t R = trans_d ? cols : rows;
    const size_t C = trans_d ? rows : cols;
    float* d0 = dst + (trans_d ? dr0 * ldd + dc0 : dc0 * ldd + dr0);
    const float* s0 = src + (trans_s ? sr0 * lds + sc0 : sc0 * lds + sr0);
    const int rel = (trans_s != 0) != (trans_d != 0);
    if (!rel && static_cast<size_t>(ldd) == R && static_cast<size_t>(lds) == R) {
        return jzhip_copy(d0, s0, R * C);
    }
    return launch2d<kOpCopy>(d0, ldd, s0, lds, rel, nullptr, 0, 0, R, C, 1.f, 0.f);
}

// hstack/vstack building blocks (cpp/hipmatrix.cpp:447-527): copy the logical
// content of a possibly transposed source into a column / row offset of a
// plain column-major destination.
JZ_API int jzhip_stack_copy_cols(float* dst, size_t dst_numrow, size_t dst_col_offset,
                                 const float* src, size_t src_numrow, size_t src_numcol,
                                 int src_transpose) {
    const size_t rows = src_transpose ? src_numcol : src_numrow;
    const size_t cols = src_transpose ? src_numrow : src_numcol;
    return jzhip_copy2d(dst, static_cast<int>(dst_numrow), 0, 0, dst_col_offset, src,
                        static_cast<int>(src_numrow), src_transpose, 0, 0, rows, cols);
}

JZ_API int jzhip_stack_copy_rows(float* dst, size_t dst_numrow, size_t dst_row_offset,
                                 const float* src, size_t src_numrow, size_t src_numcol,
                                 int src_transpose) {
    const size_t rows = src_transpose ? src_numcol : src_numrow;
    const size_t cols = src_transpose ? src_numrow : src_numcol;
    return jzhip_copy2d(dst, static_cast<int>(dst_numrow), 0, dst_row_offset, 0, src,
                        static_cast<int>(src_numrow), src_transpose, 0, 0, rows, cols);
}

// Token + position embedding lookup: out(:, n) = E(:, tok[n]) + P(:, n % S) (+ bias).
// The product of a table with a one-hot matrix copies one column per token
// (every other term is an exact zero), so this equals the two one-hot products
// and the bias broadcast bit for bit; an id outside [0, vocab) selects no
// column, as an all-zero one-hot column would.
namespace jz {
namespace {
template <int VEC>
__global__ __launch_bounds__(kBlock) void embedding_fwd_kernel(float* __restrict__ out, const float* __restrict__ E,
                                                               const float* __restrict__ P,
                                                               const float* __restrict__ bias,
                                                               const int32_t* __restrict__ tokens, int d, int vocab,
                                                               FastDiv dS, int S, FastDiv dD, size_t total) {
    const int dv = d / VEC;   // dD divides by dv
    const size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i >= total) return;
    const uint32_t n = fdiv(static_cast<uint32_t>(i), dD);
    const uint32_t r = (static_cast<uint32_t>(i) - n * dv) * VEC;
    const uint32_t pos = n - fdiv(n, dS) * S;
    const int32_t tok = tokens[n];
    const bool live = tok >= 0 && tok < vocab;
    if constexpr (VEC == 4) {
        float4 e = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live) e = *reinterpret_cast<const float4*>(E + static_cast<size_t>(tok) * d + r);
        const float4 p = *reinterpret_cast<const float4*>(P + static_cast<size_t>(pos) * d + r);
        float4 v = make_float4(e.x + p.x, e.y + p.y, e.z + p.z, e.w + p.w);
        if (bias) {
            const float4 b = *reinterpret_cast<const float4*>(bias + r);
            v = make_float4(v.x + b.x, v.y + b.y, v.z + b.z, v.w + b.w);
        }
        *reinterpret_cast<float4*>(out + static_cast<size_t>(n) * d + r) = v;
    } else {
        float v = (live ? E[static_cast<size_t>(tok) * d + r] : 0.0f) + P[static_cast<size_t>(pos) * d + r];
        if (bias) v = v + bias[r];
        out[static_cast<size_t>(n) * d + r] = v;
    }
}
}  // namespace
}  // namespace jz

JZ_API int jzhip_embedding_fwd(float* out, const float* E, const float* P, const float* bias, const int32_t* tokens,
                               int d, int vocab, int S, int N) {
    if (!out || !E || !P || !tokens || d <= 0 || vocab <= 0 || S <= 0 || N <= 0) return -1;
    const size_t elems = static_cast<size_t>(d) * N;
    if (elems >= (size_t(1) << 31)) return -1;
    const bool vec = d % 4 == 0 && aligned16(out) && aligned16(E) && aligned16(P) && (!bias || aligned16(bias));
    if (vec) {
        const size_t total = elems / 4;
        embedding_fwd_kernel<4><<<grid_cover(total, kBlock), kBlock, 0, stream()>>>(
            out, E, P, bias, tokens, d, vocab, make_fastdiv(S), S, make_fastdiv(d / 4), total);
    } else {
        embedding_fwd_kernel<1><<<grid_cover(elems, kBlock), kBlock, 0, stream()>>>(
            out, E, P, bias, tokens, d, vocab, make_fastdiv(S), S, make_fastdiv(d), elems);
    }
    return launch_rc();
}

// One-hot columns from int32 labels on the device (one_hot, ml/util.cuh:295-303,
// builds them on the host and uploads k*n floats): out is k x n column-major,
// zero except out[labels[j] + j*k] = 1.  A label outside [0, k) leaves its
// column zero.
namespace jz {
namespace {
template <int VEC>
__global__ __launch_bounds__(kBlock) void one_hot_kernel(float* __restrict__ out, const int32_t* __restrict__ labels,
                                                         int k, FastDiv dK, size_t total) {
    const int kv = k / VEC;   // dK divides by kv
    const size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i >= total) return;
    const uint32_t j = fdiv(static_cast<uint32_t>(i), dK);
    const int r = static_cast<int>(static_cast<uint32_t>(i) - j * kv) * VEC;
    const int lab = labels[j];
    if constexpr (VEC == 4) {
        const float4 v = make_float4(lab == r ? 1.f : 0.f, lab == r + 1 ? 1.f : 0.f, lab == r + 2 ? 1.f : 0.f,
                                     lab == r + 3 ? 1.f : 0.f);
        *reinterpret_cast<float4*>(out + static_cast<size_t>(j) * k + r) = v;
    } else {
        out[static_cast<size_t>(j) * k + r] = lab == r ? 1.f : 0.f;
    }
}
}  // namespace
}  // namespace jz

JZ_API int jzhip_one_hot(float* out, const int32_t* labels, int k, size_t n) {
    if (!out || !labels || k <= 0 || n == 0) return -1;
    const size_t elems = static_cast<size_t>(k) * n;
    if (elems >= (size_t(1) << 31)) return -1;
    if (k % 4 == 0 && aligned16(out)) {
        const size_t total = elems / 4;
        one_hot_kernel<4><<<grid_cover(total, kBlock), kBlock, 0, stream()>>>(out, labels, k, make_fastdiv(k / 4), total);
    } else {
        one_hot_kernel<1><<<grid_cover(elems, kBlock), kBlock, 0, stream()>>>(out, labels, k, make_fastdiv(k), elems);
    }
    return launch_rc();
}

// slice get / set (cpp/hipmatrix.cpp:268-324).
JZ_API int jzhip_slice_extract(float* dst, size_t dst_numrow, const float* src, size_t src_numrow,
                               int src_transpose, size_t rstart, size_t cstart, size_t rows,
                               size_t cols) {
    return jzhip_copy2d(dst, static_cast<int>(dst_numrow), 0, 0, 0, src,
                        static_cast<int>(src_numrow), src_transpose, rstart, cstart, rows, cols);
}

JZ_API int jzhip_slice_assign(float* dst, size_t dst_numrow, int dst_transpose, size_t rstart,
                              size_t cstart, const float* src, size_t src_numrow,
                              int src_transpose, size_t rows, size_t cols) {
    return jzhip_copy2d(dst, static_cast<int>(dst_numrow), dst_transpose, rstart, cstart, src,
                        static_cast<int>(src_numrow), src_transpose, 0, 0, rows, cols);
}
