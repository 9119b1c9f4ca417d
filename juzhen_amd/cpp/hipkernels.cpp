// Juzhen::Rocm* device API (cpp/hipbackend.hpp:10-136) as forwarders to the C
// ABI of libjzhip.so.  Replaces the reference's cpp/hipkernels.cpp: the
// one-thread-per-element kernels, the rocRAND generator and the hipBLAS handle
// that lived there are gone; each function below is one call.  The ROCm conv
// layers (ml/layer.hpp:1611-1869) and cpp/helper.hpp:207-285 call these
// directly with raw pointers, so the signatures are frozen.
//
// RocmGemm / RocmGemmNN / RocmGemv live in hipmatrix.cpp, as upstream.
#include <cstddef>
#include <cstdint>

#include "jzhip.h"

namespace Juzhen {

bool RocmRuntimeAvailable() { return jzhip_runtime_available() != 0; }

int RocmMalloc(float** ptr, std::size_t count) { return jzhip_malloc(ptr, count); }
int RocmFree(float* ptr) { return jzhip_free(ptr); }
int RocmMemcpyH2D(float* dst, const float* src, std::size_t count) { return jzhip_memcpy_h2d(dst, src, count); }
int RocmMemcpyD2H(float* dst, const float* src, std::size_t count) { return jzhip_memcpy_d2h(dst, src, count); }
int RocmMemcpyD2D(float* dst, const float* src, std::size_t count) { return jzhip_memcpy_d2d(dst, src, count); }

int RocmRandUniform(float* dst, std::size_t count, std::uint64_t seed) { return jzhip_rand_uniform(dst, count, seed); }
int RocmRandNormal(float* dst, std::size_t count, float mean, float stddev, std::uint64_t seed) {
    return jzhip_rand_normal(dst, count, mean, stddev, seed);
}

int RocmFill(float* dst, std::size_t count, float value) { return jzhip_fill(dst, count, value); }
int RocmExpInplace(float* x, std::size_t count) { return jzhip_exp_inplace(x, count); }
int RocmLogInplace(float* x, std::size_t count) { return jzhip_log_inplace(x, count); }
int RocmAxpby(float* out, const float* a, const float* b, std::size_t count, float s1, float s2) {
    return jzhip_axpby(out, a, b, count, s1, s2);
}
int RocmAffineInplace(float* x, std::size_t count, float s1, float a) { return jzhip_affine_inplace(x, count, s1, a); }
int RocmHadamard(float* out, const float* a, const float* b, std::size_t count) {
    return jzhip_hadamard(out, a, b, count);
}
int RocmHadamardInplace(float* x, const float* other, std::size_t count) {
    return jzhip_hadamard_inplace(x, other, count);
}
int RocmElemInvInplace(float* x, std::size_t count, float l) { return jzhip_eleminv_inplace(x, count, l); }
int RocmCopy(float* dst, const float* src, std::size_t count) { return jzhip_copy(dst, src, count); }
int RocmSquare(float* out, const float* in, std::size_t count) { return jzhip_square(out, in, count); }
int RocmSquareInplace(float* x, std::size_t count) { return jzhip_square_inplace(x, count); }
int RocmTanh(float* out, const float* in, std::size_t count) { return jzhip_tanh(out, in, count); }
int RocmTanhInplace(float* x, std::size_t count) { return jzhip_tanh_inplace(x, count); }
int RocmDTanh(float* out, const float* in, std::size_t count) { return jzhip_dtanh(out, in, count); }
int RocmDTanhInplace(float* x, std::size_t count) { return jzhip_dtanh_inplace(x, count); }

int RocmStackCopyCols(float* dst, std::size_t dst_numrow, std::size_t dst_col_offset, const float* src,
                      std::size_t src_numrow, std::size_t src_numcol, bool src_transpose) {
    return jzhip_stack_copy_cols(dst, dst_numrow, dst_col_offset, src, src_numrow, src_numcol, src_transpose);
}
int RocmStackCopyRows(float* dst, std::size_t dst_numrow, std::size_t dst_row_offset, const float* src,
                      std::size_t src_numrow, std::size_t src_numcol, bool src_transpose) {
    return jzhip_stack_copy_rows(dst, dst_numrow, dst_row_offset, src, src_numrow, src_numcol, src_transpose);
}
int RocmSliceExtract(float* dst, std::size_t dst_numrow, const float* src, std::size_t src_numrow,
                     bool src_transpose, std::size_t rstart, std::size_t cstart, std::size_t rows,
                     std::size_t cols) {
    return jzhip_slice_extract(dst, dst_numrow, src, src_numrow, src_transpose, rstart, cstart, rows, cols);
}
int RocmSliceAssign(float* dst, std::size_t dst_numrow, bool dst_transpose, std::size_t rstart,
                    std::size_t cstart, const float* src, std::size_t src_numrow, bool src_transpose,
                    std::size_t rows, std::size_t cols) {
    return jzhip_slice_assign(dst, dst_numrow, dst_transpose, rstart, cstart, src, src_numrow, src_transpose, rows,
                              cols);
}

int RocmIm2col(const float* input, float* col, int C_in, int H_in, int W_in, int kH, int kW, int pad_h, int pad_w,
               int stride_h, int stride_w, int H_out, int W_out, int N) {
    return jzhip_im2col(input, col, C_in, H_in, W_in, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N);
}
int RocmCol2im(const float* col, float* dx, int C_in, int H_in, int W_in, int kH, int kW, int pad_h, int pad_w,
               int stride_h, int stride_w, int H_out, int W_out, int N) {
    return jzhip_col2im(col, dx, C_in, H_in, W_in, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out, N);
}
int RocmConvForwardReshapeBias(const float* y2d, float* out, const float* bias, int C_out, int P, int N) {
    return jzhip_conv_forward_reshape_bias(y2d, out, bias, C_out, P, N);
}
int RocmConvBackwardReshape(const float* t, float* t2d, int C_out, int P, int N) {
    return jzhip_conv_backward_reshape(t, t2d, C_out, P, N);
}
int RocmConvTransScatter(const float* patches, float* out, const float* bias, int C_out, int H_out, int W_out,
                         int H_in, int W_in, int kH, int kW, int pad_h, int pad_w, int stride_h, int stride_w,
                         int N) {
    return jzhip_convtrans_scatter(patches, out, bias, C_out, H_out, W_out, H_in, W_in, kH, kW, pad_h, pad_w,
                                   stride_h, stride_w, N);
}
int RocmConvTransGather(const float* t, float* tp, int C_out, int H_out, int W_out, int H_in, int W_in, int kH,
                        int kW, int pad_h, int pad_w, int stride_h, int stride_w, int N) {
    return jzhip_convtrans_gather(t, tp, C_out, H_out, W_out, H_in, W_in, kH, kW, pad_h, pad_w, stride_h, stride_w,
                                  N);
}
int RocmConvTransReshape(const float* src, float* dst, int C, int spatial, int N, int direction) {
    return jzhip_convtrans_reshape(src, dst, C, spatial, N, direction);
}

}  // namespace Juzhen
