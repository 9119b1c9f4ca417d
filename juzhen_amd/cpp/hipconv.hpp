// ConvLayer for the ROCm backend: drop-in for the class of that name in the
// `#if defined(ROCM_HIP)` block of ml/layer.hpp (:1562-1725).  Same constructor,
// same members, same layouts (input (C_in*H_in*W_in, N), output
// (C_out*H_out*W_out, N), weights the (K, C_out) column-major matrix stored as a
// (C_out*C_in*kH*kW, 1) column, ml/layer.hpp:1566-1569), same order of
// operations in backward() (input gradient with the weights before their
// update, then the update).
//
// What changes: the reference always writes the patch matrix col(K, P*N) with
// RocmIm2col, multiplies it and reshapes the result.  Here each of the three
// products takes the route that is faster for the layer's shape:
//   * implicit GEMM (jzhip_conv2d_forward / _backward_weights / _backward_data, and
//     jzhip_conv2d_transposed for the input gradients of a strided layer):
//     the patch matrix is formed inside the product and never stored; bias,
//     ReLU and the (C_out*P, N) layout are part of the forward store;
//   * the patch-matrix route of the reference (im2col, product, reshape or
//     col2im) for layers with few output pixels per image or very few
//     channels, where the implicit form cannot fill the matrix cores.
// Integration: replace the ROCm ConvLayer and convtransLayer blocks of ml/layer.hpp by
// `#include "../cpp/hipconv.hpp"`; nothing else in the file refers to it.
#ifndef JZ_HIPCONV_HPP
#define JZ_HIPCONV_HPP

#include "jzhip.h"

namespace Juzhen {

class ConvLayer : public Layer<ROCMfloat> {
    using D = ROCMfloat;

    int C_in, H_in, W_in;
    int C_out, kH, kW;
    int pad_h, pad_w, stride_h, stride_w;
    int H_out, W_out;
    int batchN;
    bool use_relu = true;
    // route per product, fixed by the shape (thresholds measured on MI355X)
    bool fwd_implicit, dw_implicit, dx_implicit, dx_transposed;

    static float* ptr(const Matrix<D>& m) { return JzRocmFused::ptr(m); }
    static void must(int rc, const char* what) { rocm_detail::must(rc, what); }

    // col(K, P*N) of `x`
    Matrix<D> patches(const Matrix<D>& x) const {
        const int K = C_in * kH * kW, P = H_out * W_out;
        Matrix<D> col("conv_col", K, (size_t)P * batchN);
        must(jzhip_im2col(ptr(x), ptr(col), C_in, H_in, W_in, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out, W_out,
                          batchN),
             "im2col");
        return col;
    }
    // out(C_out*P, N) = W^T col (+ bias) in the layer's layout; relu applied when asked
    void conv_into(Matrix<D>& out, const Matrix<D>& x, const float* bias_ptr, bool relu) const {
        const int K = C_in * kH * kW, P = H_out * W_out;
        if (fwd_implicit) {
            must(jzhip_conv2d_forward(ptr(x), ptr(this->weights), bias_ptr, ptr(out), C_in, H_in, W_in, C_out, kH, kW,
                                      pad_h, pad_w, stride_h, stride_w, H_out, W_out, batchN, relu ? 1 : 0),
                 "conv2d_forward");
            return;
        }
        Matrix<D> col = patches(x);
        Matrix<D> y2d("conv_y2d", C_out, (size_t)P * batchN);
        must(jzhip_gemm(ptr(this->weights), ptr(col), ptr(y2d), C_out, P * batchN, K, 1, 0, K, K, C_out, 1.0f, 0.0f),
             "gemm");
        if (bias_ptr) {
            must(jzhip_conv_forward_reshape_bias(ptr(y2d), ptr(out), bias_ptr, C_out, P, batchN), "conv reshape");
        } else {
            Matrix<D> zero = Matrix<D>::zeros(C_out, 1);
            must(jzhip_conv_forward_reshape_bias(ptr(y2d), ptr(out), ptr(zero), C_out, P, batchN), "conv reshape");
        }
        if (relu) must(jzhip_relu(ptr(out), ptr(out), (size_t)C_out * P * batchN), "relu");
    }

   public:
    ConvLayer(int N, int C_in, int H_in, int W_in, int C_out, int kH, int kW, int pad = 0, int stride = 1,
              bool relu = true)
        : Layer<D>(C_out * ((H_in + 2 * pad - kH) / stride + 1) * ((W_in + 2 * pad - kW) / stride + 1), 1, N),
          C_in(C_in), H_in(H_in), W_in(W_in), C_out(C_out), kH(kH), kW(kW), pad_h(pad), pad_w(pad), stride_h(stride),
          stride_w(stride), H_out((H_in + 2 * pad - kH) / stride + 1), W_out((W_in + 2 * pad - kW) / stride + 1),
          batchN(N), use_relu(relu) {
        if (H_out <= 0 || W_out <= 0) {
            LOG_ERROR("Invalid conv output shape: H_out={}, W_out={}", H_out, W_out);
            ERROR_OUT;
        }
        const int K = C_in * kH * kW;
        this->weights = Matrix<D>::randn((size_t)C_out * K, 1) * 0.001f;
        this->bias = Matrix<D>::zeros(C_out, 1);
        this->val = Matrix<D>("conv_out", (size_t)C_out * H_out * W_out, N);
        this->adamW = adam_state<D>(0.0001, (size_t)C_out * K, 1);
        this->adamb = adam_state<D>(0.0001, C_out, 1);
        const long long P = (long long)H_out * W_out, J = P * N;
        // forward: the implicit form needs enough output pixels to fill the chip with 64-row tiles
        // (measured down to a 14 x 14 grid: 21 against 35 us for 32 -> 64 channels at batch 128)
        fwd_implicit = J >= 16384 && (P >= 144 || K <= 64);
        // weight gradients: wins when the patch matrix is cheap to form relative to the product
        // (and always with at most four output channels on a 3x3 kernel: a direct kernel streams the input once)
        dw_implicit = (K <= 288) || (stride == 1 && C_out >= 32 && K <= 1152) || (C_out <= 4 && kH == 3 && kW == 3);
        // input gradients: stride 1 only; needs channels on both sides and a grid of 16 x 16 or more
        dx_implicit = stride == 1 && pad <= kH - 1 && pad <= kW - 1 && C_in >= 32 && (long long)H_in * W_in >= 256 &&
                      (long long)H_in * W_in * N >= 16384;
        // shapes beyond what the implicit entry points accept keep the patch-matrix route
        auto accepted = [&](int which) {
            return jzhip_conv2d_check(which, C_in, H_in, W_in, C_out, kH, kW, pad, pad, stride, stride, H_out, W_out,
                                      N) == 0;
        };
        // (the forward and input-gradient kernels that stage image strips win wherever they apply)
        fwd_implicit = (fwd_implicit || accepted(5)) && accepted(0);
        // 3x3 stride-1 layers with channels in multiples of 32: the weight-gradient kernel that
        // stages image strips in LDS wins at every size it takes
        dw_implicit = (dw_implicit || accepted(4)) && accepted(1);
        dx_implicit = (dx_implicit || accepted(6)) && accepted(2);
        // input gradients of a strided layer: the transposed convolution of the upstream gradient
        // with the stored weights; pays when its output channels (C_in) fill a 64-wide tile
        dx_transposed = stride > 1 && C_in >= 64 && (long long)H_in * W_in * N >= 16384 &&
                        jzhip_conv2d_check(3, C_out, H_out, W_out, C_in, kH, kW, pad, pad, stride, stride, H_in, W_in,
                                           N) == 0;
    }

    void eval(const Matrix<D>& input) override { conv_into(this->val, input, ptr(this->bias), use_relu); }

    // Convolution is linear in its input: the tangent takes the same route with
    // no bias, then the activation mask cached by eval().
    Matrix<D> jvp(const Matrix<D>&, const Matrix<D>& tangent) override {
        const size_t P = (size_t)H_out * W_out;
        Matrix<D> out("conv_jvp", C_out * P, batchN);
        conv_into(out, tangent, nullptr, false);
        if (use_relu) must(jzhip_drelu_mul(ptr(out), ptr(this->val), ptr(out), C_out * P * batchN), "drelu_mul");
        return out;
    }

    Matrix<D> grad(const Matrix<D>&) const override { return Matrix<D>::ones(1, 1); }

    Matrix<D> backward(const Matrix<D>& input, Matrix<D>&& upstream_grad) override {
        const int K = C_in * kH * kW, P = H_out * W_out;
        const size_t out_count = (size_t)C_out * P * batchN;
        Matrix<D> t = std::move(upstream_grad);
        // hadmd(d_relu(val), upstream): val > 0 exactly where the pre-activation was
        if (use_relu) must(jzhip_drelu_mul(ptr(t), ptr(this->val), ptr(t), out_count), "drelu_mul");

        const bool need_t2d = !dw_implicit || !(dx_implicit || dx_transposed);
        Matrix<D> t2d("conv_t2d", need_t2d ? C_out : 1, need_t2d ? (size_t)P * batchN : 1);
        if (need_t2d) must(jzhip_conv_backward_reshape(ptr(t), ptr(t2d), C_out, P, batchN), "conv reshape");

        // weight gradients in the stored (K, C_out) layout
        Matrix<D> dW("conv_dW", (size_t)C_out * K, 1);
        if (dw_implicit) {
            must(jzhip_conv2d_backward_weights(ptr(input), ptr(t), ptr(dW), C_in, H_in, W_in, C_out, kH, kW, pad_h, pad_w,
                                               stride_h, stride_w, H_out, W_out, batchN),
                 "conv2d_backward_weights");
        } else {
            Matrix<D> col = patches(input);
            must(jzhip_gemm(ptr(col), ptr(t2d), ptr(dW), K, C_out, P * batchN, 0, 1, K, C_out, K, 1.0f, 0.0f), "gemm");
        }

        // input gradients, with the weights as they were in the forward pass
        Matrix<D> dx("conv_dx", (size_t)C_in * H_in * W_in, batchN);
        if (dx_implicit) {
            must(jzhip_conv2d_backward_data(ptr(t), ptr(this->weights), ptr(dx), C_in, H_in, W_in, C_out, kH, kW, pad_h,
                                            pad_w, stride_h, stride_w, H_out, W_out, batchN),
                 "conv2d_backward_data");
        } else if (dx_transposed) {
            must(jzhip_conv2d_transposed(ptr(t), ptr(this->weights), nullptr, ptr(dx), C_out, H_out, W_out, C_in, kH, kW,
                                         pad_h, pad_w, stride_h, stride_w, H_in, W_in, batchN, 0),
                 "conv2d_transposed");
        } else {
            Matrix<D> dx_col("conv_dx_col", K, (size_t)P * batchN);
            must(jzhip_gemm(ptr(this->weights), ptr(t2d), ptr(dx_col), K, P * batchN, C_out, 0, 0, K, C_out, K, 1.0f, 0.0f),
                 "gemm");
            must(jzhip_col2im(ptr(dx_col), ptr(dx), C_in, H_in, W_in, kH, kW, pad_h, pad_w, stride_h, stride_w, H_out,
                              W_out, batchN),
                 "col2im");
        }

        // bias gradients: db(co) = sum over pixels and images of t
        Matrix<D> db("conv_db", C_out, 1);
        if (need_t2d) {
            db = sum(t2d, 1);
        } else {
            // t is (P, C_out*N) column-major when read as a matrix: column sums, then the N images
            Matrix<D> per_image("conv_db_n", C_out, batchN);
            must(jzhip_sum_cols(ptr(per_image), ptr(t), P, C_out * batchN, P), "sum_cols");
            must(jzhip_sum_rows(ptr(db), ptr(per_image), C_out, batchN, C_out), "sum_rows");
        }

        // weights and bias in one optimiser launch (Layer::update, ml/layer.hpp:108-112, is two
        // adam_update chains and two subtractions)
        if (this->need_update)
            rocm_detail::fused_update({{&this->weights, &dW, &this->adamW}, {&this->bias, &db, &this->adamb}});
        return dx;
    }
};

// Transposed convolution for the ROCm backend: drop-in for convtransLayer of the
// `#if defined(ROCM_HIP)` block of ml/layer.hpp (:1728-1870); same constructor, members,
// layouts (weights the (C_out*kH*kW, C_in) column-major matrix stored as a column) and
// order of operations.  eval() and jvp() run jzhip_conv2d_transposed (one stride-1
// convolution per residue class of the output pixels, bias and ReLU in its store) where it
// accepts the shape and the reference's route (pack, product, scatter) elsewhere.
// backward() differs too: the reference gathers the upstream gradient into
// tp(C_out*kH*kW, P_in*N), which is the patch matrix of a convolution over t seen as a
// (C_out, H_out, W_out) image on the H_in x W_in patch grid, so
//   dx = W^T tp       is jzhip_conv2d_forward of t with the stored weights, landing in
//                     the layer's (C_in*P_in, N) layout without the unpack step, and
//   dW = tp x2d^T     is jzhip_conv2d_backward_weights with the layer input as the
//                     "upstream" operand;
// the gathered matrix is never written.
class convtransLayer : public Layer<ROCMfloat> {
    using D = ROCMfloat;

    int C_in, H_in, W_in;
    int C_out, kH, kW;
    int pad_h, pad_w, stride_h, stride_w;
    int H_out, W_out;
    int batchN;
    bool use_relu = true;
    // backward() as two implicit products; false for shapes those entry points refuse,
    // which keep the gather + product route
    bool bwd_implicit = true;
    // eval() and jvp() without the patch matrix
    bool fwd_implicit = false;

    static float* ptr(const Matrix<D>& m) { return JzRocmFused::ptr(m); }
    static void must(int rc, const char* what) { rocm_detail::must(rc, what); }

    // out(C_out*H_out*W_out, N) = scatter(W x2d) + bias (bias_ptr may be null), then relu when asked
    void deconv_into(Matrix<D>& out, const Matrix<D>& x, const float* bias_ptr, bool relu) const {
        const int P_in = H_in * W_in, rows = C_out * kH * kW;
        if (fwd_implicit) {
            must(jzhip_conv2d_transposed(ptr(x), ptr(this->weights), bias_ptr, ptr(out), C_in, H_in, W_in, C_out, kH, kW,
                                         pad_h, pad_w, stride_h, stride_w, H_out, W_out, batchN, relu ? 1 : 0),
                 "conv2d_transposed");
            return;
        }
        Matrix<D> zero = bias_ptr ? Matrix<D>("deconv_nobias", 1, 1) : Matrix<D>::zeros(C_out, 1);
        const float* b = bias_ptr ? bias_ptr : ptr(zero);
        Matrix<D> x2d("deconv_x2d", C_in, (size_t)P_in * batchN);
        must(jzhip_convtrans_reshape(ptr(x), ptr(x2d), C_in, P_in, batchN, 0), "convtrans reshape");
        Matrix<D> patches("deconv_patches", rows, (size_t)P_in * batchN);
        must(jzhip_gemm(ptr(this->weights), ptr(x2d), ptr(patches), rows, P_in * batchN, C_in, 0, 0, rows, C_in, rows,
                        1.0f, 0.0f),
             "gemm");
        must(jzhip_convtrans_scatter(ptr(patches), ptr(out), b, C_out, H_out, W_out, H_in, W_in, kH, kW, pad_h, pad_w,
                                     stride_h, stride_w, batchN),
             "convtrans scatter");
        if (relu) must(jzhip_relu(ptr(out), ptr(out), (size_t)C_out * H_out * W_out * batchN), "relu");
    }

   public:
    convtransLayer(int N, int C_in, int H_in, int W_in, int C_out, int kH, int kW, int pad = 0, int stride = 1,
                   bool relu = true)
        : Layer<D>(C_out * ((H_in - 1) * stride - 2 * pad + kH) * ((W_in - 1) * stride - 2 * pad + kW), 1, N),
          C_in(C_in), H_in(H_in), W_in(W_in), C_out(C_out), kH(kH), kW(kW), pad_h(pad), pad_w(pad), stride_h(stride),
          stride_w(stride), H_out((H_in - 1) * stride - 2 * pad + kH), W_out((W_in - 1) * stride - 2 * pad + kW),
          batchN(N), use_relu(relu) {
        if (H_out <= 0 || W_out <= 0) {
            LOG_ERROR("Invalid transposed-conv output shape: H_out={}, W_out={}", H_out, W_out);
            ERROR_OUT;
        }
        const size_t wcount = (size_t)C_in * C_out * kH * kW;
        this->weights = Matrix<D>::randn(wcount, 1) * 0.001f;
        this->bias = Matrix<D>::zeros(C_out, 1);
        this->val = Matrix<D>("convtrans_out", (size_t)C_out * H_out * W_out, N);
        this->adamW = adam_state<D>(0.0001, wcount, 1);
        this->adamb = adam_state<D>(0.0001, C_out, 1);
        // the two products of backward() seen as a convolution over the upstream gradient
        bwd_implicit = jzhip_conv2d_check(0, C_out, H_out, W_out, C_in, kH, kW, pad, pad, stride, stride, H_in, W_in,
                                          N) == 0 &&
                       jzhip_conv2d_check(1, C_out, H_out, W_out, C_in, kH, kW, pad, pad, stride, stride, H_in, W_in,
                                          N) == 0;
        // forward as stride-1 convolutions per residue class: needs channels for a 64-wide tile
        // and enough output pixels to fill the chip
        fwd_implicit = C_out >= 32 && (long long)H_out * W_out * N >= 16384 &&
                       jzhip_conv2d_check(3, C_in, H_in, W_in, C_out, kH, kW, pad, pad, stride, stride, H_out, W_out,
                                          N) == 0;
    }

    void eval(const Matrix<D>& input) override { deconv_into(this->val, input, ptr(this->bias), use_relu); }

    Matrix<D> jvp(const Matrix<D>&, const Matrix<D>& tangent) override {
        const size_t count = (size_t)C_out * H_out * W_out * batchN;
        Matrix<D> out("convtrans_jvp", (size_t)C_out * H_out * W_out, batchN);
        deconv_into(out, tangent, nullptr, false);
        if (use_relu) must(jzhip_drelu_mul(ptr(out), ptr(this->val), ptr(out), count), "drelu_mul");
        return out;
    }

    Matrix<D> grad(const Matrix<D>&) const override { return Matrix<D>::ones(1, 1); }

    Matrix<D> backward(const Matrix<D>& input, Matrix<D>&& upstream_grad) override {
        const int P_in = H_in * W_in, P_out = H_out * W_out, rows = C_out * kH * kW;
        Matrix<D> t = std::move(upstream_grad);
        if (use_relu)
            must(jzhip_drelu_mul(ptr(t), ptr(this->val), ptr(t), (size_t)C_out * P_out * batchN), "drelu_mul");

        // weight gradients in the stored (rows, C_in) layout, and input gradients with the
        // weights as they were in the forward pass
        Matrix<D> dW("deconv_dW", (size_t)rows * C_in, 1);
        Matrix<D> dx("deconv_dx", (size_t)C_in * P_in, batchN);
        if (bwd_implicit) {
            must(jzhip_conv2d_backward_weights(ptr(t), ptr(input), ptr(dW), C_out, H_out, W_out, C_in, kH, kW, pad_h,
                                               pad_w, stride_h, stride_w, H_in, W_in, batchN),
                 "conv2d_backward_weights");
            must(jzhip_conv2d_forward(ptr(t), ptr(this->weights), nullptr, ptr(dx), C_out, H_out, W_out, C_in, kH, kW,
                                      pad_h, pad_w, stride_h, stride_w, H_in, W_in, batchN, 0),
                 "conv2d_forward");
        } else {
            // the sequence of ml/layer.hpp:1826-1852: tp = gather(t), x2d = pack(input),
            // dW = tp x2d^T, dx = unpack(W^T tp)
            const size_t cols = (size_t)P_in * batchN;
            Matrix<D> tp("deconv_tp", rows, cols);
            must(jzhip_convtrans_gather(ptr(t), ptr(tp), C_out, H_out, W_out, H_in, W_in, kH, kW, pad_h, pad_w, stride_h,
                                        stride_w, batchN),
                 "convtrans gather");
            Matrix<D> x2d("deconv_x2d", C_in, cols);
            must(jzhip_convtrans_reshape(ptr(input), ptr(x2d), C_in, P_in, batchN, 0), "convtrans reshape");
            must(jzhip_gemm(ptr(tp), ptr(x2d), ptr(dW), rows, C_in, (int)cols, 0, 1, rows, C_in, rows, 1.0f, 0.0f), "gemm");
            Matrix<D> dx2d("deconv_dx2d", C_in, cols);
            must(jzhip_gemm(ptr(this->weights), ptr(tp), ptr(dx2d), C_in, (int)cols, rows, 1, 0, rows, rows, C_in, 1.0f,
                            0.0f),
                 "gemm");
            must(jzhip_convtrans_reshape(ptr(dx2d), ptr(dx), C_in, P_in, batchN, 1), "convtrans reshape");
        }
        // bias gradients: t read as a (P_out, C_out*N) matrix, column sums, then the N images
        Matrix<D> db("deconv_db", C_out, 1);
        {
            Matrix<D> per_image("deconv_db_n", C_out, batchN);
            must(jzhip_sum_cols(ptr(per_image), ptr(t), P_out, C_out * batchN, P_out), "sum_cols");
            must(jzhip_sum_rows(ptr(db), ptr(per_image), C_out, batchN, C_out), "sum_rows");
        }
        if (this->need_update)
            rocm_detail::fused_update({{&this->weights, &dW, &this->adamW}, {&this->bias, &db, &this->adamb}});
        return dx;
    }
};

using ConvTransLayer = convtransLayer;

}  // namespace Juzhen

#endif
