"""Convolution products without the patch matrix (jzhip_conv2d_forward,
_backward_weights, _backward_data, _transposed) through the C ABI.

Small cases are compared with the CPU oracle's restatement of the layer's own
chain (make_im2col + gemm + reshape/bias, ml/layer.hpp:1897-1999 and the ROCm
ConvLayer :1611-1719) within the GEMM tolerance 1e-3, and with a float64
direct convolution (the method of tests/testConvBackendParity.cu:46-124).
Layer-sized cases (the CNN and UNet configurations) are compared with the
patch-matrix route on the device, jzhip_im2col + jzhip_gemm + the reshape
kernels, which the other GPU tests pin to the oracle.
"""
import ctypes as C

import numpy as np
import pytest

from util import dev_empty, dp, dptr, hptr, rel_err, to_dev, to_host

pytestmark = pytest.mark.gpu
TOL_GEMM = 1e-3


def dims(H, W, kH, kW, pad, stride):
    return (H + 2 * pad - kH) // stride + 1, (W + 2 * pad - kW) // stride + 1


def direct_conv64(x, w, b, N, Ci, H, W, Co, kH, kW, pad, stride, relu):
    """x: (N, Ci, H, W) float64, w stored (K, Co) column-major -> (Co, Ci, kH, kW)."""
    Ho, Wo = dims(H, W, kH, kW, pad, stride)
    wk = w.astype(np.float64).reshape(Co, Ci, kH, kW)
    xp = np.zeros((N, Ci, H + 2 * pad, W + 2 * pad))
    xp[:, :, pad:pad + H, pad:pad + W] = x
    out = np.zeros((N, Co, Ho, Wo))
    for ky in range(kH):
        for kx in range(kW):
            patch = xp[:, :, ky:ky + stride * (Ho - 1) + 1:stride, kx:kx + stride * (Wo - 1) + 1:stride]
            out += np.einsum("nchw,oc->nohw", patch, wk[:, :, ky, kx])
    if b is not None:
        out += b.astype(np.float64)[None, :, None, None]
    return np.maximum(out, 0) if relu else out


SMALL = [
    # N, Ci, H, W, Co, kH, kW, pad, stride
    (2, 1, 5, 5, 3, 3, 3, 1, 1),
    (3, 3, 8, 8, 5, 3, 3, 1, 2),
    (2, 4, 7, 9, 70, 3, 3, 1, 1),     # channel tile with a masked edge, odd pixel count
    (1, 2, 6, 6, 130, 3, 3, 0, 1),    # two channel tiles
    (4, 5, 10, 10, 8, 5, 5, 2, 1),
    (2, 11, 12, 12, 16, 3, 3, 1, 1),  # K = 99: not a multiple of the K stage
    (5, 6, 9, 7, 4, 1, 1, 0, 1),
    (2, 3, 9, 9, 6, 4, 4, 1, 2),
    (3, 7, 8, 8, 20, 3, 3, 1, 1),     # K = 63 > two stages: tap table with a ragged last stage, W_out % 4 == 0
    (2, 5, 16, 16, 9, 4, 4, 1, 2),    # 4x4 stride 2 (the transposed layers' backward), W_out = 8
    (1, 40, 4, 4, 8, 3, 3, 1, 1),     # W_out = 4: a stage of 16 columns spans four rows
    (2, 9, 7, 6, 3, 3, 3, 1, 1),      # at most four output channels: the direct kernels, ragged channel split
    (3, 8, 9, 9, 2, 3, 3, 1, 2),      # the same with stride 2
    (2, 8, 8, 8, 4, 5, 5, 2, 1),      # four channels, 5x5: direct forward, tiled weight gradients
    (2, 3, 6, 6, 16, 3, 3, 1, 1),     # input gradients of a 3-channel image: the direct forward kernel with flipped weights
    # kernels of more than 32 taps and patch rows beyond the tap table (K > 3072) take the loaders that
    # decode every element's index, here with three and more K stages
    (2, 3, 12, 12, 8, 7, 7, 3, 1),    # 7x7 stem, K = 147
    (2, 3, 12, 12, 8, 7, 7, 3, 2),    # the same with stride 2
    (1, 344, 4, 4, 8, 3, 3, 1, 1),    # K = 3096
    # one to four input channels, rows in multiples of four pixels: the kernels that keep a pixel quad's window
    # in registers (forward and weight gradients)
    (3, 1, 28, 28, 32, 3, 3, 1, 1),
    (2, 3, 8, 12, 20, 3, 3, 1, 1),    # channel groups with a ragged end
    (2, 4, 4, 4, 9, 3, 3, 1, 1),      # one quad per row, nine output channels
    (5, 2, 12, 8, 10, 3, 3, 1, 1),
    (9, 1, 256, 256, 32, 3, 3, 1, 1), # pixel blocks fill the chip: all output channels in one workgroup, several passes per workgroup in the weight gradients
]


@pytest.mark.parametrize("case", SMALL)
@pytest.mark.parametrize("relu", [0, 1])
def test_forward_small(gpu, oracle_lib, case, relu):
    N, Ci, H, W, Co, kH, kW, pad, stride = case
    Ho, Wo = dims(H, W, kH, kW, pad, stride)
    K, P = Ci * kH * kW, Ho * Wo
    r = np.random.default_rng(sum(case))
    x = r.normal(0, 1, N * Ci * H * W).astype(np.float32)
    w = r.normal(0, 1 / np.sqrt(K), K * Co).astype(np.float32)
    b = r.normal(0, 0.5, Co).astype(np.float32)
    # oracle: the layer's own chain
    col = np.empty(K * P * N, np.float32)
    oracle_lib.jzo_im2col(hptr(x), hptr(col), Ci, H, W, kH, kW, pad, pad, stride, stride, Ho, Wo, N)
    y2d = np.zeros(Co * P * N, np.float32)
    oracle_lib.jzo_gemm(1, 0, Co, P * N, K, 1.0, hptr(w), K, hptr(col), K, 0.0, hptr(y2d), Co)
    want = np.empty(Co * P * N, np.float32)
    oracle_lib.jzo_conv_forward_reshape_bias(hptr(y2d), hptr(want), hptr(b), Co, P, N)
    if relu:
        oracle_lib.jzo_relu(hptr(want), hptr(want), want.size)
    out = to_dev(np.full(Co * P * N, np.nan, np.float32))
    gpu.conv2d_forward(dp(x), dp(w), dp(b), dptr(out), Ci, H, W, Co, kH, kW, pad, pad, stride, stride, Ho, Wo, N, relu)
    got = to_host(out)
    assert np.isfinite(got).all()
    assert rel_err(got, want) <= TOL_GEMM
    exact = direct_conv64(x.reshape(N, Ci, H, W), w, b, N, Ci, H, W, Co, kH, kW, pad, stride, relu)
    assert rel_err(got, exact.reshape(-1)) <= TOL_GEMM
    # without a bias
    gpu.conv2d_forward(dp(x), dp(w), None, dptr(out), Ci, H, W, Co, kH, kW, pad, pad, stride, stride, Ho, Wo, N, 0)
    exact0 = direct_conv64(x.reshape(N, Ci, H, W), w, None, N, Ci, H, W, Co, kH, kW, pad, stride, 0)
    assert rel_err(to_host(out), exact0.reshape(-1)) <= TOL_GEMM


@pytest.mark.parametrize("case", SMALL)
def test_backward_small(gpu, oracle_lib, case):
    N, Ci, H, W, Co, kH, kW, pad, stride = case
    Ho, Wo = dims(H, W, kH, kW, pad, stride)
    K, P = Ci * kH * kW, Ho * Wo
    r = np.random.default_rng(sum(case) + 1)
    x = r.normal(0, 1, N * Ci * H * W).astype(np.float32)
    w = r.normal(0, 1 / np.sqrt(K), K * Co).astype(np.float32)
    t = r.normal(0, 1, Co * P * N).astype(np.float32)
    # oracle chain of ConvLayer::backward (ml/layer.hpp:1679-1709)
    t2d = np.empty(Co * P * N, np.float32)
    oracle_lib.jzo_conv_backward_reshape(hptr(t), hptr(t2d), Co, P, N)
    col = np.empty(K * P * N, np.float32)
    oracle_lib.jzo_im2col(hptr(x), hptr(col), Ci, H, W, kH, kW, pad, pad, stride, stride, Ho, Wo, N)
    dW = np.zeros(K * Co, np.float32)
    oracle_lib.jzo_gemm(0, 1, K, Co, P * N, 1.0, hptr(col), K, hptr(t2d), Co, 0.0, hptr(dW), K)
    got = to_dev(np.full(K * Co, np.nan, np.float32))
    gpu.conv2d_backward_weights(dp(x), dp(t), dptr(got), Ci, H, W, Co, kH, kW, pad, pad, stride, stride, Ho, Wo, N)
    assert rel_err(to_host(got), dW) <= TOL_GEMM
    if stride == 1:
        dcol = np.zeros(K * P * N, np.float32)
        oracle_lib.jzo_gemm(0, 0, K, P * N, Co, 1.0, hptr(w), K, hptr(t2d), Co, 0.0, hptr(dcol), K)
        dx = np.empty(Ci * H * W * N, np.float32)
        oracle_lib.jzo_col2im(hptr(dcol), hptr(dx), Ci, H, W, kH, kW, pad, pad, stride, stride, Ho, Wo, N)
        gdx = to_dev(np.full(Ci * H * W * N, np.nan, np.float32))
        gpu.conv2d_backward_data(dp(t), dp(w), dptr(gdx), Ci, H, W, Co, kH, kW, pad, pad, stride, stride, Ho, Wo, N)
        assert rel_err(to_host(gdx), dx) <= TOL_GEMM
    else:
        from juzhen_amd import capi
        lib = capi.load()
        d = dev_empty(4)
        assert lib.jzhip_conv2d_backward_data(dptr(d), dptr(d), dptr(d), Ci, H, W, Co, kH, kW, pad, pad, stride, stride,
                                              Ho, Wo, N) == -1


LAYERS = [
    # the CNN configuration (batch 128) and the UNet configuration's 3x3 layers
    (128, 1, 28, 28, 32, 3, 3, 1, 1), (128, 32, 28, 28, 64, 3, 3, 1, 2),
    (128, 3, 32, 32, 64, 3, 3, 1, 1), (128, 64, 32, 32, 64, 3, 3, 1, 1), (128, 64, 32, 32, 128, 3, 3, 1, 2),
    (128, 128, 16, 16, 128, 3, 3, 1, 1), (128, 128, 16, 16, 256, 3, 3, 1, 2), (128, 256, 8, 8, 256, 3, 3, 1, 1),
    (128, 256, 16, 16, 128, 3, 3, 1, 1), (128, 128, 32, 32, 64, 3, 3, 1, 1), (128, 64, 32, 32, 3, 3, 3, 1, 1),
    (64, 32, 32, 32, 128, 3, 3, 1, 1),   # forward strips with 128-channel tiles (512 pixel tiles x 1)
    # the backward pass of the UNet's 4x4 stride-2 transposed convolutions is a convolution over the
    # upstream gradient: image = (C_out, H_out, W_out), patch grid = (H_in, W_in), "channels out" = C_in
    (128, 128, 16, 16, 256, 4, 4, 1, 2), (128, 64, 32, 32, 128, 4, 4, 1, 2),
]


@pytest.mark.parametrize("case", LAYERS)
def test_layer_sizes_against_the_patch_matrix_route(gpu, case):
    import torch
    N, Ci, H, W, Co, kH, kW, pad, stride = case
    Ho, Wo = dims(H, W, kH, kW, pad, stride)
    K, P = Ci * kH * kW, Ho * Wo
    g = torch.Generator(device="cuda")
    g.manual_seed(sum(case))
    x = torch.randn(N * Ci * H * W, generator=g, device="cuda")
    w = torch.randn(K * Co, generator=g, device="cuda") / np.sqrt(K)
    b = torch.randn(Co, generator=g, device="cuda")
    t = torch.randn(Co * P * N, generator=g, device="cuda")
    col = torch.empty(K * P * N, device="cuda")
    gpu.im2col(dptr(x), dptr(col), Ci, H, W, kH, kW, pad, pad, stride, stride, Ho, Wo, N)
    y2d = torch.empty(Co * P * N, device="cuda")
    gpu.gemm(dptr(w), dptr(col), dptr(y2d), Co, P * N, K, 1, 0, K, K, Co, 1.0, 0.0)
    want = torch.empty(Co * P * N, device="cuda")
    gpu.conv_forward_reshape_bias(dptr(y2d), dptr(want), dptr(b), Co, P, N)
    gpu.relu(dptr(want), dptr(want), Co * P * N)
    got = torch.full((Co * P * N,), float("nan"), device="cuda")
    gpu.conv2d_forward(dptr(x), dptr(w), dptr(b), dptr(got), Ci, H, W, Co, kH, kW, pad, pad, stride, stride, Ho, Wo, N, 1)
    gpu.synchronize()
    assert bool(torch.isfinite(got).all())
    assert float((got - want).norm() / want.norm()) <= 1e-5
    # weight gradients
    t2d = torch.empty(Co * P * N, device="cuda")
    gpu.conv_backward_reshape(dptr(t), dptr(t2d), Co, P, N)
    dW = torch.empty(K * Co, device="cuda")
    gpu.gemm(dptr(col), dptr(t2d), dptr(dW), K, Co, P * N, 0, 1, K, Co, K, 1.0, 0.0)
    gW = torch.full((K * Co,), float("nan"), device="cuda")
    gpu.conv2d_backward_weights(dptr(x), dptr(t), dptr(gW), Ci, H, W, Co, kH, kW, pad, pad, stride, stride, Ho, Wo, N)
    gpu.synchronize()
    assert float((gW - dW).norm() / dW.norm()) <= 1e-4
    if stride == 1:
        dcol = col                       # reuse the buffer
        gpu.gemm(dptr(w), dptr(t2d), dptr(dcol), K, P * N, Co, 0, 0, K, Co, K, 1.0, 0.0)
        dx = torch.empty(Ci * H * W * N, device="cuda")
        gpu.col2im(dptr(dcol), dptr(dx), Ci, H, W, kH, kW, pad, pad, stride, stride, Ho, Wo, N)
        gdx = torch.full((Ci * H * W * N,), float("nan"), device="cuda")
        gpu.conv2d_backward_data(dptr(t), dptr(w), dptr(gdx), Ci, H, W, Co, kH, kW, pad, pad, stride, stride, Ho, Wo, N)
        gpu.synchronize()
        assert float((gdx - dx).norm() / dx.norm()) <= 1e-5


def test_rejects_bad_arguments(gpu):
    from juzhen_amd import capi
    lib = capi.load()
    d = dev_empty(64)
    assert lib.jzhip_conv2d_forward(None, dptr(d), None, dptr(d), 1, 4, 4, 1, 3, 3, 1, 1, 1, 1, 4, 4, 1, 0) == -1
    assert lib.jzhip_conv2d_forward(dptr(d), dptr(d), None, dptr(d), 1, 4, 4, 1, 3, 3, 1, 1, 0, 1, 4, 4, 1, 0) == -1
    assert lib.jzhip_conv2d_backward_weights(dptr(d), dptr(d), None, 1, 4, 4, 1, 3, 3, 1, 1, 1, 1, 4, 4, 1) == -1
    # a patch grid larger than the geometry implies: (4 + 2 - 3)/1 + 1 = 4, not 5
    assert lib.jzhip_conv2d_forward(dptr(d), dptr(d), None, dptr(d), 1, 4, 4, 1, 3, 3, 1, 1, 1, 1, 5, 4, 1, 0) == -1
    assert lib.jzhip_conv2d_backward_weights(dptr(d), dptr(d), dptr(d), 1, 4, 4, 1, 3, 3, 1, 1, 1, 1, 4, 5, 1) == -1
    # input gradients need H_in == H_out + kH - 1 - 2*pad: a 3x3 grid under a 4x4 input with pad 1 is not that
    assert lib.jzhip_conv2d_backward_data(dptr(d), dptr(d), dptr(d), 1, 4, 4, 1, 3, 3, 1, 1, 1, 1, 3, 3, 1) == -1
    # the same answers from the query that launches nothing
    assert lib.jzhip_conv2d_check(0, 1, 4, 4, 1, 3, 3, 1, 1, 1, 1, 4, 4, 1) == 0
    assert lib.jzhip_conv2d_check(0, 1, 4, 4, 1, 3, 3, 1, 1, 1, 1, 5, 4, 1) == -1
    assert lib.jzhip_conv2d_check(2, 1, 4, 4, 1, 3, 3, 1, 1, 2, 2, 2, 2, 1) == -1      # stride 2
    assert lib.jzhip_conv2d_check(2, 2048, 4, 4, 1024, 3, 3, 1, 1, 1, 1, 4, 4, 1) == -1   # 18.9 Mi weights
    assert lib.jzhip_conv2d_check(1, 2048, 4, 4, 1024, 3, 3, 1, 1, 1, 1, 4, 4, 1) == 0
    assert lib.jzhip_conv2d_check(7, 1, 4, 4, 1, 3, 3, 1, 1, 1, 1, 4, 4, 1) == -1
    # which = 5 / 6: forward and input gradients from image strips
    assert lib.jzhip_conv2d_check(5, 64, 32, 32, 64, 3, 3, 1, 1, 1, 1, 32, 32, 128) == 0
    assert lib.jzhip_conv2d_check(5, 64, 32, 32, 32, 3, 3, 1, 1, 1, 1, 32, 32, 128) == -1   # 32 output channels
    assert lib.jzhip_conv2d_check(5, 3, 32, 32, 64, 3, 3, 1, 1, 1, 1, 32, 32, 128) == -1    # 3 input channels
    assert lib.jzhip_conv2d_check(6, 64, 32, 32, 8, 3, 3, 1, 1, 1, 1, 32, 32, 128) == 0     # dx: 8 channels in, 64 out
    assert lib.jzhip_conv2d_check(6, 8, 32, 32, 64, 3, 3, 1, 1, 1, 1, 32, 32, 128) == -1    # dx would have 8 output channels
    assert lib.jzhip_conv2d_check(5, 64, 6, 32, 64, 3, 3, 1, 1, 1, 1, 6, 32, 128) == -1     # six rows: no whole tiles of four
    # which = 4: weight gradients from image strips
    assert lib.jzhip_conv2d_check(4, 64, 32, 32, 64, 3, 3, 1, 1, 1, 1, 32, 32, 128) == 0
    assert lib.jzhip_conv2d_check(4, 64, 32, 32, 48, 3, 3, 1, 1, 1, 1, 32, 32, 128) == -1   # 48 output channels
    assert lib.jzhip_conv2d_check(4, 64, 28, 28, 64, 3, 3, 1, 1, 1, 1, 28, 28, 128) == -1   # rows of 28 pixels
    assert lib.jzhip_conv2d_check(4, 64, 32, 32, 64, 3, 3, 1, 1, 2, 2, 16, 16, 128) == -1   # stride 2
    assert lib.jzhip_conv2d_check(4, 32, 8, 8, 32, 3, 3, 1, 1, 1, 1, 8, 8, 3) == -1         # three stages in all
    # transposed: 4x4 -> (4-1)*2 - 2 + 4 = 8; one row more is the input grid of a strided layer, two are not
    assert lib.jzhip_conv2d_check(3, 1, 4, 4, 1, 4, 4, 1, 1, 2, 2, 8, 8, 1) == 0
    assert lib.jzhip_conv2d_check(3, 1, 4, 4, 1, 4, 4, 1, 1, 2, 2, 9, 9, 1) == 0
    assert lib.jzhip_conv2d_check(3, 1, 4, 4, 1, 4, 4, 1, 1, 2, 2, 10, 8, 1) == -1
    assert lib.jzhip_conv2d_check(3, 1, 4, 4, 1, 1, 1, 0, 0, 2, 2, 7, 7, 1) == -1      # kernel extent below the stride
    assert lib.jzhip_conv2d_check(3, 1, 4, 4, 1, 3, 3, 1, 1, 3, 3, 10, 10, 1) == -1    # nine residue classes
    assert lib.jzhip_conv2d_transposed(dptr(d), dptr(d), None, dptr(d), 1, 4, 4, 1, 4, 4, 1, 1, 2, 2, 10, 8, 1, 0) == -1
    assert lib.jzhip_conv2d_transposed(dptr(d), None, None, dptr(d), 1, 4, 4, 1, 4, 4, 1, 1, 2, 2, 8, 8, 1, 0) == -1


# ── transposed convolution as stride-1 convolutions per residue class ─────────
def direct_transposed64(x, w, b, N, Ci, H, W, Co, kH, kW, pad, sh, sw, Ho, Wo):
    """Scatter formulation in float64: x (N, Ci, H, W); w the (Co*kH*kW, Ci) column-major matrix."""
    wk = w.astype(np.float64).reshape(Ci, Co, kH, kW)
    big = np.zeros((N, Co, (H - 1) * sh + kH + sh, (W - 1) * sw + kW + sw))
    for ky in range(kH):
        for kx in range(kW):
            big[:, :, ky:ky + sh * (H - 1) + 1:sh, kx:kx + sw * (W - 1) + 1:sw] += np.einsum(
                "nchw,co->nohw", x, wk[:, :, ky, kx])
    out = big[:, :, pad:pad + Ho, pad:pad + Wo].copy()
    if b is not None:
        out += b.astype(np.float64)[None, :, None, None]
    return out


TRANSPOSED = [
    # N, Ci, H, W, Co, kH, kW, pad, stride_h, stride_w
    (2, 3, 4, 4, 5, 4, 4, 1, 2, 2),      # the UNet's up-sampling geometry
    (3, 5, 5, 7, 4, 3, 3, 1, 2, 2),      # odd extents, classes with 2x2, 2x1, 1x2 and 1x1 taps
    (2, 4, 6, 6, 70, 4, 4, 1, 2, 2),     # masked channel tile
    (1, 6, 5, 5, 130, 2, 2, 0, 2, 2),    # non-overlapping up-sampling, two channel tiles
    (2, 7, 6, 5, 3, 5, 5, 2, 2, 2),      # 3x3 / 3x2 / 2x3 / 2x2 sub-kernels
    (2, 5, 7, 7, 6, 3, 3, 1, 1, 1),      # stride 1: a single class, the flipped kernel
    (3, 2, 6, 6, 4, 3, 3, 0, 1, 1),
    (2, 40, 4, 4, 8, 4, 4, 1, 2, 2),     # K of a class = 160: the tap-table loaders
    (2, 48, 5, 5, 64, 4, 4, 1, 2, 2),    # K = 192, full channel tile: the unchecked weight loader
    (2, 3, 5, 6, 4, 4, 3, 1, 2, 1),      # stride on one axis only
    (2, 3, 5, 6, 4, 3, 4, 0, 1, 2),
    (2, 9, 3, 3, 5, 4, 4, 0, 2, 2),      # no padding: output 8x8 from 3x3
    (1, 2, 1, 1, 3, 4, 4, 1, 2, 2),      # a single input pixel
]


@pytest.mark.parametrize("case", TRANSPOSED)
@pytest.mark.parametrize("relu", [0, 1])
def test_transposed_small(gpu, oracle_lib, case, relu):
    """Against the oracle's chain of convtransLayer::eval (ml/layer.hpp:1770-1790): pack the input,
    one GEMM with the stored weights, scatter + bias; and against the float64 scatter sum."""
    N, Ci, H, W, Co, kH, kW, pad, sh, sw = case
    Ho, Wo = (H - 1) * sh - 2 * pad + kH, (W - 1) * sw - 2 * pad + kW
    R, Pin = Co * kH * kW, H * W
    r = np.random.default_rng(sum(case) + 7 * relu)
    x = r.normal(0, 1, N * Ci * H * W).astype(np.float32)
    w = r.normal(0, 1 / np.sqrt(Ci * kH * kW / (sh * sw)), R * Ci).astype(np.float32)
    b = r.normal(0, 0.5, Co).astype(np.float32)
    x2d = np.empty(Ci * Pin * N, np.float32)
    oracle_lib.jzo_convtrans_reshape(hptr(x), hptr(x2d), Ci, Pin, N, 0)
    patches = np.zeros(R * Pin * N, np.float32)
    oracle_lib.jzo_gemm(0, 0, R, Pin * N, Ci, 1.0, hptr(w), R, hptr(x2d), Ci, 0.0, hptr(patches), R)
    want = np.empty(Co * Ho * Wo * N, np.float32)
    oracle_lib.jzo_convtrans_scatter(hptr(patches), hptr(want), hptr(b), Co, Ho, Wo, H, W, kH, kW, pad, pad, sh, sw, N)
    if relu:
        want = np.maximum(want, 0)
    got = to_dev(np.full(Co * Ho * Wo * N, np.nan, np.float32))
    from juzhen_amd import capi
    lib = capi.load()
    assert lib.jzhip_conv2d_check(3, Ci, H, W, Co, kH, kW, pad, pad, sh, sw, Ho, Wo, N) == 0
    gpu.conv2d_transposed(dp(x), dp(w), dp(b), dptr(got), Ci, H, W, Co, kH, kW, pad, pad, sh, sw, Ho, Wo, N, relu)
    got = to_host(got)
    assert np.isfinite(got).all()
    assert rel_err(got, want) <= TOL_GEMM
    ref = direct_transposed64(x.reshape(N, Ci, H, W).astype(np.float64), w, b, N, Ci, H, W, Co, kH, kW, pad, sh, sw, Ho, Wo)
    if relu:
        ref = np.maximum(ref, 0)
    assert rel_err(got, ref) <= TOL_GEMM
    if not relu:   # without the bias pointer the sum alone
        got0 = to_dev(np.full(Co * Ho * Wo * N, np.nan, np.float32))
        gpu.conv2d_transposed(dp(x), dp(w), None, dptr(got0), Ci, H, W, Co, kH, kW, pad, pad, sh, sw, Ho, Wo, N, 0)
        assert rel_err(to_host(got0) + np.tile(np.repeat(b, Ho * Wo), N), want) <= TOL_GEMM


@pytest.mark.parametrize("case", [c for c in SMALL if c[8] > 1] + [
    (2, 6, 9, 9, 5, 3, 3, 1, 2),       # (9 + 2 - 3) % 2 == 0: every input row is reached
    (2, 6, 10, 10, 5, 3, 3, 1, 2),     # the last input row is reached by no patch from below: one row beyond the natural extent
    (2, 4, 11, 8, 7, 3, 3, 0, 2),
    (2, 4, 12, 12, 6, 2, 2, 0, 2),
])
def test_strided_input_gradients_through_the_transposed_product(gpu, oracle_lib, case):
    """dx of a strided ConvLayer (ml/layer.hpp:1698-1709: W t2d, then col2im) is the transposed
    convolution of the upstream gradient with the layer's stored weights read as a
    (C_in*kH*kW, C_out) matrix."""
    N, Ci, H, W, Co, kH, kW, pad, stride = case
    Ho, Wo = dims(H, W, kH, kW, pad, stride)
    K, P = Ci * kH * kW, Ho * Wo
    r = np.random.default_rng(sum(case) + 3)
    w = r.normal(0, 1 / np.sqrt(K), K * Co).astype(np.float32)
    t = r.normal(0, 1, Co * P * N).astype(np.float32)
    t2d = np.empty(Co * P * N, np.float32)
    oracle_lib.jzo_conv_backward_reshape(hptr(t), hptr(t2d), Co, P, N)
    dcol = np.zeros(K * P * N, np.float32)
    oracle_lib.jzo_gemm(0, 0, K, P * N, Co, 1.0, hptr(w), K, hptr(t2d), Co, 0.0, hptr(dcol), K)
    dx = np.empty(Ci * H * W * N, np.float32)
    oracle_lib.jzo_col2im(hptr(dcol), hptr(dx), Ci, H, W, kH, kW, pad, pad, stride, stride, Ho, Wo, N)
    gdx = to_dev(np.full(Ci * H * W * N, np.nan, np.float32))
    gpu.conv2d_transposed(dp(t), dp(w), None, dptr(gdx), Co, Ho, Wo, Ci, kH, kW, pad, pad, stride, stride, H, W, N, 0)
    got = to_host(gdx)
    assert np.isfinite(got).all()
    assert rel_err(got, dx) <= TOL_GEMM


TRANSPOSED_LAYERS = [
    # the UNet configuration's up-sampling layers (batch 128): N, Ci, H, W, Co, kH, kW, pad, stride
    (128, 256, 8, 8, 128, 4, 4, 1, 2), (128, 128, 16, 16, 64, 4, 4, 1, 2),
]


@pytest.mark.parametrize("case", TRANSPOSED_LAYERS)
def test_transposed_layer_sizes_against_the_scatter_route(gpu, case):
    import torch
    N, Ci, H, W, Co, kH, kW, pad, s = case
    Ho, Wo = (H - 1) * s - 2 * pad + kH, (W - 1) * s - 2 * pad + kW
    R, Pin = Co * kH * kW, H * W
    g = torch.Generator(device="cuda")
    g.manual_seed(sum(case))
    x = torch.randn(N * Ci * Pin, generator=g, device="cuda")
    w = torch.randn(R * Ci, generator=g, device="cuda") / np.sqrt(Ci * 4)
    b = torch.randn(Co, generator=g, device="cuda")
    x2d = torch.empty_like(x)
    gpu.convtrans_reshape(dptr(x), dptr(x2d), Ci, Pin, N, 0)
    patches = torch.empty(R * Pin * N, device="cuda")
    gpu.gemm(dptr(w), dptr(x2d), dptr(patches), R, Pin * N, Ci, 0, 0, R, Ci, R, 1.0, 0.0)
    want = torch.empty(Co * Ho * Wo * N, device="cuda")
    gpu.convtrans_scatter(dptr(patches), dptr(want), dptr(b), Co, Ho, Wo, H, W, kH, kW, pad, pad, s, s, N)
    gpu.relu(dptr(want), dptr(want), want.numel())
    got = torch.full((Co * Ho * Wo * N,), float("nan"), device="cuda")
    gpu.conv2d_transposed(dptr(x), dptr(w), dptr(b), dptr(got), Ci, H, W, Co, kH, kW, pad, pad, s, s, Ho, Wo, N, 1)
    gpu.synchronize()
    assert bool(torch.isfinite(got).all())
    assert float((got - want).norm() / want.norm()) <= 1e-5


@pytest.mark.parametrize("case", [c for c in LAYERS if c[8] > 1])
def test_strided_layer_input_gradients_against_the_patch_matrix_route(gpu, case):
    import torch
    N, Ci, H, W, Co, kH, kW, pad, stride = case
    Ho, Wo = dims(H, W, kH, kW, pad, stride)
    K, P = Ci * kH * kW, Ho * Wo
    g = torch.Generator(device="cuda")
    g.manual_seed(sum(case) + 5)
    w = torch.randn(K * Co, generator=g, device="cuda") / np.sqrt(K)
    t = torch.randn(Co * P * N, generator=g, device="cuda")
    t2d = torch.empty_like(t)
    gpu.conv_backward_reshape(dptr(t), dptr(t2d), Co, P, N)
    dcol = torch.empty(K * P * N, device="cuda")
    gpu.gemm(dptr(w), dptr(t2d), dptr(dcol), K, P * N, Co, 0, 0, K, Co, K, 1.0, 0.0)
    dx = torch.empty(Ci * H * W * N, device="cuda")
    gpu.col2im(dptr(dcol), dptr(dx), Ci, H, W, kH, kW, pad, pad, stride, stride, Ho, Wo, N)
    gdx = torch.full((Ci * H * W * N,), float("nan"), device="cuda")
    gpu.conv2d_transposed(dptr(t), dptr(w), None, dptr(gdx), Co, Ho, Wo, Ci, kH, kW, pad, pad, stride, stride, H, W, N, 0)
    gpu.synchronize()
    assert bool(torch.isfinite(gdx).all())
    assert float((gdx - dx).norm() / dx.norm()) <= 1e-5


# ── weight gradients from image strips (3x3, stride 1, pad 1, channels in multiples of 32) ──
DW_STRIP = [
    # N, Ci, H, W, Co: rows of 8, 16, 32 and 64 pixels; chunk counts that are and are not multiples of 8;
    # a last chunk shorter than the others; several tiles on either side
    (4, 32, 8, 8, 32), (5, 32, 16, 16, 32), (3, 64, 16, 16, 32), (2, 32, 32, 32, 64), (16, 32, 32, 32, 64),
    (9, 64, 32, 32, 96), (2, 32, 4, 64, 32), (7, 32, 8, 8, 64), (33, 32, 8, 8, 32), (3, 32, 6, 32, 32),
]


@pytest.mark.parametrize("case", DW_STRIP)
def test_weight_gradients_from_strips(gpu, oracle_lib, case):
    """Against the oracle's col * t2d^T of ConvLayer::backward (ml/layer.hpp:1679-1695) and a float64
    sum over shifted images; the general kernel (JZHIP_CONV_DW_STRIP unset selects the strip form
    for these shapes) is covered by test_backward_small."""
    N, Ci, H, W, Co = case
    K, P = Ci * 9, H * W
    r = np.random.default_rng(sum(case))
    x = r.normal(0, 1, N * Ci * P).astype(np.float32)
    t = r.normal(0, 1, Co * P * N).astype(np.float32)
    t2d = np.empty(Co * P * N, np.float32)
    oracle_lib.jzo_conv_backward_reshape(hptr(t), hptr(t2d), Co, P, N)
    col = np.empty(K * P * N, np.float32)
    oracle_lib.jzo_im2col(hptr(x), hptr(col), Ci, H, W, 3, 3, 1, 1, 1, 1, H, W, N)
    dW = np.zeros(K * Co, np.float32)
    oracle_lib.jzo_gemm(0, 1, K, Co, P * N, 1.0, hptr(col), K, hptr(t2d), Co, 0.0, hptr(dW), K)
    got = to_dev(np.full(K * Co, np.nan, np.float32))
    gpu.conv2d_backward_weights(dp(x), dp(t), dptr(got), Ci, H, W, Co, 3, 3, 1, 1, 1, 1, H, W, N)
    got = to_host(got)
    assert np.isfinite(got).all()
    assert rel_err(got, dW) <= TOL_GEMM
    xp = np.zeros((N, Ci, H + 2, W + 2))
    xp[:, :, 1:-1, 1:-1] = x.reshape(N, Ci, H, W)
    t4 = t.reshape(N, Co, H, W).astype(np.float64)
    ref = np.empty((Co, Ci, 3, 3))
    for ky in range(3):
        for kx in range(3):
            ref[:, :, ky, kx] = np.einsum("nchw,nohw->oc", xp[:, :, ky:ky + H, kx:kx + W], t4)
    assert rel_err(got, ref.ravel()) <= 1e-5
    # the same sums on a second call (fixed summation order)
    again = to_dev(np.full(K * Co, np.nan, np.float32))
    gpu.conv2d_backward_weights(dp(x), dp(t), dptr(again), Ci, H, W, Co, 3, 3, 1, 1, 1, 1, H, W, N)
    assert np.array_equal(to_host(again), got)


# ── forward product and input gradients from image strips (3x3, stride 1, pad 1) ──
FWD_STRIP = [
    # N, Ci, H, W, Co: input channels in multiples of 8, output channels in multiples of 64, rows of 32 / 16 / 8
    # pixels in tiles of 4 / 8 / 8 rows; one and several stages, one and several tiles per image
    (2, 8, 4, 32, 64), (1, 16, 8, 32, 128), (3, 8, 8, 16, 64), (2, 24, 16, 16, 128), (2, 8, 8, 8, 64),
    (5, 16, 8, 8, 128), (2, 40, 4, 32, 64), (1, 8, 16, 8, 64),
]


@pytest.mark.parametrize("case", FWD_STRIP)
@pytest.mark.parametrize("relu", [0, 1])
def test_forward_from_strips(gpu, oracle_lib, case, relu):
    N, Ci, H, W, Co = case
    K, P = Ci * 9, H * W
    r = np.random.default_rng(sum(case) + relu)
    x = r.normal(0, 1, N * Ci * P).astype(np.float32)
    w = r.normal(0, 1 / np.sqrt(K), K * Co).astype(np.float32)
    b = r.normal(0, 0.5, Co).astype(np.float32)
    col = np.empty(K * P * N, np.float32)
    oracle_lib.jzo_im2col(hptr(x), hptr(col), Ci, H, W, 3, 3, 1, 1, 1, 1, H, W, N)
    y2d = np.zeros(Co * P * N, np.float32)
    oracle_lib.jzo_gemm(1, 0, Co, P * N, K, 1.0, hptr(w), K, hptr(col), K, 0.0, hptr(y2d), Co)
    want = np.empty(Co * P * N, np.float32)
    oracle_lib.jzo_conv_forward_reshape_bias(hptr(y2d), hptr(want), hptr(b), Co, P, N)
    if relu:
        want = np.maximum(want, 0)
    got = to_dev(np.full(Co * P * N, np.nan, np.float32))
    gpu.conv2d_forward(dp(x), dp(w), dp(b), dptr(got), Ci, H, W, Co, 3, 3, 1, 1, 1, 1, H, W, N, relu)
    got = to_host(got)
    assert np.isfinite(got).all()
    assert rel_err(got, want) <= TOL_GEMM
    ref = direct_conv64(x.reshape(N, Ci, H, W).astype(np.float64), w, b, N, Ci, H, W, Co, 3, 3, 1, 1, relu)
    assert rel_err(got, ref) <= 1e-5
    if not relu:   # without the bias pointer
        got0 = to_dev(np.full(Co * P * N, np.nan, np.float32))
        gpu.conv2d_forward(dp(x), dp(w), None, dptr(got0), Ci, H, W, Co, 3, 3, 1, 1, 1, 1, H, W, N, 0)
        ref0 = direct_conv64(x.reshape(N, Ci, H, W).astype(np.float64), w, None, N, Ci, H, W, Co, 3, 3, 1, 1, 0)
        assert rel_err(to_host(got0), ref0) <= 1e-5


@pytest.mark.parametrize("case", FWD_STRIP)
def test_input_gradients_from_strips(gpu, oracle_lib, case):
    """The layer of each case read backwards: Co channels come in as the upstream gradient of a
    layer with Co input channels... the roles swap, so the layer here has C_in = the case's Co and
    C_out = the case's Ci (the product's input channels)."""
    N, Cout_l, H, W, Cin_l = case
    K, P = Cin_l * 9, H * W
    r = np.random.default_rng(sum(case) + 11)
    w = r.normal(0, 1 / np.sqrt(K), K * Cout_l).astype(np.float32)
    t = r.normal(0, 1, Cout_l * P * N).astype(np.float32)
    t2d = np.empty(Cout_l * P * N, np.float32)
    oracle_lib.jzo_conv_backward_reshape(hptr(t), hptr(t2d), Cout_l, P, N)
    dcol = np.zeros(K * P * N, np.float32)
    oracle_lib.jzo_gemm(0, 0, K, P * N, Cout_l, 1.0, hptr(w), K, hptr(t2d), Cout_l, 0.0, hptr(dcol), K)
    dx = np.empty(Cin_l * P * N, np.float32)
    oracle_lib.jzo_col2im(hptr(dcol), hptr(dx), Cin_l, H, W, 3, 3, 1, 1, 1, 1, H, W, N)
    gdx = to_dev(np.full(Cin_l * P * N, np.nan, np.float32))
    gpu.conv2d_backward_data(dp(t), dp(w), dptr(gdx), Cin_l, H, W, Cout_l, 3, 3, 1, 1, 1, 1, H, W, N)
    got = to_host(gdx)
    assert np.isfinite(got).all()
    assert rel_err(got, dx) <= TOL_GEMM
