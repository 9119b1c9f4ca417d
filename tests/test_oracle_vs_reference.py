"""Validates the C restatement (oracle/jz_oracle.c) against the reference's
own CPU path compiled from its sources (oracle/_ref/libjzref.so).  Bit-exact
wherever the restatement claims to follow the reference's rounding; skipped
when the reference library was never built.  Runs without a GPU."""
import ctypes as C

import numpy as np
import pytest

import oracle
from util import hptr

ref = oracle.load_ref()
pytestmark = pytest.mark.skipif(ref is None, reason="oracle/_ref/libjzref.so not built")


def R(seed):
    return np.random.default_rng(seed)


def phys(logical, trans):
    """dense column-major physical buffer of a logical matrix stored with `trans`"""
    m = logical.T if trans else logical
    return np.ascontiguousarray(m.T).reshape(-1), m.shape[0], m.shape[1]


@pytest.mark.parametrize("ta", [0, 1])
@pytest.mark.parametrize("tb", [0, 1])
@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (4, 3, 5), (17, 9, 33), (2, 40, 1), (1, 7, 6)])
def test_dot(oracle_lib, ta, tb, m, n, k):
    r = R(m + n + k)
    A, ar, ac = phys(r.normal(size=(m, k)).astype(np.float32), ta)
    B, br, bc = phys(r.normal(size=(k, n)).astype(np.float32), tb)
    want = np.empty(m * n, np.float32)
    ref.jzref_dot(hptr(want), hptr(A), ar, ac, ta, hptr(B), br, bc, tb)
    got = np.empty(m * n, np.float32)
    oracle_lib.jzo_dot(hptr(got), hptr(A), ar, ta, hptr(B), br, tb, m, n, k)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("ta", [0, 1])
@pytest.mark.parametrize("tb", [0, 1])
def test_add_and_hadmd_flags(oracle_lib, ta, tb):
    r = R(ta * 2 + tb)
    rows, cols = 5, 8
    A, ar, ac = phys(r.normal(size=(rows, cols)).astype(np.float32), ta)
    B, br, bc = phys(r.normal(size=(rows, cols)).astype(np.float32), tb)
    want = np.empty(rows * cols, np.float32)
    flag = ref.jzref_add(hptr(want), hptr(A), ar, ac, ta, hptr(B), br, bc, tb, 1.5, -0.5)
    assert flag == 0                                           # cpp/core.hpp:420
    got = np.empty_like(want)
    oracle_lib.jzo_axpby2d(hptr(got), rows, 0, hptr(A), ar, ta, hptr(B), br, tb, rows, cols, 1.5, -0.5)
    assert np.array_equal(got, want)
    flag = ref.jzref_hadmd(hptr(want), hptr(A), ar, ac, ta, hptr(B), br, bc, tb)
    assert flag == 0                                           # cpp/matrix.hpp:436
    oracle_lib.jzo_hadamard2d(hptr(got), rows, 0, hptr(A), ar, ta, hptr(B), br, tb, rows, cols)
    assert np.array_equal(got, want)
    # in-place: the destination keeps its own layout
    A2 = A.copy()
    ref.jzref_add_inplace(hptr(A2), ar, ac, ta, hptr(B), br, bc, tb, 2.0, 3.0)
    got = A.copy()
    oracle_lib.jzo_axpby2d(hptr(got), ar, ta, hptr(A), ar, ta, hptr(B), br, tb, rows, cols, 2.0, 3.0)
    assert np.array_equal(got, A2)


UN = [(0, "jzo_exp", None), (1, "jzo_log", None), (2, "jzo_tanh", None), (3, "jzo_dtanh", None),
      (4, "jzo_square", None), (7, "jzo_relu", None), (8, "jzo_drelu", None), (9, "jzo_sqrt", None)]


@pytest.mark.parametrize("op,name,_", UN)
def test_unary(oracle_lib, op, name, _):
    n = 1001
    x = R(op).normal(0, 2, n).astype(np.float32)
    if op in (1, 9):
        x = np.abs(x) + 1e-3
    want, got = np.empty(n, np.float32), np.empty(n, np.float32)
    assert ref.jzref_unary(op, hptr(want), hptr(x), n, 0.0, 0.0) == 0
    getattr(oracle_lib, name)(hptr(got), hptr(x), n)
    assert np.array_equal(got, want)


def test_affine_eleminv_clamp(oracle_lib):
    n = 777
    x = R(5).normal(0, 2, n).astype(np.float32)
    want, got = np.empty(n, np.float32), np.empty(n, np.float32)
    ref.jzref_unary(5, hptr(want), hptr(x), n, 0.37, -1.25)
    oracle_lib.jzo_affine(hptr(got), hptr(x), n, 0.37, -1.25)
    assert np.array_equal(got, want)
    ref.jzref_unary(6, hptr(want), hptr(x), n, 0.1, 0.0)
    oracle_lib.jzo_eleminv(hptr(got), hptr(x), n, 0.1)
    assert np.array_equal(got, want)
    ref.jzref_unary(10, hptr(want), hptr(x), n, -0.5, 0.75)
    oracle_lib.jzo_clamp(hptr(got), hptr(x), n, -0.5, 0.75)
    assert np.array_equal(got, want)


def test_readme_chain(oracle_lib):
    r = R(9)
    m, k, n = 6, 5, 7
    A = r.normal(size=m * k).astype(np.float32)
    B = r.normal(size=k * n).astype(np.float32)
    want = np.empty(m * n, np.float32)
    ref.jzref_chain(hptr(want), hptr(A), m, k, hptr(B), n)
    c = np.empty(m * n, np.float32)
    oracle_lib.jzo_dot(hptr(c), hptr(A), m, 0, hptr(B), k, 0, m, n, k)
    oracle_lib.jzo_exp(hptr(c), hptr(c), m * n)
    oracle_lib.jzo_affine(hptr(c), hptr(c), m * n, 1.0, 1.0)
    oracle_lib.jzo_log(hptr(c), hptr(c), m * n)
    oracle_lib.jzo_affine(hptr(c), hptr(c), m * n, np.float32(1.0 / 5.0), 0.0)
    assert np.array_equal(c, want)


@pytest.mark.parametrize("trans", [0, 1])
@pytest.mark.parametrize("dim", [0, 1])
def test_sum_and_norm(oracle_lib, trans, dim):
    r = R(trans + 2 * dim)
    pr, pc = 7, 11
    A = r.normal(size=pr * pc).astype(np.float32)
    lr_, lc = (pc, pr) if trans else (pr, pc)
    nout = lc if dim == 0 else lr_
    want = np.empty(nout, np.float32)
    ref.jzref_sum(hptr(want), hptr(A), pr, pc, trans, dim)
    # sum over the logical dim `dim` == physical dim (dim xor trans)
    got = np.empty(nout, np.float32)
    oracle_lib.jzo_sum_phys(hptr(got), hptr(A), pr, pc, pr, dim ^ trans)
    assert np.array_equal(got, want)
    assert oracle_lib.jzo_norm(hptr(A), pr * pc) == ref.jzref_norm(hptr(A), pr * pc)


@pytest.mark.parametrize("ts", [0, 1])
def test_slice_and_stack(oracle_lib, ts):
    r = R(ts)
    L = r.normal(size=(9, 6)).astype(np.float32)
    A, ar, ac = phys(L, ts)
    want = np.empty(4 * 3, np.float32)
    ref.jzref_slice(hptr(want), hptr(A), ar, ac, ts, 2, 6, 1, 4)
    got = np.empty_like(want)
    oracle_lib.jzo_copy2d(hptr(got), 4, 0, 0, 0, hptr(A), ar, ts, 2, 1, 4, 3)
    assert np.array_equal(got, want)
    assert np.array_equal(want.reshape(3, 4).T, L[2:6, 1:4])
    for tm in (0, 1):
        Mv, mr, mc = phys(r.normal(size=(4, 3)).astype(np.float32), tm)
        A2 = A.copy()
        ref.jzref_slice_assign(hptr(A2), ar, ac, ts, 2, 6, 1, 4, hptr(Mv), mr, mc, tm)
        got = A.copy()
        oracle_lib.jzo_copy2d(hptr(got), ar, ts, 2, 1, hptr(Mv), mr, tm, 0, 0, 4, 3)
        assert np.array_equal(got, A2)
    for tb in (0, 1):
        for horizontal in (0, 1):
            Lb = r.normal(size=(9, 4) if horizontal else (5, 6)).astype(np.float32)
            B, br, bc = phys(Lb, tb)
            rows, cols = (9, 10) if horizontal else (14, 6)
            want = np.empty(rows * cols, np.float32)
            ref.jzref_stack2(hptr(want), horizontal, hptr(A), ar, ac, ts, hptr(B), br, bc, tb)
            got = np.zeros(rows * cols, np.float32)
            oracle_lib.jzo_copy2d(hptr(got), rows, 0, 0, 0, hptr(A), ar, ts, 0, 0, 9, 6)
            if horizontal:
                oracle_lib.jzo_copy2d(hptr(got), rows, 0, 0, 6, hptr(B), br, tb, 0, 0, 9, 4)
            else:
                oracle_lib.jzo_copy2d(hptr(got), rows, 0, 9, 0, hptr(B), br, tb, 0, 0, 5, 6)
            assert np.array_equal(got, want)


@pytest.mark.parametrize("rows,cols", [(1, 1), (10, 16), (37, 5)])
def test_softmax(oracle_lib, rows, cols):
    x = R(rows).normal(0, 3, rows * cols).astype(np.float32)
    want, got = np.empty_like(x), np.empty_like(x)
    ref.jzref_softmax(hptr(want), hptr(x), rows, cols, 0, 0)
    oracle_lib.jzo_softmax_cols(hptr(got), hptr(x), rows, cols, rows)
    assert np.array_equal(got, want)
    ref.jzref_softmax(hptr(want), hptr(x), rows, cols, 0, 1)
    oracle_lib.jzo_softmax_rows(hptr(got), hptr(x), rows, cols, rows)
    assert np.array_equal(got, want)
    m1, m2 = np.empty(cols, np.float32), np.empty(cols, np.float32)
    ref.jzref_max_cols(hptr(m1), hptr(x), rows, cols)
    oracle_lib.jzo_max_cols(hptr(m2), hptr(x), rows, cols, rows)
    assert np.array_equal(m1, m2)


def test_adam(oracle_lib):
    n = 513
    r = R(1)
    g0 = r.normal(size=n).astype(np.float32)
    m1, v1 = np.zeros(n, np.float32), np.zeros(n, np.float32)
    m2, v2 = m1.copy(), v1.copy()
    for it in range(1, 5):
        ga, gb = g0 * np.float32(it), g0 * np.float32(it)
        ref.jzref_adam_update(hptr(ga), hptr(m1), hptr(v1), n, 1e-3, 0.9, 0.999, 1e-8, it)
        oracle_lib.jzo_adam_update(hptr(gb), hptr(m2), hptr(v2), n, 1e-3, 0.9, 0.999, 1e-8, it)
        assert np.array_equal(ga, gb) and np.array_equal(m1, m2) and np.array_equal(v1, v2)


def test_layernorm(oracle_lib):
    dim, N = 24, 7
    r = R(2)
    x = r.normal(0.4, 2, dim * N).astype(np.float32)
    g = r.normal(1, .2, dim).astype(np.float32)
    b = r.normal(0, .2, dim).astype(np.float32)
    y1, h1, i1 = np.empty_like(x), np.empty_like(x), np.empty(N, np.float32)
    y2, h2, i2 = np.empty_like(x), np.empty_like(x), np.empty(N, np.float32)
    ref.jzref_layernorm_fwd(hptr(y1), hptr(h1), hptr(i1), hptr(x), hptr(g), hptr(b), dim, N)
    oracle_lib.jzo_layernorm_fwd(hptr(y2), hptr(h2), hptr(i2), hptr(x), hptr(g), hptr(b), dim, N)
    # the generic op chain sums with ones-GEMVs and rounds products separately;
    # the restatement follows the same order, so agreement is to the last ulps
    assert np.allclose(y2, y1, rtol=2e-6, atol=1e-6)
    assert np.allclose(h2, h1, rtol=2e-6, atol=1e-6) and np.allclose(i2, i1, rtol=1e-6)
    dy = r.normal(size=dim * N).astype(np.float32)
    dx1, dg1, db1 = np.empty_like(x), np.empty(dim, np.float32), np.empty(dim, np.float32)
    ref.jzref_layernorm_bwd(hptr(dx1), hptr(dg1), hptr(db1), hptr(dy), hptr(x), hptr(g), hptr(b), dim, N)
    dx2, dg2, db2 = np.empty_like(x), np.empty(dim, np.float32), np.empty(dim, np.float32)
    oracle_lib.jzo_layernorm_bwd(hptr(dx2), hptr(dy), hptr(g), hptr(h1), hptr(i1), dim, N)
    oracle_lib.jzo_layernorm_param_grads(hptr(dg2), hptr(db2), hptr(dy), hptr(h1), dim, N)
    assert np.allclose(dx2, dx1, rtol=1e-5, atol=1e-6)
    assert np.allclose(dg2, dg1, rtol=1e-5, atol=1e-6) and np.allclose(db2, db1, rtol=1e-5, atol=1e-6)


def test_layernorm_jvp(oracle_lib):
    """LayerNorm<float>::jvp (ml/layer.hpp:2690-2702) of the compiled reference, the
    restatement, and central differences of the reference's own forward pass along
    the tangent (float64 differences of a float32 forward: 1e-3)."""
    dim, N = 24, 7
    r = R(12)
    x = r.normal(0.4, 2, dim * N).astype(np.float32)
    g = r.normal(1, .2, dim).astype(np.float32)
    b = r.normal(0, .2, dim).astype(np.float32)
    u = r.normal(size=dim * N).astype(np.float32)
    y, h, inv = np.empty_like(x), np.empty_like(x), np.empty(N, np.float32)
    ref.jzref_layernorm_fwd(hptr(y), hptr(h), hptr(inv), hptr(x), hptr(g), hptr(b), dim, N)
    j1, j2 = np.empty_like(x), np.empty_like(x)
    ref.jzref_layernorm_jvp(hptr(j1), hptr(u), hptr(x), hptr(g), hptr(b), dim, N)
    oracle_lib.jzo_layernorm_jvp(hptr(j2), hptr(u), hptr(g), hptr(h), hptr(inv), dim, N)
    assert np.allclose(j2, j1, rtol=1e-5, atol=1e-6)
    # closed form in float64: d/de LN(x + e u) at e = 0
    X, U = x.reshape(N, dim).astype(np.float64), u.reshape(N, dim).astype(np.float64)

    def ln(z):
        mu = z.mean(1, keepdims=True)
        var = ((z - mu) ** 2).mean(1, keepdims=True)
        return (z - mu) / np.sqrt(var + 1e-5) * g + b
    e = 1e-6
    fd = (ln(X + e * U) - ln(X - e * U)) / (2 * e)
    assert np.allclose(j2.reshape(N, dim), fd, rtol=1e-4, atol=1e-5)
    # the tangent is not the backward pass: gamma multiplies outside the projection
    bw = np.empty_like(x)
    oracle_lib.jzo_layernorm_bwd(hptr(bw), hptr(u), hptr(g), hptr(h), hptr(inv), dim, N)
    assert not np.allclose(bw, j2, rtol=1e-3, atol=1e-4)


def test_logistic(oracle_lib):
    K, N = 10, 33
    r = R(3)
    x = r.normal(0, 2, K * N).astype(np.float32)
    lab = r.integers(0, K, N).astype(np.int32)
    onehot = np.zeros((N, K), np.float32)
    onehot[np.arange(N), lab] = 1
    g1, g2 = np.empty_like(x), np.empty_like(x)
    l1 = ref.jzref_logistic(hptr(g1), hptr(x), hptr(onehot.reshape(-1)), K, N)
    l2 = oracle_lib.jzo_softmax_xent(hptr(g2), hptr(x), hptr(lab), K, N, K)
    assert abs(l1 - l2) <= 2e-6 * abs(l1)
    assert np.allclose(g2, g1, rtol=1e-5, atol=1e-8)


CONV = [(2, 1, 5, 5, 3, 3, 1, 1), (2, 3, 8, 7, 3, 3, 1, 2), (1, 2, 6, 6, 2, 2, 0, 2), (2, 2, 7, 5, 5, 3, 2, 1)]


@pytest.mark.parametrize("case", CONV)
def test_im2col_col2im_through_the_reference_layer(oracle_lib, case):
    """With identity 2-D weights, zero bias and no ReLU the reference ConvLayer's
    output is its im2col matrix (ml/layer.hpp:2046-2050) and its input gradient
    is col2im of the upstream (ml/layer.hpp:2070-2081), so both index maps are
    pinned bit-exactly to the reference's private loops."""
    N, Cc, H, W, kH, kW, pad, stride = case
    Ho, Wo = (H + 2 * pad - kH) // stride + 1, (W + 2 * pad - kW) // stride + 1
    K, P = Cc * kH * kW, Ho * Wo
    Co = K
    r = R(sum(case))
    x = r.normal(size=Cc * H * W * N).astype(np.float32)
    w = np.eye(K, dtype=np.float32).reshape(-1)     # w2d(co, k) = delta
    b = np.zeros(Co, np.float32)
    out = np.empty(Co * P * N, np.float32)
    ref.jzref_conv_eval(hptr(out), hptr(x), hptr(w), hptr(b), N, Cc, H, W, Co, kH, kW, pad, stride, 0)
    args = (Cc, H, W, kH, kW, pad, pad, stride, stride, Ho, Wo, N)
    col = np.empty(K * P * N, np.float32)
    oracle_lib.jzo_im2col(hptr(x), hptr(col), *args)
    packed = np.empty_like(col)
    oracle_lib.jzo_conv_forward_reshape_bias(hptr(col), hptr(packed), hptr(b), Co, P, N)
    assert np.array_equal(packed, out)
    up = r.normal(size=Co * P * N).astype(np.float32)
    dx = np.empty_like(x)
    ref.jzref_conv_backward(hptr(dx), hptr(x), hptr(w), hptr(b), hptr(up), N, Cc, H, W, Co, kH, kW, pad, stride, 0)
    t2d = np.empty_like(up)
    oracle_lib.jzo_conv_backward_reshape(hptr(up), hptr(t2d), Co, P, N)
    dx2 = np.empty_like(x)
    oracle_lib.jzo_col2im(hptr(t2d), hptr(dx2), *args)
    assert np.array_equal(dx2, dx)


@pytest.mark.parametrize("case", [(2, 2, 4, 4, 3, 4, 4, 1, 2), (1, 3, 5, 3, 2, 3, 3, 0, 1), (2, 1, 3, 4, 2, 2, 2, 0, 2)])
def test_conv_layers_full(oracle_lib, case):
    """ConvLayer and convtransLayer forward/backward with random weights equal the
    restated pipeline (im2col/GEMM/reshape, GEMM/scatter)."""
    o = oracle_lib
    N, Cc, H, W, Co, kH, kW, pad, stride = case
    r = R(sum(case) + 1)
    # ── convolution
    Ho, Wo = (H + 2 * pad - kH) // stride + 1, (W + 2 * pad - kW) // stride + 1
    if Ho > 0 and Wo > 0:
        K, P = Cc * kH * kW, Ho * Wo
        x = r.normal(size=Cc * H * W * N).astype(np.float32)
        w = r.normal(size=Co * K).astype(np.float32)
        b = r.normal(size=Co).astype(np.float32)
        want = np.empty(Co * P * N, np.float32)
        ref.jzref_conv_eval(hptr(want), hptr(x), hptr(w), hptr(b), N, Cc, H, W, Co, kH, kW, pad, stride, 1)
        args = (Cc, H, W, kH, kW, pad, pad, stride, stride, Ho, Wo, N)
        col = np.empty(K * P * N, np.float32)
        o.jzo_im2col(hptr(x), hptr(col), *args)
        y2d = np.empty(Co * P * N, np.float32)
        o.jzo_gemm(1, 0, Co, P * N, K, 1.0, hptr(w), K, hptr(col), K, 0.0, hptr(y2d), Co)
        got = np.empty_like(want)
        o.jzo_conv_forward_reshape_bias(hptr(y2d), hptr(got), hptr(b), Co, P, N)
        o.jzo_relu(hptr(got), hptr(got), got.size)
        assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
    # ── transposed convolution: x (C*H*W, N) -> (Co*Ho*Wo, N)
    Ho, Wo = (H - 1) * stride - 2 * pad + kH, (W - 1) * stride - 2 * pad + kW
    Rr, Pin = Co * kH * kW, H * W
    x = r.normal(size=Cc * H * W * N).astype(np.float32)
    w = r.normal(size=Cc * Rr).astype(np.float32)       # (R, C_in) column-major
    b = r.normal(size=Co).astype(np.float32)
    want = np.empty(Co * Ho * Wo * N, np.float32)
    ref.jzref_convtrans_eval(hptr(want), hptr(x), hptr(w), hptr(b), N, Cc, H, W, Co, kH, kW, pad, stride, 0)
    x2d = np.empty_like(x)
    o.jzo_convtrans_reshape(hptr(x), hptr(x2d), Cc, Pin, N, 0)
    patches = np.empty(Rr * Pin * N, np.float32)
    o.jzo_gemm(0, 0, Rr, Pin * N, Cc, 1.0, hptr(w), Rr, hptr(x2d), Cc, 0.0, hptr(patches), Rr)
    got = np.empty_like(want)
    o.jzo_convtrans_scatter(hptr(patches), hptr(got), hptr(b), Co, Ho, Wo, H, W, kH, kW, pad, pad, stride, stride, N)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
    up = r.normal(size=want.size).astype(np.float32)
    dxw = np.empty_like(x)
    ref.jzref_convtrans_backward(hptr(dxw), hptr(x), hptr(w), hptr(b), hptr(up), N, Cc, H, W, Co, kH, kW, pad,
                                 stride, 0)
    tp = np.empty(Rr * Pin * N, np.float32)
    o.jzo_convtrans_gather(hptr(up), hptr(tp), Co, Ho, Wo, H, W, kH, kW, pad, pad, stride, stride, N)
    dx2d = np.empty(Cc * Pin * N, np.float32)
    o.jzo_gemm(1, 0, Cc, Pin * N, Rr, 1.0, hptr(w), Rr, hptr(tp), Rr, 0.0, hptr(dx2d), Cc)
    dxg = np.empty_like(x)
    o.jzo_convtrans_reshape(hptr(dx2d), hptr(dxg), Cc, Pin, N, 1)
    assert np.allclose(dxg, dxw, rtol=1e-5, atol=1e-6)
