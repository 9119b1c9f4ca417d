"""Pins the CPU oracle (oracle/jz_oracle.c) to the reference's own golden
vectors and to closed forms, so that a dropped term, a wrong sign or a
transposed operand in the restatement fails here.  Runs without a GPU.

Golden data are the values the reference's tests hold:
  * tests/basic.testdata (2x3 fixture of tests/testbasic.cu:11-16), committed
    as tests/golden/basic_chain.json by tests/golden/make_fixtures.py,
  * README.md:36-41, tests/testRocmOpsSmoke.cu:26-84,
    tests/testRocmDeviceProof.cu:36-41, tests/testbasic.cu:58-81,
    tests/testElementwiseReduceTorchDump.cu:36-64.
"""
import json
from pathlib import Path

import numpy as np
import pytest

from util import hptr

GOLD = Path(__file__).parent / "golden"


def cm(rows):
    """nested row list -> (column-major float32 vector, nrow, ncol)"""
    a = np.array(rows, dtype=np.float32)
    return np.ascontiguousarray(a.T).reshape(-1), a.shape[0], a.shape[1]


def as_rows(v, nrow, ncol):
    return np.asarray(v).reshape(ncol, nrow).T


def test_basic_chain_fixture(oracle_lib):
    """log(exp(-A/B) + exp(hadmd(B,A))) - (A.T()*B).rows(0,2) == basic.testdata"""
    o = oracle_lib
    gold = json.loads((GOLD / "basic_chain.json").read_text())
    A, ar, ac = cm([[1, 2, 3], [3, 4, 5]])
    B, _, _ = cm([[6, 7, 8], [9, 10, 11]])
    n = ar * ac
    negA = np.empty(n, np.float32)
    o.jzo_affine(hptr(negA), hptr(A), n, -1.0, 0.0)            # operator-(M) = add(0,-1)
    invB = np.empty(n, np.float32)
    o.jzo_eleminv(hptr(invB), hptr(B), n, 1.0)                 # A/B = hadmd(A, B.eleminv(1))
    q = np.empty(n, np.float32)
    o.jzo_hadamard2d(hptr(q), ar, 0, hptr(negA), ar, 0, hptr(invB), ar, 0, ar, ac)
    e1 = np.empty(n, np.float32)
    o.jzo_exp(hptr(e1), hptr(q), n)
    h = np.empty(n, np.float32)
    o.jzo_hadamard2d(hptr(h), ar, 0, hptr(B), ar, 0, hptr(A), ar, 0, ar, ac)
    e2 = np.empty(n, np.float32)
    o.jzo_exp(hptr(e2), hptr(h), n)
    s = np.empty(n, np.float32)
    o.jzo_axpby2d(hptr(s), ar, 0, hptr(e1), ar, 0, hptr(e2), ar, 0, ar, ac, 1.0, 1.0)
    lg = np.empty(n, np.float32)
    o.jzo_log(hptr(lg), hptr(s), n)
    AtB = np.empty(9, np.float32)
    o.jzo_dot(hptr(AtB), hptr(A), ar, 1, hptr(B), ar, 0, 3, 3, 2)  # A.T() (3x2) * B (2x3)
    top = np.empty(6, np.float32)
    o.jzo_copy2d(hptr(top), 2, 0, 0, 0, hptr(AtB), 3, 0, 0, 0, 2, 3)
    C = np.empty(n, np.float32)
    o.jzo_axpby2d(hptr(C), 2, 0, hptr(lg), 2, 0, hptr(top), 2, 0, 2, 3, 1.0, -1.0)
    assert gold["numrow"] == 2 and gold["numcol"] == 3 and gold["transpose"] == 0
    assert np.linalg.norm(C - np.array([float.fromhex(h) for h in gold["data"]], np.float32)) < 1e-5   # testbasic.cu:16


def test_readme_known_answer(oracle_lib):
    """README.md:29-41: log(exp(A*B)+1)/5 for A=[[1,2,3],[4,5,6]], B=[[.1,.2],[.3,.4],[.5,.6]]"""
    o = oracle_lib
    A, ar, ac = cm([[1, 2, 3], [4, 5, 6]])
    B, br, bc = cm([[.1, .2], [.3, .4], [.5, .6]])
    P = np.empty(4, np.float32)
    o.jzo_dot(hptr(P), hptr(A), ar, 0, hptr(B), br, 0, 2, 2, 3)
    E = np.empty(4, np.float32)
    o.jzo_exp(hptr(E), hptr(P), 4)
    o.jzo_affine(hptr(E), hptr(E), 4, 1.0, 1.0)
    L = np.empty(4, np.float32)
    o.jzo_log(hptr(L), hptr(E), 4)
    o.jzo_affine(hptr(L), hptr(L), 4, np.float32(1.0 / 5.0), 0.0)
    want = np.array([[0.461017, 0.571807], [0.981484, 1.28033]])
    assert np.allclose(as_rows(L, 2, 2), want, rtol=2e-6, atol=0)


def test_ops_smoke_known_answers(oracle_lib):
    """tests/testRocmOpsSmoke.cu:26-84 and tests/testRocmDeviceProof.cu:36-41"""
    o = oracle_lib
    A, _, _ = cm([[1, 2], [3, 4]])
    B, _, _ = cm([[5, 6], [7, 8]])
    out = np.empty(4, np.float32)
    o.jzo_axpby2d(hptr(out), 2, 0, hptr(A), 2, 0, hptr(B), 2, 0, 2, 2, 1.0, 1.0)
    assert np.array_equal(as_rows(out, 2, 2), [[6, 8], [10, 12]])
    o.jzo_affine(hptr(out), hptr(A), 4, 2.0, 0.0)
    assert np.array_equal(as_rows(out, 2, 2), [[2, 4], [6, 8]])
    o.jzo_hadamard2d(hptr(out), 2, 0, hptr(A), 2, 0, hptr(B), 2, 0, 2, 2)
    assert np.array_equal(as_rows(out, 2, 2), [[5, 12], [21, 32]])
    s = np.empty(2, np.float32)
    o.jzo_sum_phys(hptr(s), hptr(A), 2, 2, 2, 0)      # sum(A,0) = [4,6]
    assert np.array_equal(s, [4, 6])
    o.jzo_sum_phys(hptr(s), hptr(A), 2, 2, 2, 1)      # sum(A,1) = [3,7]
    assert np.array_equal(s, [3, 7])
    o.jzo_eleminv(hptr(out), hptr(A), 4, 1.0)
    assert np.array_equal(as_rows(out, 2, 2), np.array([[1, .5], [np.float32(1) / np.float32(3), .25]], np.float32))
    o.jzo_dot(hptr(out), hptr(A), 2, 0, hptr(B), 2, 0, 2, 2, 2)
    assert np.array_equal(as_rows(out, 2, 2), [[19, 22], [43, 50]])
    # transposed operands: A.T()*B and A*B.T() against numpy
    a, b = as_rows(A, 2, 2), as_rows(B, 2, 2)
    o.jzo_dot(hptr(out), hptr(A), 2, 1, hptr(B), 2, 0, 2, 2, 2)
    assert np.array_equal(as_rows(out, 2, 2), a.T @ b)
    o.jzo_dot(hptr(out), hptr(A), 2, 0, hptr(B), 2, 1, 2, 2, 2)
    assert np.array_equal(as_rows(out, 2, 2), a @ b.T)


def test_stack_and_slice_semantics(oracle_lib):
    """tests/testbasic.cu:58-81: columns/rows assignment then vstack/hstack."""
    o = oracle_lib
    A, _, _ = cm([[1, 2, 3], [3, 4, 5]])
    B, _, _ = cm([[6, 7, 8], [9, 10, 11]])
    T1, _, _ = cm([[1, 1], [1, 1]])
    T2, _, _ = cm([[-1, -1, -1]])
    o.jzo_copy2d(hptr(A), 2, 0, 0, 0, hptr(T1), 2, 0, 0, 0, 2, 2)      # A.columns(0,2,T)
    o.jzo_copy2d(hptr(B), 2, 0, 0, 0, hptr(T2), 1, 0, 0, 0, 1, 3)      # B.rows(0,1,T)
    v = np.zeros(12, np.float32)
    o.jzo_copy2d(hptr(v), 4, 0, 0, 0, hptr(A), 2, 0, 0, 0, 2, 3)
    o.jzo_copy2d(hptr(v), 4, 0, 2, 0, hptr(B), 2, 0, 0, 0, 2, 3)
    assert np.array_equal(as_rows(v, 4, 3), [[1, 1, 3], [1, 1, 5], [-1, -1, -1], [9, 10, 11]])
    h = np.zeros(12, np.float32)
    o.jzo_copy2d(hptr(h), 2, 0, 0, 0, hptr(A), 2, 0, 0, 0, 2, 3)
    o.jzo_copy2d(hptr(h), 2, 0, 0, 3, hptr(B), 2, 0, 0, 0, 2, 3)
    assert np.array_equal(as_rows(h, 2, 6), [[1, 1, 3, -1, -1, -1], [1, 1, 5, 9, 10, 11]])
    # a transposed source: logical (i,j) of A.T() is A(j,i)
    t = np.zeros(6, np.float32)
    o.jzo_copy2d(hptr(t), 3, 0, 0, 0, hptr(A), 2, 1, 0, 0, 3, 2)
    assert np.array_equal(as_rows(t, 3, 2), as_rows(A, 2, 3).T)


def test_transposed_add_bruteforce(oracle_lib):
    """Logical-index semantics of add/hadmd with mismatched flags (cpp/core.hpp:414-449)."""
    o = oracle_lib
    r = np.random.default_rng(0)
    rows, cols = 4, 7
    La, Lb = r.normal(size=(rows, cols)).astype(np.float32), r.normal(size=(rows, cols)).astype(np.float32)
    for ta in (0, 1):
        for tb in (0, 1):
            for to in (0, 1):
                # physical buffers: flag 1 stores the transpose column-major
                pa = (La if ta else La.T).reshape(-1).copy()
                pb = (Lb if tb else Lb.T).reshape(-1).copy()
                out = np.empty(rows * cols, np.float32)
                o.jzo_axpby2d(hptr(out), cols if to else rows, to, hptr(pa), cols if ta else rows, ta,
                              hptr(pb), cols if tb else rows, tb, rows, cols, 2.0, -3.0)
                want = np.float32(2.0) * La + np.float32(-3.0) * Lb
                got = out.reshape(rows, cols) if to else out.reshape(cols, rows).T
                assert np.array_equal(got, want)
                o.jzo_hadamard2d(hptr(out), cols if to else rows, to, hptr(pa), cols if ta else rows, ta,
                                 hptr(pb), cols if tb else rows, tb, rows, cols)
                got = out.reshape(rows, cols) if to else out.reshape(cols, rows).T
                assert np.array_equal(got, La * Lb)


def test_elementwise_reduce_closed_forms(oracle_lib):
    """tests/testElementwiseReduceTorchDump.cu:36-64 inputs; column/row sums and maxima."""
    o = oracle_lib
    vals = np.array([-3.0, -1.5, -0.25, 0.0, 0.5, 1.25, 2.0, 3.5, 4.0, -2.0, 0.75, 5.0], np.float32)  # 3x4
    s0 = np.empty(4, np.float32)
    o.jzo_sum_phys(hptr(s0), hptr(vals), 3, 4, 3, 0)
    assert np.allclose(s0, vals.reshape(4, 3).sum(1))
    s1 = np.empty(3, np.float32)
    o.jzo_sum_phys(hptr(s1), hptr(vals), 3, 4, 3, 1)
    assert np.allclose(s1, vals.reshape(4, 3).sum(0))
    m = np.empty(4, np.float32)
    o.jzo_max_cols(hptr(m), hptr(vals), 3, 4, 3)
    assert np.array_equal(m, vals.reshape(4, 3).max(1))
    assert abs(o.jzo_norm(hptr(vals), 12) - np.linalg.norm(vals.astype(np.float64))) < 1e-5


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_vs_double(oracle_lib, ta, tb):
    """Method of tests/testCpuLinalg.cu:54-66,152-172: naive double triple loop, padded ld, alpha/beta."""
    o = oracle_lib
    r = np.random.default_rng(ta * 2 + tb)
    for m, n, k in ((1, 1, 1), (3, 4, 5), (7, 1, 9), (1, 6, 2), (17, 13, 1), (31, 29, 37)):
        for alpha in (0.0, 1.0, 0.75):
            for beta in (0.0, 1.0, -0.5):
                pad = 2
                lda, ldb, ldc = (k if ta else m) + pad, (n if tb else k) + pad, m + pad
                A = r.normal(size=lda * (m if ta else k)).astype(np.float32)
                B = r.normal(size=ldb * (k if tb else n)).astype(np.float32)
                C0 = r.normal(size=ldc * n).astype(np.float32)
                Am = A.reshape(-1, lda).T.astype(np.float64)
                Bm = B.reshape(-1, ldb).T.astype(np.float64)
                opA = Am[:k, :m].T if ta else Am[:m, :k]
                opB = Bm[:n, :k].T if tb else Bm[:k, :n]
                want = C0.reshape(n, ldc).T.astype(np.float64).copy()
                want[:m, :] = alpha * (opA @ opB) + beta * want[:m, :]
                C = C0.copy()
                o.jzo_gemm(ta, tb, m, n, k, alpha, hptr(A), lda, hptr(B), ldb, beta, hptr(C), ldc)
                got = C.reshape(n, ldc).T
                assert np.allclose(got[:m], want[:m], rtol=5e-3, atol=5e-3)
                assert np.array_equal(got[m:], C0.reshape(n, ldc).T[m:])  # padding untouched


def test_softmax_and_layernorm_invariants(oracle_lib):
    o = oracle_lib
    r = np.random.default_rng(3)
    rows, cols = 9, 11
    x = r.normal(0, 3, rows * cols).astype(np.float32)
    y = np.empty_like(x)
    o.jzo_softmax_cols(hptr(y), hptr(x), rows, cols, rows)
    X = x.reshape(cols, rows).astype(np.float64)
    want = np.exp(X - X.max(1, keepdims=True))
    want /= want.sum(1, keepdims=True)
    assert np.allclose(y.reshape(cols, rows), want, rtol=1e-5, atol=1e-7)
    o.jzo_softmax_rows(hptr(y), hptr(x), rows, cols, rows)
    want = np.exp(X - X.max(0, keepdims=True))
    want /= want.sum(0, keepdims=True)
    assert np.allclose(y.reshape(cols, rows), want, rtol=1e-5, atol=1e-7)
    # LayerNorm: float64 definition (tests/testTransformerRef.cu:82-100 restates the same)
    dim, N = 16, 5
    xx = r.normal(0.5, 2, dim * N).astype(np.float32)
    g = r.normal(1, .1, dim).astype(np.float32)
    b = r.normal(0, .1, dim).astype(np.float32)
    yy, xh, inv = np.empty_like(xx), np.empty_like(xx), np.empty(N, np.float32)
    o.jzo_layernorm_fwd(hptr(yy), hptr(xh), hptr(inv), hptr(xx), hptr(g), hptr(b), dim, N)
    Xd = xx.reshape(N, dim).astype(np.float64)
    mu, var = Xd.mean(1, keepdims=True), Xd.var(1, keepdims=True)
    assert np.allclose(yy.reshape(N, dim), (Xd - mu) / np.sqrt(var + 1e-5) * g + b, rtol=1e-5, atol=1e-6)
    # backward against central finite differences of the float64 forward
    dy = r.normal(size=dim * N).astype(np.float32)
    dx = np.empty_like(xx)
    o.jzo_layernorm_bwd(hptr(dx), hptr(dy), hptr(g), hptr(xh), hptr(inv), dim, N)

    def f(Xv):
        m_, v_ = Xv.mean(1, keepdims=True), Xv.var(1, keepdims=True)
        return (((Xv - m_) / np.sqrt(v_ + 1e-5) * g + b) * dy.reshape(N, dim)).sum()
    num = np.zeros_like(Xd)
    eps = 1e-5
    for idx in np.ndindex(*Xd.shape):
        Xp, Xm = Xd.copy(), Xd.copy()
        Xp[idx] += eps
        Xm[idx] -= eps
        num[idx] = (f(Xp) - f(Xm)) / (2 * eps)
    assert np.allclose(dx.reshape(N, dim), num, rtol=1e-3, atol=1e-4)


def test_adam_closed_form(oracle_lib):
    """Step 1 of Adam from zero state: update = alpha*g/(|g|+eps') ~ alpha*sign(g)."""
    o = oracle_lib
    g = np.array([0.5, -2.0, 3.0, -0.01], np.float32)
    g0 = g.copy()
    m, v = np.zeros(4, np.float32), np.zeros(4, np.float32)
    o.jzo_adam_update(hptr(g), hptr(m), hptr(v), 4, 1e-3, 0.9, 0.999, 1e-8, 1)
    assert np.allclose(g, 1e-3 * np.sign(g0), rtol=1e-5)
    assert np.allclose(m, 0.1 * g0, rtol=1e-6) and np.allclose(v, float(1 - np.float32(0.999)) * g0 * g0, rtol=1e-6)
    # float64 recurrence for 3 further steps
    md, vd = m.astype(np.float64), v.astype(np.float64)
    for it in (2, 3, 4):
        gi = g0 * np.float32(it)
        gg = gi.copy()
        o.jzo_adam_update(hptr(gg), hptr(m), hptr(v), 4, 1e-3, 0.9, 0.999, 1e-8, it)
        b1, b2 = float(np.float32(0.9)), float(np.float32(0.999))   # the floats the reference holds
        md = b1 * md + float(1 - np.float32(0.9)) * gi
        vd = b2 * vd + float(1 - np.float32(0.999)) * gi.astype(np.float64) ** 2
        want = float(np.float32(1e-3)) * (md / (1 - b1 ** it)) / (np.sqrt(vd / (1 - b2 ** it)) + 1e-8)
        assert np.allclose(gg, want, rtol=1e-5)


def naive_conv(x, w, bias, N, C, H, W, Co, kH, kW, pad, stride):
    """Direct convolution, the method of tests/testConvBackendParity.cu:46-85."""
    Ho, Wo = (H + 2 * pad - kH) // stride + 1, (W + 2 * pad - kW) // stride + 1
    out = np.zeros((N, Co, Ho, Wo))
    xi = x.reshape(N, C, H, W).astype(np.float64)
    wi = w.reshape(Co, C, kH, kW).astype(np.float64)
    for n in range(N):
        for co in range(Co):
            for oh in range(Ho):
                for ow in range(Wo):
                    acc = float(bias[co])
                    for ci in range(C):
                        for kh in range(kH):
                            for kw in range(kW):
                                ih, iw = oh * stride - pad + kh, ow * stride - pad + kw
                                if 0 <= ih < H and 0 <= iw < W:
                                    acc += xi[n, ci, ih, iw] * wi[co, ci, kh, kw]
                    out[n, co, oh, ow] = acc
    return out


@pytest.mark.parametrize("case", [(2, 2, 5, 6, 3, 3, 3, 1, 1), (1, 3, 7, 7, 2, 3, 3, 1, 2), (2, 1, 6, 5, 4, 2, 2, 0, 2)])
def test_conv_pipeline_vs_direct(oracle_lib, case):
    """im2col + GEMM + reshape/bias equals a direct convolution; col2im is im2col's adjoint."""
    o = oracle_lib
    N, C, H, W, Co, kH, kW, pad, stride = case
    Ho, Wo = (H + 2 * pad - kH) // stride + 1, (W + 2 * pad - kW) // stride + 1
    K, P = C * kH * kW, Ho * Wo
    r = np.random.default_rng(sum(case))
    x = r.normal(size=C * H * W * N).astype(np.float32)
    w = r.normal(size=Co * K).astype(np.float32)        # (K, C_out) column-major = (C_out,C,kH,kW) flat
    bias = r.normal(size=Co).astype(np.float32)
    args = (C, H, W, kH, kW, pad, pad, stride, stride, Ho, Wo, N)
    col = np.empty(K * P * N, np.float32)
    o.jzo_im2col(hptr(x), hptr(col), *args)
    y2d = np.zeros(Co * P * N, np.float32)
    o.jzo_gemm(1, 0, Co, P * N, K, 1.0, hptr(w), K, hptr(col), K, 0.0, hptr(y2d), Co)
    out = np.empty(Co * P * N, np.float32)
    o.jzo_conv_forward_reshape_bias(hptr(y2d), hptr(out), hptr(bias), Co, P, N)
    want = naive_conv(x, w, bias, N, C, H, W, Co, kH, kW, pad, stride)
    assert np.allclose(out.reshape(N, Co, Ho, Wo), want, rtol=1e-4, atol=1e-5)
    back = np.empty_like(out)
    o.jzo_conv_backward_reshape(hptr(out), hptr(back), Co, P, N)
    assert np.array_equal(back, (y2d.reshape(N * P, Co) + bias).reshape(-1))
    c2 = r.normal(size=K * P * N).astype(np.float32)
    dx = np.empty_like(x)
    o.jzo_col2im(hptr(c2), hptr(dx), *args)
    assert abs(np.dot(col.astype(np.float64), c2) - np.dot(x.astype(np.float64), dx)) < 1e-4


def test_convtrans_is_conv_adjoint(oracle_lib):
    """Transposed conv scatter is the adjoint of the gather with the same geometry
    (tests/testConvBackendParity.cu:88-124 checks the same relation through a direct loop)."""
    o = oracle_lib
    N, Co, Hi, Wi, kH, kW, pad, stride = 2, 3, 4, 5, 4, 4, 1, 2
    Ho, Wo = (Hi - 1) * stride - 2 * pad + kH, (Wi - 1) * stride - 2 * pad + kW
    R, Pin = Co * kH * kW, Hi * Wi
    r = np.random.default_rng(1)
    patches = r.normal(size=R * Pin * N).astype(np.float32)
    t = r.normal(size=Co * Ho * Wo * N).astype(np.float32)
    args = (Co, Ho, Wo, Hi, Wi, kH, kW, pad, pad, stride, stride, N)
    out = np.empty_like(t)
    zero = np.zeros(Co, np.float32)
    o.jzo_convtrans_scatter(hptr(patches), hptr(out), hptr(zero), *args)
    tp = np.empty_like(patches)
    o.jzo_convtrans_gather(hptr(t), hptr(tp), *args)
    assert abs(np.dot(out.astype(np.float64), t) - np.dot(patches.astype(np.float64), tp)) < 1e-3
    # bias-only: zero patches -> exact bias everywhere (tests/testUNet.cu:150-173)
    bias = r.normal(size=Co).astype(np.float32)
    o.jzo_convtrans_scatter(hptr(np.zeros_like(patches)), hptr(out), hptr(bias), *args)
    assert np.array_equal(out.reshape(N, Co, Ho * Wo), np.broadcast_to(bias[None, :, None], (N, Co, Ho * Wo)))
    # reshape round trip
    a = r.normal(size=Co * 7 * N).astype(np.float32)
    b_, c_ = np.empty_like(a), np.empty_like(a)
    o.jzo_convtrans_reshape(hptr(a), hptr(b_), Co, 7, N, 0)
    o.jzo_convtrans_reshape(hptr(b_), hptr(c_), Co, 7, N, 1)
    assert np.array_equal(a, c_)
    assert np.array_equal(b_.reshape(N, 7, Co), a.reshape(N, Co, 7).transpose(0, 2, 1))


def test_gelu_closed_form(oracle_lib):
    from math import erf, sqrt
    x = np.linspace(-5, 5, 101).astype(np.float32)
    y = np.empty_like(x)
    oracle_lib.jzo_gelu(hptr(y), hptr(x), x.size)
    want = np.array([0.5 * v * (1 + erf(v / sqrt(2))) for v in x.astype(np.float64)])
    assert np.allclose(y, want, rtol=1e-6, atol=1e-7)
    up = np.ones_like(x)
    d = np.empty_like(x)
    oracle_lib.jzo_dgelu_mul(hptr(d), hptr(x), hptr(up), x.size)
    eps = 1e-4
    num = [(0.5 * (v + eps) * (1 + erf((v + eps) / sqrt(2))) - 0.5 * (v - eps) * (1 + erf((v - eps) / sqrt(2)))) / (2 * eps)
           for v in x.astype(np.float64)]
    assert np.allclose(d, num, rtol=1e-4, atol=1e-6)


def test_embedding_lookup_is_the_one_hot_product(oracle_lib):
    """The lookup is defined by the reference's one-hot formulation
    (examples/demo_transformer.cu:133-149): it must equal E*onehot(tok) +
    P*onehot(pos) + bias computed by the oracle's own GEMM, bit for bit (every
    product with a zero adds an exact zero), including ids outside the table."""
    o = oracle_lib
    r = np.random.default_rng(11)
    d, V, S, B = 12, 7, 5, 3
    N = S * B
    E = r.normal(size=(V, d)).astype(np.float32)       # row v = column v of the (d, V) table
    Pm = r.normal(size=(S, d)).astype(np.float32)
    bias = r.normal(size=d).astype(np.float32)
    tok = r.integers(0, V, N).astype(np.int32)
    tok[3], tok[7] = -1, V                             # invalid ids: zero column
    oh = np.zeros((N, V), np.float32)
    for n, t in enumerate(tok):
        if 0 <= t < V:
            oh[n, t] = 1.0
    op = np.zeros((N, S), np.float32)
    op[np.arange(N), np.arange(N) % S] = 1.0
    want = np.zeros((N, d), np.float32)
    o.jzo_gemm(0, 0, d, N, V, 1.0, hptr(E), d, hptr(oh), V, 0.0, hptr(want), d)
    o.jzo_gemm(0, 0, d, N, S, 1.0, hptr(Pm), d, hptr(op), S, 1.0, hptr(want), d)
    got = np.empty((N, d), np.float32)
    o.jzo_embedding_fwd(hptr(got), hptr(E), hptr(Pm), None, hptr(tok), d, V, S, N)
    assert np.array_equal(got, want)
    assert np.array_equal(got[3], Pm[3 % S]) and np.array_equal(got[7], Pm[7 % S])
    o.jzo_embedding_fwd(hptr(got), hptr(E), hptr(Pm), hptr(bias), hptr(tok), d, V, S, N)
    assert np.array_equal(got, want + bias[None, :])


def test_one_hot_is_the_identity_indexed_by_label(oracle_lib):
    """one_hot (ml/util.cuh:295-303): column j is column Y(0,j) of the k x k
    identity; a label outside [0, k) gives the zero column."""
    r = np.random.default_rng(5)
    for k, n in ((10, 128), (7, 33), (256, 300)):
        lab = r.integers(0, k, n).astype(np.int32)
        lab[1], lab[n - 2] = -1, k
        out = np.full((n, k), 7.0, np.float32)          # row j of this array = column j of the k x n matrix
        oracle_lib.jzo_one_hot(hptr(out), hptr(lab), k, n)
        want = np.zeros((n, k), np.float32)
        ok = (lab >= 0) & (lab < k)
        want[ok] = np.eye(k, dtype=np.float32)[lab[ok]]
        assert np.array_equal(out, want)
        assert out.sum() == n - 2

