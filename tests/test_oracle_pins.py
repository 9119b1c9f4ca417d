"""CPU pins for the oracle functions that no reference golden vector and no
reference build entry point reaches directly: AdamW, the attention softmax and
its backward, GEMV with general alpha/beta/increments, the ReLU-derivative
product and the first-maximum argmax.  Each is held to an independent float64
statement of the mathematics (numpy / torch.optim written from the published
definitions), chosen so that a dropped term, a wrong sign, a swapped index or
a mask on the wrong side fails.  Runs without a GPU."""
import numpy as np
import pytest

from util import hptr


def r_(seed):
    return np.random.default_rng(seed)


# ── AdamW ─────────────────────────────────────────────────────────────────
def adamw_f64(w, g, m, v, lr, b1, b2, eps, wd, t):
    """Decoupled weight decay (Loshchilov & Hutter): w <- w(1 - lr*wd), then
    the bias-corrected Adam step lr*m_hat/(sqrt(v_hat)+eps)."""
    m = b1 * m + (1 - b1) * g
    v = b2 * v + (1 - b2) * g * g
    mh = m / (1 - b1 ** t)
    vh = v / (1 - b2 ** t)
    w = w * (1 - lr * wd) - lr * mh / (np.sqrt(vh) + eps)
    return w, m, v


@pytest.mark.parametrize("wd", [0.0, 0.01, 0.3])
def test_adamw_step_closed_form_and_torch(oracle_lib, wd):
    import torch
    r = r_(17)
    # the C ABI takes floats: give float64 exactly the values the oracle receives
    n = 100
    lr, b1, b2, eps, wd = (float(np.float32(c)) for c in (3e-3, 0.9, 0.999, 1e-8, wd))
    w0 = r.normal(0, 1, n).astype(np.float32)
    w = w0.copy()
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    w64, m64, v64 = w0.astype(np.float64), np.zeros(n), np.zeros(n)
    tw = torch.tensor(w0, dtype=torch.float64, requires_grad=True)
    opt = torch.optim.AdamW([tw], lr=lr, betas=(b1, b2), eps=eps, weight_decay=wd)
    for t in range(1, 8):
        g = r.normal(0, 0.5, n).astype(np.float32)
        g_before = g.copy()
        oracle_lib.jzo_adamw_step(hptr(w), hptr(g), hptr(m), hptr(v), n, lr, b1, b2, eps, wd, t)
        assert np.array_equal(g, g_before)                       # g is an input only
        w64, m64, v64 = adamw_f64(w64, g.astype(np.float64), m64, v64, lr, b1, b2, eps, wd, t)
        tw.grad = torch.tensor(g, dtype=torch.float64)
        opt.step()
        assert np.allclose(w, w64, rtol=1e-5, atol=1e-6), t
        assert np.allclose(m, m64, rtol=1e-5, atol=1e-7) and np.allclose(v, v64, rtol=1e-5, atol=1e-10)
        # torch divides by sqrt(v)/sqrt(bc2)+eps: same mathematics, other grouping
        assert np.allclose(w, tw.detach().numpy(), rtol=1e-5, atol=1e-6), t
    assert not np.allclose(w, w0, atol=1e-3)


def test_adamw_without_decay_is_adam_then_subtract(oracle_lib):
    """wd == 0 must be bit-identical to W -= adam_update(g) (ml/layer.hpp:108-111),
    whose adam_update is pinned against the compiled reference."""
    r = r_(3)
    n = 257
    w = r.normal(0, 1, n).astype(np.float32)
    g = r.normal(0, 1, n).astype(np.float32)
    m = r.normal(0, 0.1, n).astype(np.float32)
    v = r.uniform(0, 0.1, n).astype(np.float32)
    w2, g2, m2, v2 = w.copy(), g.copy(), m.copy(), v.copy()
    oracle_lib.jzo_adamw_step(hptr(w), hptr(g), hptr(m), hptr(v), n, 1e-3, 0.9, 0.999, 1e-8, 0.0, 5)
    oracle_lib.jzo_adam_update(hptr(g2), hptr(m2), hptr(v2), n, 1e-3, 0.9, 0.999, 1e-8, 5)
    assert np.array_equal(w, w2 - g2) and np.array_equal(m, m2) and np.array_equal(v, v2)


def test_adamw_first_step_sign(oracle_lib):
    """At step 1 from zero moments the Adam step is lr*g/(|g|+eps) = lr*sign(g)."""
    n, lr, wd = 64, 0.01, 0.1
    g = np.linspace(-2, 2, n).astype(np.float32)
    g[g == 0] = 0.5
    w = np.ones(n, np.float32)
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    oracle_lib.jzo_adamw_step(hptr(w), hptr(g), hptr(m), hptr(v), n, lr, 0.9, 0.999, 1e-8, wd, 1)
    assert np.allclose(w, (1 - lr * wd) - lr * np.sign(g), rtol=1e-5)


# ── attention softmax ────────────────────────────────────────────────────
def attn_softmax_f64(x, S, nblk, scale, causal, keys_along_rows):
    """x: nblk blocks of S*S floats, column-major. Returns probabilities in the
    same layout: softmax over keys of scale*x with key > query masked."""
    blocks = x.astype(np.float64).reshape(nblk, S, S)        # [b][col][row]
    out = np.empty_like(blocks)
    for b in range(nblk):
        phys = blocks[b].T                                    # phys[row, col]
        sc = phys * scale
        qk = sc.T if keys_along_rows else sc                  # qk[query, key]
        if causal:
            q, k = np.meshgrid(np.arange(S), np.arange(S), indexing="ij")
            qk = np.where(k > q, -1e9, qk)
        e = np.exp(qk - qk.max(axis=1, keepdims=True))
        p = e / e.sum(axis=1, keepdims=True)
        phys_out = p.T if keys_along_rows else p
        out[b] = phys_out.T
    return out.reshape(-1)


@pytest.mark.parametrize("keys_along_rows", [0, 1])
@pytest.mark.parametrize("causal", [0, 1])
@pytest.mark.parametrize("S,nblk", [(1, 2), (5, 3), (16, 4), (33, 2)])
def test_attn_softmax_against_float64(oracle_lib, S, nblk, causal, keys_along_rows):
    r = r_(S * 7 + nblk + causal)
    x = r.normal(0, 3, nblk * S * S).astype(np.float32)
    scale = 0.37
    got = np.empty_like(x)
    oracle_lib.jzo_attn_softmax(hptr(got), hptr(x), S, nblk, scale, causal, keys_along_rows)
    want = attn_softmax_f64(x, S, nblk, scale, causal, keys_along_rows)
    assert np.allclose(got, want, rtol=2e-6, atol=1e-9)
    # the mask is on the right side: query 0 sees key 0 only
    if causal and S > 1:
        blk = got.reshape(nblk, S, S)[0].T                   # phys[row, col]
        qk = blk.T if keys_along_rows else blk
        assert qk[0, 0] == pytest.approx(1.0, abs=1e-6) and np.all(qk[0, 1:] == 0.0)
        assert np.all(np.triu(qk, 1) == 0.0) and np.all(np.diag(qk) > 0)
    # in place
    y = x.copy()
    oracle_lib.jzo_attn_softmax(hptr(y), hptr(y), S, nblk, scale, causal, keys_along_rows)
    assert np.array_equal(y, got)


@pytest.mark.parametrize("keys_along_rows", [0, 1])
@pytest.mark.parametrize("S,nblk", [(4, 2), (9, 3)])
def test_attn_softmax_bwd_is_the_derivative_of_the_forward(oracle_lib, S, nblk, keys_along_rows):
    """dS must be the vector-Jacobian product of p = softmax(scale*x) with dA:
    checked against central differences of the float64 forward the test above
    pins the oracle's forward to."""
    r = r_(S + nblk)
    n = nblk * S * S
    x = r.normal(0, 1, n)
    dA = r.normal(0, 1, n).astype(np.float32)
    scale = 0.6
    p = attn_softmax_f64(x, S, nblk, scale, 0, keys_along_rows).astype(np.float32)
    got = np.empty(n, np.float32)
    oracle_lib.jzo_attn_softmax_bwd(hptr(got), hptr(p), hptr(dA), S, nblk, scale, keys_along_rows)
    h = 1e-6
    want = np.empty(n)
    for i in range(n):
        xp, xm = x.copy(), x.copy()
        xp[i] += h
        xm[i] -= h
        fp = attn_softmax_f64(xp, S, nblk, scale, 0, keys_along_rows)
        fm = attn_softmax_f64(xm, S, nblk, scale, 0, keys_along_rows)
        want[i] = np.dot(dA.astype(np.float64), (fp - fm) / (2 * h))
    assert np.allclose(got, want, rtol=2e-4, atol=2e-6)
    # in place on dA
    d2 = dA.copy()
    oracle_lib.jzo_attn_softmax_bwd(hptr(d2), hptr(p), hptr(d2), S, nblk, scale, keys_along_rows)
    assert np.array_equal(d2, got)


# ── GEMV ────────────────────────────────────────────────────────────────
@pytest.mark.parametrize("trans", [0, 1])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (0.75, 1.0), (-1.5, -0.5), (0.0, 2.0)])
@pytest.mark.parametrize("m,n,pad,incx,incy", [(1, 1, 0, 1, 1), (5, 3, 0, 1, 1), (7, 4, 2, 2, 3), (33, 65, 1, 3, 2)])
def test_gemv_general_against_float64(oracle_lib, trans, alpha, beta, m, n, pad, incx, incy):
    """y = alpha*op(A)x + beta*y, A physically m x n with leading dimension
    m + pad (cpp/cpulinalg.hpp:96-131), strided x and y."""
    r = r_(m * 100 + n)
    lda = m + pad
    A = r.normal(0, 1, lda * n).astype(np.float32)
    lenx, leny = (m, n) if trans else (n, m)
    x = r.normal(0, 1, lenx * incx).astype(np.float32)
    y = r.normal(0, 1, leny * incy).astype(np.float32)
    y0 = y.copy()
    oracle_lib.jzo_gemv(trans, m, n, alpha, hptr(A), lda, hptr(x), incx, beta, hptr(y), incy)
    A2 = A.reshape(n, lda)[:, :m].T.astype(np.float64)            # logical m x n
    op = A2.T if trans else A2
    want = alpha * (op @ x[::incx][:lenx].astype(np.float64)) + beta * y0[::incy][:leny].astype(np.float64)
    assert np.allclose(y[::incy][:leny], want, rtol=1e-5, atol=1e-5)
    # entries between the strides are untouched
    mask = np.ones(y.size, bool)
    mask[::incy] = False
    assert np.array_equal(y[mask], y0[mask])


def test_gemv_beta_zero_ignores_nans_in_y(oracle_lib):
    """beta == 0 overwrites y (BLAS convention the reference's sum() relies on:
    the result buffer comes dirty from the pool, cpp/matrix.hpp:74-91)."""
    A = np.arange(6, dtype=np.float32)
    x = np.ones(2, np.float32)
    y = np.full(3, np.nan, np.float32)
    oracle_lib.jzo_gemv(0, 3, 2, 1.0, hptr(A), 3, hptr(x), 1, 0.0, hptr(y), 1)
    assert np.array_equal(y, np.array([3, 5, 7], np.float32))


# ── d_relu product and argmax ───────────────────────────────────────────
def test_drelu_mul_against_numpy(oracle_lib):
    r = r_(9)
    n = 1001
    pre = r.normal(0, 1, n).astype(np.float32)
    pre[:5] = [0.0, -0.0, 1e-38, -1e-38, np.float32(np.nextafter(np.float32(0), np.float32(1)))]
    up = r.normal(0, 1, n).astype(np.float32)
    got = np.empty(n, np.float32)
    oracle_lib.jzo_drelu_mul(hptr(got), hptr(pre), hptr(up), n)
    want = np.where(pre > 0, up, np.float32(0.0) * up)
    assert np.array_equal(got, want)
    assert got[0] == 0 and got[1] == 0 and got[2] == up[2] and got[3] == 0 and got[4] == up[4]
    # equals hadmd(d_relu(pre), up) formed from the two separately pinned pieces
    d = np.empty(n, np.float32)
    oracle_lib.jzo_drelu(hptr(d), hptr(pre), n)
    h = np.empty(n, np.float32)
    oracle_lib.jzo_hadamard2d(hptr(h), n, 0, hptr(d), n, 0, hptr(up), n, 0, n, 1)
    assert np.array_equal(got, h)


@pytest.mark.parametrize("numrow,numcol,pad", [(1, 4, 0), (10, 128, 0), (7, 33, 3), (256, 50, 0), (300, 9, 4)])
def test_argmax_cols_first_maximum_with_ties(oracle_lib, numrow, numcol, pad):
    r = r_(numrow + numcol)
    ld = numrow + pad
    # few distinct values: ties in nearly every column
    a = r.integers(0, 4, ld * numcol).astype(np.float32)
    if pad:
        a.reshape(numcol, ld)[:, numrow:] = 100.0                 # padding must not be looked at
    got = np.empty(numcol, np.int32)
    oracle_lib.jzo_argmax_cols(hptr(got), hptr(a), numrow, numcol, ld)
    want = np.argmax(a.reshape(numcol, ld)[:, :numrow], axis=1)   # numpy returns the first maximum
    assert np.array_equal(got, want.astype(np.int32))
    mx = np.empty(numcol, np.float32)
    oracle_lib.jzo_max_cols(hptr(mx), hptr(a), numrow, numcol, ld)
    assert np.array_equal(mx, a.reshape(numcol, ld)[np.arange(numcol), got])
