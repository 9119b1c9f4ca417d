"""The bandwidth-bound kernels at launch sizes of 512 MB and more (the threshold is 384 MB), where their loads and
stores carry the non-temporal hint (a separate template instance of every kernel).

A hinted launch must produce what the plain launch produces.  Elementwise forms are run
once over the whole buffer (hinted) and once in pieces that stay below the threshold
(plain) and compared bit for bit; reductions and normalisations are compared with torch on
the device in float64 within the reduction tolerance, the index-valued ones exactly.
torch is device-memory plumbing and the float64 reference here, as in the other tests of
floating-point kernels.
"""
import ctypes as C

import pytest

pytestmark = pytest.mark.gpu

TOL_RED = 1e-4
THRESHOLD = 512 << 20


def dptr(t):
    return C.c_void_p(t.data_ptr())


@pytest.fixture(scope="module")
def jz(gpu):
    return gpu


def randn(*shape, seed=0):
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return torch.randn(*shape, generator=g, device="cuda")


def test_elementwise_whole_against_pieces(jz):
    import torch
    n = (1 << 26) + 8                      # two buffers of 256 MB: past the threshold
    a, b = randn(n, seed=1), randn(n, seed=2)
    whole, pieces = torch.empty_like(a), torch.empty_like(a)
    assert 2 * n * 4 >= THRESHOLD
    cuts = [0, n // 4, n // 2, 3 * n // 4, n]
    cuts = [c // 4 * 4 for c in cuts[:-1]] + [n]       # pieces keep float4 alignment

    def both(call):
        call(whole, a, b, 0, n)
        for lo, hi in zip(cuts[:-1], cuts[1:]):
            call(pieces, a, b, lo, hi)
        torch.cuda.synchronize()
        assert torch.equal(whole, pieces)

    both(lambda o, x, y, lo, hi: jz.copy(dptr(o[lo:]), dptr(x[lo:]), hi - lo))
    assert torch.equal(whole, a)
    both(lambda o, x, y, lo, hi: jz.exp(dptr(o[lo:]), dptr(x[lo:]), hi - lo))
    both(lambda o, x, y, lo, hi: jz.axpby(dptr(o[lo:]), dptr(x[lo:]), dptr(y[lo:]), hi - lo, 0.5, 2.0))
    assert torch.equal(whole, 0.5 * a + 2.0 * b)
    both(lambda o, x, y, lo, hi: jz.hadamard(dptr(o[lo:]), dptr(x[lo:]), dptr(y[lo:]), hi - lo))
    both(lambda o, x, y, lo, hi: jz.mse_grad(dptr(o[lo:]), dptr(x[lo:]), dptr(y[lo:]), hi - lo, 1.0 / 128))
    # in place: one buffer of 512 MB
    big = randn(1 << 27, seed=3)
    ref = big * 3.0 + 1.0
    jz.affine_inplace(dptr(big), big.numel(), 3.0, 1.0)
    torch.cuda.synchronize()
    assert torch.equal(big, ref)


def test_reductions(jz):
    import torch
    numrow, numcol = 8192, 16384           # 512 MB, column-major: tensor (numcol, numrow)
    a = randn(numcol, numrow, seed=4)
    a64 = a.double()
    out_c, out_r = torch.empty(numcol, device="cuda"), torch.empty(numrow, device="cuda")
    jz.sum_cols(dptr(out_c), dptr(a), numrow, numcol, numrow)
    jz.sum_rows(dptr(out_r), dptr(a), numrow, numcol, numrow)
    scale_c = a64.abs().sum(1).norm().item()
    scale_r = a64.abs().sum(0).norm().item()
    assert (out_c.double() - a64.sum(1)).norm().item() <= TOL_RED * scale_c
    assert (out_r.double() - a64.sum(0)).norm().item() <= TOL_RED * scale_r
    jz.max_cols(dptr(out_c), dptr(a), numrow, numcol, numrow)
    assert torch.equal(out_c, a.max(1).values)
    idx = torch.empty(numcol, device="cuda", dtype=torch.int32)
    ties = torch.randint(-3, 4, (numcol, numrow), device="cuda").float()
    jz.argmax_cols(dptr(idx), dptr(ties), numrow, numcol, numrow)
    # the first maximum wins
    pos = torch.arange(numrow, device="cuda", dtype=torch.int32)[None, :].expand(numcol, numrow)
    first = torch.where(ties == ties.max(1, keepdim=True).values, pos, numrow).min(1).values.int()
    assert torch.equal(idx, first)
    del ties, pos
    one = torch.empty(1, device="cuda")
    jz.nrm2(dptr(one), dptr(a), a.numel())
    exact = a64.norm().item()
    assert abs(one.item() - exact) <= TOL_RED * exact
    b = randn(numcol, numrow, seed=5)
    jz.mse_loss(dptr(one), dptr(a), dptr(b), a.numel(), 1.0 / numcol)
    exact = ((a - b).double() ** 2).sum().item() / numcol
    assert abs(one.item() - exact) <= TOL_RED * exact
    # matrix-vector products with the 512 MB matrix
    x = randn(numrow, seed=6)
    y = torch.empty(numcol, device="cuda")
    jz.gemv(dptr(a), dptr(x), dptr(y), numrow, numcol, 1, numrow, 1, 1, 1.0, 0.0)     # y = A^T x
    want = a64 @ x.double()
    assert (y.double() - want).norm().item() <= TOL_RED * want.norm().item() + 1e-3
    x2 = randn(numcol, seed=7)
    y2 = torch.empty(numrow, device="cuda")
    jz.gemv(dptr(a), dptr(x2), dptr(y2), numrow, numcol, 0, numrow, 1, 1, 1.0, 0.0)   # y = A x
    want = a64.T @ x2.double()
    assert (y2.double() - want).norm().item() <= TOL_RED * want.norm().item() + 1e-3
    # bias broadcast in place
    bias = randn(numrow, seed=8)
    ref = a + bias[None, :]
    jz.add_bias(dptr(a), dptr(bias), numrow, numcol)
    torch.cuda.synchronize()
    assert torch.equal(a, ref)


def test_softmax_both_directions(jz):
    import torch
    numrow, numcol = 16384, 8192           # 512 MB
    a = randn(numcol, numrow, seed=9) * 2
    out = torch.empty_like(a)
    jz.softmax_cols(dptr(out), dptr(a), numrow, numcol, numrow)
    ref = torch.softmax(a.double(), dim=1)
    assert (out.double() - ref).abs().max().item() <= TOL_RED * ref.max().item()
    jz.softmax_rows(dptr(out), dptr(a), numrow, numcol, numrow)
    ref = torch.softmax(a.double(), dim=0)
    assert (out.double() - ref).abs().max().item() <= TOL_RED * ref.max().item()


def test_layernorm_and_optimiser(jz):
    import torch
    dim, N = 512, 131072 + 64              # streams of 268 MB each
    x = randn(N, dim, seed=10) * 2 + 0.3
    gamma, beta = randn(dim, seed=11) * 0.2 + 1, randn(dim, seed=12) * 0.2
    y, xhat, inv = torch.empty_like(x), torch.empty_like(x), torch.empty(N, device="cuda")
    jz.layernorm_fwd(dptr(y), dptr(xhat), dptr(inv), dptr(x), dptr(gamma), dptr(beta), dim, N)
    x64 = x.double()
    mu = x64.mean(1, keepdim=True)
    var = ((x64 - mu) ** 2).mean(1, keepdim=True)
    xh = (x64 - mu) / torch.sqrt(var + 1e-5)
    want = xh * gamma.double() + beta.double()
    assert (y.double() - want).norm().item() <= TOL_RED * want.norm().item()
    assert (xhat.double() - xh).norm().item() <= TOL_RED * xh.norm().item()
    dy = randn(N, dim, seed=13)
    dx = torch.empty_like(x)
    jz.layernorm_bwd(dptr(dx), dptr(dy), dptr(gamma), dptr(xhat), dptr(inv), dim, N)
    g = dy.double() * gamma.double()
    xh32 = xhat.double()
    wantdx = inv.double()[:, None] * (g - g.mean(1, keepdim=True) - xh32 * (g * xh32).mean(1, keepdim=True))
    assert (dx.double() - wantdx).norm().item() <= TOL_RED * wantdx.norm().item()
    dg, db = torch.empty(dim, device="cuda"), torch.empty(dim, device="cuda")
    jz.layernorm_param_grads(dptr(dg), dptr(db), dptr(dy), dptr(xhat), dim, N)
    wdg, wdb = (dy.double() * xh32).sum(0), dy.double().sum(0)
    assert (dg.double() - wdg).norm().item() <= TOL_RED * (dy.double() * xh32).abs().sum(0).norm().item()
    assert (db.double() - wdb).norm().item() <= TOL_RED * dy.double().abs().sum(0).norm().item()
    # the optimiser at 40 M parameters against the same call on two halves (plain instances)
    n = 40 << 20
    w, gr = randn(n, seed=14), randn(n, seed=15)
    m, v = randn(n, seed=16) * 0.1, randn(n, seed=17).abs() * 0.01
    w2, m2, v2 = w.clone(), m.clone(), v.clone()
    args = (3e-4, 0.9, 0.999, 1e-8, 0.01, 7)
    jz.adamw_step(dptr(w), dptr(gr), dptr(m), dptr(v), n, *args)
    h = n // 2
    for lo in (0, h):
        jz.adamw_step(dptr(w2[lo:]), dptr(gr[lo:]), dptr(m2[lo:]), dptr(v2[lo:]), h, *args)
    torch.cuda.synchronize()
    assert torch.equal(w, w2) and torch.equal(m, m2) and torch.equal(v, v2)


def test_transposed_and_patches(jz):
    import torch
    rows, cols = 8192, 8192 + 256          # two and three buffers of 264 MB
    A, B = randn(rows, cols, seed=18), randn(rows, cols, seed=19)     # logical matrices
    a = A.T.contiguous()                   # column-major
    bt = B.contiguous()                    # B stored transposed
    out = torch.empty(cols, rows, device="cuda")
    jz.axpby2d(dptr(out), rows, 0, dptr(a), rows, 0, dptr(bt), cols, 1, rows, cols, 0.5, 2.0)
    assert torch.equal(out.T, 0.5 * A + 2.0 * B)
    jz.copy2d(dptr(out), rows, 0, 0, 0, dptr(bt), cols, 1, 0, 0, rows, cols)
    assert torch.equal(out.T, B)
    # a row block of a vertical stack: nothing is turned, 1 KB runs
    dst = torch.zeros(cols, 2 * rows, device="cuda")
    jz.stack_copy_rows(dptr(dst), 2 * rows, rows, dptr(a), rows, cols, 0)
    assert torch.equal(dst[:, rows:], a) and not dst[:, :rows].any()
    del out, dst, a, bt, A, B
    # im2col with 540 MB of patches against the same call on two halves of the batch
    N, Cc, H, W, k = 120, 128, 32, 32, 3
    K, P = Cc * k * k, H * W
    x = randn(N, Cc * H * W, seed=20)
    col, col2 = torch.empty(N * P, K, device="cuda"), torch.empty(N * P, K, device="cuda")
    assert col.numel() * 4 >= THRESHOLD
    geom = (Cc, H, W, k, k, 1, 1, 1, 1, H, W)
    jz.im2col(dptr(x), dptr(col), *geom, N)
    h = N // 2
    jz.im2col(dptr(x), dptr(col2), *geom, h)
    jz.im2col(dptr(x[h:]), dptr(col2[h * P:]), *geom, N - h)
    torch.cuda.synchronize()
    assert torch.equal(col, col2)
