"""GPU parity: every C-ABI entry point against the CPU oracle on identical
seeded inputs.  Tolerances are the ones the task fixes: bit-exact for index
maps and argmax; relative 1e-5 for elementwise ops; 1e-4 for reductions,
softmax and LayerNorm; 1e-3 for GEMM.
"""
import ctypes as C
import math

import numpy as np
import pytest

import oracle
from util import dev_empty, dp, dptr, hp, hptr, max_rel, rel_err, to_dev, to_host

pytestmark = pytest.mark.gpu

TOL_EW = 1e-5
TOL_RED = 1e-4
TOL_GEMM = 1e-3


def rng(seed):
    return np.random.default_rng(seed)


# ── flat elementwise ─────────────────────────────────────────────────────
UNARY = [
    ("exp", "jzo_exp", (), lambda r, n: r.normal(0, 2, n)),
    ("log", "jzo_log", (), lambda r, n: r.uniform(1e-3, 50, n)),
    ("tanh", "jzo_tanh", (), lambda r, n: r.normal(0, 2, n)),
    ("dtanh", "jzo_dtanh", (), lambda r, n: r.normal(0, 2, n)),
    ("square", "jzo_square", (), lambda r, n: r.normal(0, 3, n)),
    ("relu", "jzo_relu", (), lambda r, n: r.normal(0, 1, n)),
    ("drelu", "jzo_drelu", (), lambda r, n: r.normal(0, 1, n)),
    ("sqrt", "jzo_sqrt", (), lambda r, n: r.uniform(0, 9, n)),
    ("gelu", "jzo_gelu", (), lambda r, n: r.normal(0, 2, n)),
]


@pytest.mark.parametrize("n", [1, 3, 4, 255, 1024, 4099, 1 << 20])
@pytest.mark.parametrize("name,oname,extra,gen", UNARY, ids=[u[0] for u in UNARY])
def test_unary(gpu, oracle_lib, name, oname, extra, gen, n):
    x = gen(rng(n), n).astype(np.float32)
    ref = np.empty_like(x)
    getattr(oracle_lib, oname)(hptr(ref), hptr(x), n, *extra)
    dx = to_dev(x)
    dy = dev_empty(n)
    getattr(gpu, name)(dptr(dy), dptr(dx), n, *extra)
    got = to_host(dy)
    if name in ("square", "relu", "drelu", "sqrt"):
        assert np.array_equal(got, ref)
    elif name == "gelu":
        # oracle evaluates the closed form in double; the kernel in fp32
        assert np.max(np.abs(got - ref)) <= 1e-6 + TOL_EW * np.max(np.abs(ref))
    else:
        assert max_rel(got, ref, floor=1e-30) <= TOL_EW
    # in-place form returns the same numbers
    if name in ("exp", "log", "tanh", "dtanh", "square"):
        getattr(gpu, name + "_inplace")(dptr(dx), n)
        assert np.array_equal(to_host(dx), got)


@pytest.mark.parametrize("n", [1, 5, 1000, 65537])
def test_unary_unaligned_pointer(gpu, oracle_lib, n):
    """Sub-buffer views are not 16-byte aligned: the scalar path must agree."""
    x = rng(1).normal(0, 1, n + 3).astype(np.float32)
    dx = to_dev(x)
    dy = dev_empty(n + 3)
    gpu.exp(C.c_void_p(dy.data_ptr() + 4), C.c_void_p(dx.data_ptr() + 8), n)
    ref = np.empty(n, dtype=np.float32)
    oracle_lib.jzo_exp(hptr(ref), hp(x[2:2 + n].copy()), n)
    assert max_rel(to_host(dy)[1:1 + n], ref) <= TOL_EW


@pytest.mark.parametrize("n", [1, 7, 4096, 100003])
def test_affine_eleminv_clamp_fill_copy(gpu, oracle_lib, n):
    r = rng(n)
    x = r.normal(0, 2, n).astype(np.float32)
    x[np.abs(x) < 1e-3] = 0.5
    dx = to_dev(x)
    dy = dev_empty(n)
    ref = np.empty_like(x)

    oracle_lib.jzo_affine(hptr(ref), hptr(x), n, 0.37, -1.25)
    gpu.affine(dptr(dy), dptr(dx), n, 0.37, -1.25)
    assert np.array_equal(to_host(dy), ref)

    oracle_lib.jzo_eleminv(hptr(ref), hptr(x), n, 0.1)
    gpu.eleminv(dptr(dy), dptr(dx), n, 0.1)
    assert np.array_equal(to_host(dy), ref)

    oracle_lib.jzo_clamp(hptr(ref), hptr(x), n, -0.5, 0.75)
    gpu.clamp(dptr(dy), dptr(dx), n, -0.5, 0.75)
    assert np.array_equal(to_host(dy), ref)

    gpu.fill(dptr(dy), n, 3.5)
    assert np.array_equal(to_host(dy), np.full(n, 3.5, np.float32))
    gpu.copy(dptr(dy), dptr(dx), n)
    assert np.array_equal(to_host(dy), x)

    # in-place forms
    d2 = to_dev(x)
    gpu.affine_inplace(dptr(d2), n, 2.0, 1.0)
    oracle_lib.jzo_affine(hptr(ref), hptr(x), n, 2.0, 1.0)
    assert np.array_equal(to_host(d2), ref)
    d2 = to_dev(x)
    gpu.eleminv_inplace(dptr(d2), n, 1.0)
    oracle_lib.jzo_eleminv(hptr(ref), hptr(x), n, 1.0)
    assert np.array_equal(to_host(d2), ref)


@pytest.mark.parametrize("n", [1, 6, 2048, 77777])
def test_binary_flat(gpu, oracle_lib, n):
    r = rng(n + 1)
    a = r.normal(0, 1, n).astype(np.float32)
    b = r.normal(0, 1, n).astype(np.float32)
    da, db, do = to_dev(a), to_dev(b), dev_empty(n)
    ref = np.empty_like(a)
    oracle_lib.jzo_axpby2d(hptr(ref), n, 0, hptr(a), n, 0, hptr(b), n, 0, n, 1, 1.5, -0.25)
    gpu.axpby(dptr(do), dptr(da), dptr(db), n, 1.5, -0.25)
    assert np.array_equal(to_host(do), ref)
    oracle_lib.jzo_hadamard2d(hptr(ref), n, 0, hptr(a), n, 0, hptr(b), n, 0, n, 1)
    gpu.hadamard(dptr(do), dptr(da), dptr(db), n)
    assert np.array_equal(to_host(do), ref)
    oracle_lib.jzo_drelu_mul(hptr(ref), hptr(a), hptr(b), n)
    gpu.drelu_mul(dptr(do), dptr(da), dptr(db), n)
    assert np.array_equal(to_host(do), ref)
    oracle_lib.jzo_dgelu_mul(hptr(ref), hptr(a), hptr(b), n)
    gpu.dgelu_mul(dptr(do), dptr(da), dptr(db), n)
    assert np.max(np.abs(to_host(do) - ref)) <= 1e-6 + TOL_EW * np.max(np.abs(ref))
    # aliasing: out == a
    gpu.hadamard_inplace(dptr(da), dptr(db), n)
    oracle_lib.jzo_hadamard2d(hptr(ref), n, 0, hptr(a), n, 0, hptr(b), n, 0, n, 1)
    assert np.array_equal(to_host(da), ref)


# ── transpose-aware 2-D ops ──────────────────────────────────────────────
@pytest.mark.parametrize("rows,cols", [(1, 1), (3, 5), (33, 65), (128, 96), (257, 1000)])
@pytest.mark.parametrize("to,ta,tb", [(0, 0, 0), (0, 1, 0), (0, 0, 1), (0, 1, 1), (1, 0, 0), (1, 0, 1), (1, 1, 0)])
def test_axpby_hadamard_2d(gpu, oracle_lib, rows, cols, to, ta, tb):
    r = rng(rows * 1000 + cols)
    a = r.normal(0, 1, rows * cols).astype(np.float32)
    b = r.normal(0, 1, rows * cols).astype(np.float32)
    ldo = cols if to else rows
    lda = cols if ta else rows
    ldb = cols if tb else rows
    da, db, do = to_dev(a), to_dev(b), dev_empty(rows * cols)
    ref = np.empty(rows * cols, np.float32)
    oracle_lib.jzo_axpby2d(hptr(ref), ldo, to, hptr(a), lda, ta, hptr(b), ldb, tb, rows, cols, 0.5, 2.0)
    gpu.axpby2d(dptr(do), ldo, to, dptr(da), lda, ta, dptr(db), ldb, tb, rows, cols, 0.5, 2.0)
    assert np.array_equal(to_host(do), ref)
    oracle_lib.jzo_hadamard2d(hptr(ref), ldo, to, hptr(a), lda, ta, hptr(b), ldb, tb, rows, cols)
    gpu.hadamard2d(dptr(do), ldo, to, dptr(da), lda, ta, dptr(db), ldb, tb, rows, cols)
    assert np.array_equal(to_host(do), ref)


@pytest.mark.parametrize("rows,cols", [(4096, 4096), (8192, 2048 + 64), (1024, 16384 + 128)])
@pytest.mark.parametrize("to,ta,tb", [(0, 1, 0), (0, 0, 1), (0, 1, 1), (1, 0, 0)])
def test_transposed_operands_many_full_tiles(gpu, rows, cols, to, ta, tb):
    """Several thousand full 64 x 64 tiles: the form in which a workgroup walks a sequence of
    tiles with the next tile's operands in flight.  Checked against numpy's own transposes
    (s1*a + s2*b and a*b round as two products and a sum / one product in float32)."""
    r = rng(rows + cols + ta * 2 + tb)
    A = r.normal(0, 1, (rows, cols)).astype(np.float32)     # logical matrices
    B = r.normal(0, 1, (rows, cols)).astype(np.float32)
    phys = lambda M, t: np.ascontiguousarray(M if t else M.T).reshape(-1)   # column-major, or its transpose
    a, b = phys(A, ta), phys(B, tb)
    ldo, lda, ldb = (cols if to else rows), (cols if ta else rows), (cols if tb else rows)
    da, db, do = to_dev(a), to_dev(b), dev_empty(rows * cols)
    gpu.axpby2d(dptr(do), ldo, to, dptr(da), lda, ta, dptr(db), ldb, tb, rows, cols, 0.5, 2.0)
    want = np.float32(0.5) * A + np.float32(2.0) * B
    assert np.array_equal(to_host(do), phys(want, to))
    gpu.hadamard2d(dptr(do), ldo, to, dptr(da), lda, ta, dptr(db), ldb, tb, rows, cols)
    assert np.array_equal(to_host(do), phys(A * B, to))
    if ta != to:
        gpu.copy2d(dptr(do), ldo, to, 0, 0, dptr(da), lda, ta, 0, 0, rows, cols)
        assert np.array_equal(to_host(do), phys(A, to))


@pytest.mark.parametrize("ts", [0, 1])
@pytest.mark.parametrize("td", [0, 1])
def test_slice_and_stack(gpu, oracle_lib, ts, td):
    r = rng(ts * 2 + td)
    R, Cc = 70, 45            # logical source shape
    src = r.normal(0, 1, R * Cc).astype(np.float32)
    lds = Cc if ts else R
    dsrc = to_dev(src)
    # extract logical block [5:40, 3:30]
    rows, cols = 35, 27
    ref = np.zeros(rows * cols, np.float32)
    oracle_lib.jzo_copy2d(hptr(ref), rows, 0, 0, 0, hptr(src), lds, ts, 5, 3, rows, cols)
    dout = dev_empty(rows * cols)
    gpu.slice_extract(dptr(dout), rows, dptr(dsrc), lds, ts, 5, 3, rows, cols)
    assert np.array_equal(to_host(dout), ref)
    # assign it into a destination with its own flag at (2, 4)
    DR, DC = 50, 40
    dst0 = r.normal(0, 1, DR * DC).astype(np.float32)
    ldd = DC if td else DR
    refd = dst0.copy()
    oracle_lib.jzo_copy2d(hptr(refd), ldd, td, 2, 4, hptr(ref), rows, 0, 0, 0, rows, cols)
    ddst = to_dev(dst0)
    gpu.slice_assign(dptr(ddst), ldd, td, 2, 4, dptr(dout), rows, 0, rows, cols)
    assert np.array_equal(to_host(ddst), refd)
    # stack copies: logical source placed at a column / row offset
    big = np.zeros(R * (Cc + 7), np.float32)
    refb = big.copy()
    oracle_lib.jzo_copy2d(hptr(refb), R, 0, 0, 7, hptr(src), lds, ts, 0, 0, R, Cc)
    dbig = to_dev(big)
    gpu.stack_copy_cols(dptr(dbig), R, 7, dptr(dsrc), lds, (R * Cc) // lds, ts)
    assert np.array_equal(to_host(dbig), refb)
    tall = np.zeros((R + 9) * Cc, np.float32)
    reft = tall.copy()
    oracle_lib.jzo_copy2d(hptr(reft), R + 9, 0, 9, 0, hptr(src), lds, ts, 0, 0, R, Cc)
    dtall = to_dev(tall)
    gpu.stack_copy_rows(dptr(dtall), R + 9, 9, dptr(dsrc), lds, (R * Cc) // lds, ts)
    assert np.array_equal(to_host(dtall), reft)


# ── reductions ───────────────────────────────────────────────────────────
SHAPES_RED = [(1, 1), (1, 1000), (1000, 1), (3, 8192), (10, 128), (64, 64), (7, 300), (33, 100), (1, 4096), (256, 4096), (257, 33),
              (512, 16384), (1024, 1024), (100000, 3), (1 << 20, 1)]


@pytest.mark.parametrize("numrow,numcol", SHAPES_RED)
def test_sums(gpu, oracle_lib, numrow, numcol):
    a = rng(numrow + numcol).normal(0, 1, numrow * numcol).astype(np.float32)
    da = to_dev(a)
    # the serial fp32 oracle and a tree reduction differ by rounding only:
    # compare both against float64 and require the kernel to be no worse than 1e-4
    A = a.reshape(numcol, numrow).astype(np.float64)  # row j = physical column j
    for which, exact in (("sum_cols", A.sum(axis=1)), ("sum_rows", A.sum(axis=0))):
        n_out = exact.size
        ref = np.empty(n_out, np.float32)
        oracle_lib.jzo_sum_phys(hptr(ref), hptr(a), numrow, numcol, numrow, 0 if which == "sum_cols" else 1)
        out = dev_empty(n_out)
        getattr(gpu, which)(dptr(out), dptr(da), numrow, numcol, numrow)
        got = to_host(out)
        scale = np.linalg.norm(np.abs(A).sum(axis=1 if which == "sum_cols" else 0))
        assert np.linalg.norm(got - exact) <= TOL_RED * scale
        assert np.linalg.norm(got - ref) <= TOL_RED * scale


def test_sum_with_padding_ld(gpu, oracle_lib):
    numrow, numcol, ld = 37, 50, 48
    a = rng(5).normal(0, 1, ld * numcol).astype(np.float32)
    da = to_dev(a)
    for which, dimp, n_out in (("sum_cols", 0, numcol), ("sum_rows", 1, numrow)):
        ref = np.empty(n_out, np.float32)
        oracle_lib.jzo_sum_phys(hptr(ref), hptr(a), numrow, numcol, ld, dimp)
        out = dev_empty(n_out)
        getattr(gpu, which)(dptr(out), dptr(da), numrow, numcol, ld)
        assert rel_err(to_host(out), ref) <= TOL_RED


@pytest.mark.parametrize("n", [1, 3, 1000, 65536, 1 << 22])
def test_nrm2(gpu, oracle_lib, n):
    x = rng(n).normal(0, 1, n).astype(np.float32)
    out = dev_empty(1)
    gpu.nrm2(dptr(out), dp(x), n)
    exact = np.linalg.norm(x.astype(np.float64))
    assert abs(to_host(out)[0] - exact) <= TOL_RED * exact
    # the oracle's serial fp32 accumulation (cpp/core.hpp:337-344) itself drifts
    # from the exact value by up to ~n*eps/2; the kernel must be inside that band
    band = max(TOL_RED, n * 6e-8) * exact
    assert abs(oracle_lib.jzo_norm(hptr(x), n) - exact) <= band
    assert abs(to_host(out)[0] - oracle_lib.jzo_norm(hptr(x), n)) <= band


@pytest.mark.parametrize("n,nb", [(1, 1), (4096, 4096), (3 * 1000, 1000), (8192 + 5, 7), (3072 * 128, 128)])
def test_mse_loss_and_grad(gpu, n, nb):
    """The squared-error head in one launch each (ml/layer.hpp:214-226): the gradient rounds
    as 2.0 * (input - output) / nb does through the matrix operators (cpp/operators.hpp:236-264:
    `/ nb` is a multiplication by float(1.0 / nb)), so it is compared bit for bit; the value is a
    sum and gets the reduction tolerance."""
    r = rng(n + nb)
    pred = r.normal(0, 1, n).astype(np.float32)
    target = r.normal(0, 1, n).astype(np.float32)
    inv = np.float32(1.0 / nb)
    g = dev_empty(n)
    gpu.mse_grad(dptr(g), dp(pred), dp(target), n, float(inv))
    assert np.array_equal(to_host(g), ((pred - target) * np.float32(2.0)) * inv)
    out = dev_empty(1)
    gpu.mse_loss(dptr(out), dp(target), dp(pred), n, float(inv))
    d = (target - pred).astype(np.float32)
    exact = float(np.sum((d * d).astype(np.float32).astype(np.float64))) / nb
    assert abs(to_host(out)[0] - exact) <= TOL_RED * max(exact, 1e-30)
    gpu.mse_loss(dptr(out), dp(target), dp(pred), 0, 1.0)
    assert to_host(out)[0] == 0.0


@pytest.mark.parametrize("numrow,numcol", [(1, 5), (10, 128), (256, 16384), (1000, 7), (65, 65)])
def test_max_argmax_cols(gpu, oracle_lib, numrow, numcol):
    r = rng(numrow * 7 + numcol)
    # few distinct values -> many ties, so the first-maximum rule is exercised
    a = r.integers(-3, 4, numrow * numcol).astype(np.float32)
    da = to_dev(a)
    refm = np.empty(numcol, np.float32)
    refi = np.empty(numcol, np.int32)
    oracle_lib.jzo_max_cols(hptr(refm), hptr(a), numrow, numcol, numrow)
    oracle_lib.jzo_argmax_cols(hptr(refi), hptr(a), numrow, numcol, numrow)
    om = dev_empty(numcol)
    oi = dev_empty(numcol, np.int32)
    gpu.max_cols(dptr(om), dptr(da), numrow, numcol, numrow)
    gpu.argmax_cols(dptr(oi), dptr(da), numrow, numcol, numrow)
    assert np.array_equal(to_host(om), refm)
    assert np.array_equal(to_host(oi), refi)
    assert np.array_equal(refi, a.reshape(numcol, numrow).argmax(axis=1).astype(np.int32))


# ── GEMM family ──────────────────────────────────────────────────────────
def naive_gemm64(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc):
    """Double-precision reference, the method of tests/testCpuLinalg.cu:54-66."""
    Am = A.astype(np.float64).reshape(-1, lda).T  # physical (lda x cols)
    Bm = B.astype(np.float64).reshape(-1, ldb).T
    opA = Am[:k, :m].T if ta else Am[:m, :k]
    opB = Bm[:n, :k].T if tb else Bm[:k, :n]
    C0 = Cm.astype(np.float64).reshape(-1, ldc).T.copy()
    C0[:m, :n] = alpha * (opA @ opB) + beta * C0[:m, :n]
    return C0.T.reshape(-1)


GEMM_SHAPES = [(1, 1, 1), (2, 2, 2), (3, 5, 7), (1, 40, 33), (40, 1, 33), (17, 19, 1), (64, 64, 64),
               (128, 128, 16), (129, 127, 17), (33, 300, 9), (300, 33, 70), (256, 512, 128),
               (32, 1000, 288), (10, 128, 1254), (65, 250, 130),
               # full tiles with two, three and five K stages of 16: the stage loop runs in
               # pairs, and an odd count starts half a pair in
               (256, 256, 32), (128, 384, 48), (256, 128, 80),
               # four tiles and a contraction cut into 8 chunks of five stages each
               (256, 256, 640)]


@pytest.mark.parametrize("m,n,k", GEMM_SHAPES)
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_variants(gpu, oracle_lib, m, n, k, ta, tb):
    r = rng(m * 10007 + n * 101 + k)
    for pad, alpha, beta in ((0, 1.0, 0.0), (3, 0.75, -0.5), (0, 1.0, 1.0)):
        lda = (k if ta else m) + pad
        ldb = (n if tb else k) + pad
        ldc = m + pad
        A = r.normal(0, 1, lda * (m if ta else k)).astype(np.float32)
        B = r.normal(0, 1, ldb * (k if tb else n)).astype(np.float32)
        C0 = r.normal(0, 1, ldc * n).astype(np.float32)
        exact = naive_gemm64(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C0, ldc)
        ref = C0.copy()
        oracle_lib.jzo_gemm(ta, tb, m, n, k, alpha, hptr(A), lda, hptr(B), ldb, beta, hptr(ref), ldc)
        dC = to_dev(C0)
        gpu.gemm(dp(A), dp(B), dptr(dC), m, n, k, ta, tb, lda, ldb, ldc, alpha, beta)
        got = to_host(dC)
        assert rel_err(got, exact) <= TOL_GEMM
        assert rel_err(got, ref) <= TOL_GEMM
        if pad:
            # rows m..ldc-1 of every column must be untouched (tests/testCpuLinalg.cu:152-172)
            g2 = got.reshape(n, ldc)
            assert np.array_equal(g2[:, m:], C0.reshape(n, ldc)[:, m:])


# one extent of at most 16 against a long one: the matrix-vector forms (lanes along
# k with the thin operand in LDS, or lanes along the long extent with partial sums
# over k chunks), in both roles and all four layouts, with and without padded
# leading dimensions; (64, 1216, 512) and (1216, 64, 512) take full 64 x 64 tiles
THIN_SHAPES = [(3, 4100, 576), (576, 3, 5000), (8, 2052, 128), (1028, 5, 300), (4, 1024, 64),
               (1500, 7, 257), (2, 1027, 512), (64, 1216, 512), (1216, 64, 512),
               # nine to sixteen thin vectors; a short long-extent against a very long k (the contraction cut
               # into chunks in the dot form too): the dense layer of the CNN and the first layer of the MLP
               (10, 128, 12544), (10, 12544, 128), (12544, 10, 128), (256, 16, 4096), (16, 256, 4096),
               (12, 260, 1028), (300, 9, 4100), (16, 24, 2048), (13, 64, 640)]


@pytest.mark.parametrize("m,n,k", THIN_SHAPES)
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_thin_products(gpu, oracle_lib, m, n, k, ta, tb):
    r = rng(m * 7919 + n * 31 + k + 2 * ta + tb)
    for pad, alpha, beta in ((0, 1.0, 0.0), (4, 0.75, -0.5), (8, 1.0, 1.0)):
        lda = (k if ta else m) + pad
        ldb = (n if tb else k) + pad
        ldc = m + pad
        A = r.normal(0, 1, lda * (m if ta else k)).astype(np.float32)
        B = r.normal(0, 1, ldb * (k if tb else n)).astype(np.float32)
        C0 = r.normal(0, 1, ldc * n).astype(np.float32)
        exact = naive_gemm64(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C0, ldc)
        ref = C0.copy()
        oracle_lib.jzo_gemm(ta, tb, m, n, k, alpha, hptr(A), lda, hptr(B), ldb, beta, hptr(ref), ldc)
        dC = to_dev(C0)
        gpu.gemm(dp(A), dp(B), dptr(dC), m, n, k, ta, tb, lda, ldb, ldc, alpha, beta)
        got = to_host(dC)
        assert rel_err(got, exact) <= TOL_GEMM
        assert rel_err(got, ref) <= TOL_GEMM
        if pad:
            g2 = got.reshape(n, ldc)
            assert np.array_equal(g2[:, m:], C0.reshape(n, ldc)[:, m:])


@pytest.mark.parametrize("m,n,k,ta,tb", [
    (256, 512, 128, 0, 0),        # full tiles, unchecked loaders
    (129, 127, 17, 0, 1),         # ragged edges, checked loaders
    (256, 128, 8192, 0, 1),       # split along K: partial sums and their reduction
    (64, 1216, 512, 1, 0),        # 64 x 64 tiles
    (3, 4100, 576, 1, 0),         # thin, k contiguous in the big operand
    (576, 3, 5000, 0, 1),         # thin, long extent contiguous, k chunks
    (300, 1, 70, 0, 0), (1, 300, 70, 1, 0),   # matrix-vector forms
    (40, 50, 1, 0, 0),            # rank-1
])
def test_gemm_with_beta_zero_never_reads_c(gpu, m, n, k, ta, tb):
    """dot() hands the product a fresh block from the pool (cpp/hipmatrix.cpp:134-152,
    cpp/memory.hpp:50-97): whatever bits it holds, NaN included, must not reach the
    result when beta == 0."""
    r = rng(m + 3 * n + 7 * k)
    lda, ldb = (k if ta else m), (n if tb else k)
    A = r.normal(0, 1, m * k).astype(np.float32)
    B = r.normal(0, 1, k * n).astype(np.float32)
    C0 = np.full(m * n, np.nan, np.float32)
    exact = naive_gemm64(ta, tb, m, n, k, 1.0, A, lda, B, ldb, 0.0, np.zeros(m * n, np.float32), m)
    dC = to_dev(C0)
    gpu.gemm(dp(A), dp(B), dptr(dC), m, n, k, ta, tb, lda, ldb, m, 1.0, 0.0)
    got = to_host(dC)
    assert np.isfinite(got).all()
    assert rel_err(got, exact) <= TOL_GEMM


# A layer's two parameter gradients in one call (ml/layer.hpp:99-100).  The first group takes the
# kernel that adds up A on its way into LDS: 128 x 128 tiles with K cut into chunks, one / two / three
# K stages, 64 x 64, 32 x 256, 128 x 64, 64 x 128 and 256 x 32 tiles; the second group the plain
# product followed by the sum kernels (ragged, transposed A, plain B, thin, matrix-vector, rank-1).
ROWSUM_SHAPES = [(256, 128, 8192, 0, 1), (512, 512, 4096, 0, 1), (256, 256, 16, 0, 1), (256, 256, 32, 0, 1),
                 (128, 256, 48, 0, 1), (64, 1216, 512, 0, 1), (32, 256, 128, 0, 1), (256, 64, 1024, 0, 1),
                 (64, 256, 2048, 0, 1), (1024, 32, 512, 0, 1), (256, 128, 80, 0, 1),
                 (129, 127, 17, 0, 1), (256, 128, 512, 1, 1), (256, 128, 512, 0, 0), (256, 128, 512, 1, 0),
                 (576, 3, 5000, 0, 1), (300, 1, 70, 0, 0), (1, 300, 70, 1, 0), (40, 50, 1, 0, 1)]


@pytest.mark.parametrize("m,n,k,ta,tb", ROWSUM_SHAPES)
def test_gemm_rowsum(gpu, m, n, k, ta, tb):
    r = rng(m + 5 * n + 11 * k + ta + 2 * tb)
    for pad, alpha, beta in ((0, 1.0, 0.0), (4, 0.5, 1.5)):
        lda, ldb = (k if ta else m) + pad, (n if tb else k) + pad
        A = r.normal(0.1, 1, lda * (m if ta else k)).astype(np.float32)
        B = r.normal(0, 1, ldb * (k if tb else n)).astype(np.float32)
        C0 = r.normal(0, 1, m * n).astype(np.float32) if beta else np.full(m * n, np.nan, np.float32)
        exact = naive_gemm64(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, np.nan_to_num(C0), m)
        Am = A.astype(np.float64).reshape(-1, lda).T
        want_rs = (Am[:k, :m].T if ta else Am[:m, :k]).sum(axis=1)
        dC, dR = to_dev(C0), to_dev(np.full(m, np.nan, np.float32))
        gpu.gemm_rowsum(dp(A), dp(B), dptr(dC), dptr(dR), m, n, k, ta, tb, lda, ldb, m, alpha, beta)
        got, got_rs = to_host(dC), to_host(dR)
        assert np.isfinite(got).all() and np.isfinite(got_rs).all()
        assert rel_err(got, exact) <= TOL_GEMM
        assert rel_err(got_rs, want_rs) <= TOL_RED
        # the product itself is the plain entry point's, bit for bit
        dC2 = to_dev(C0)
        gpu.gemm(dp(A), dp(B), dptr(dC2), m, n, k, ta, tb, lda, ldb, m, alpha, beta)
        assert np.array_equal(got, to_host(dC2))


def test_gemm_rowsum_at_the_transformer_weight_gradient_shapes(gpu):
    """512 x 2048, 2048 x 512 and 512 x 512 over 16384 tokens: the sums against jzhip_sum_rows and
    float64, the product against the plain entry point bit for bit; twice in a row (the
    partial sums live in the workspace the next call rewrites)."""
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    N = 16384
    for m, n in ((512, 2048), (2048, 512), (512, 512), (512, 2048)):
        t = torch.randn(m * N, generator=g, device="cuda") + 0.05
        x = torch.randn(n * N, generator=g, device="cuda")
        dW, dW2 = torch.full((m * n,), float("nan"), device="cuda"), torch.empty(m * n, device="cuda")
        db, db2 = torch.full((m,), float("nan"), device="cuda"), torch.empty(m, device="cuda")
        gpu.gemm_rowsum(dptr(t), dptr(x), dptr(dW), dptr(db), m, n, N, 0, 1, m, n, m, 1.0, 0.0)
        gpu.gemm(dptr(t), dptr(x), dptr(dW2), m, n, N, 0, 1, m, n, m, 1.0, 0.0)
        gpu.sum_rows(dptr(db2), dptr(t), m, N, m)
        gpu.synchronize()
        assert torch.equal(dW, dW2)
        want = t.view(N, m).double().sum(dim=0)
        assert float((db.double() - want).norm() / want.norm()) <= 1e-5
        assert float((db - db2).norm() / db2.norm()) <= 1e-5


def test_gemm_rowsum_rejects_bad_arguments(gpu):
    from juzhen_amd import capi
    lib = capi.load()
    d = dev_empty(16)
    assert lib.jzhip_gemm_rowsum(dptr(d), dptr(d), dptr(d), None, 2, 2, 2, 0, 1, 2, 2, 2, 1.0, 0.0) == -1
    assert lib.jzhip_gemm_rowsum(dptr(d), dptr(d), dptr(d), dptr(d), 2, 0, 2, 0, 1, 2, 2, 2, 1.0, 0.0) == -1
    assert lib.jzhip_gemm_rowsum(dptr(d), dptr(d), dptr(d), dptr(d), 2, 2, 2, 0, 1, 1, 2, 2, 1.0, 0.0) == -1


def test_gemm_thin_products_at_the_output_convolution_size(gpu):
    """3 x 131072 x 576 (forward, TN) and 576 x 3 x 131072 (weight gradient, NT) of a
    64 -> 3 channel 3x3 convolution on 128 images of 32 x 32, against float64."""
    r = rng(99)
    K, n, co = 576, 131072, 3
    W = r.normal(0, 1 / math.sqrt(K), K * co).astype(np.float32)       # K x co
    col = r.normal(0, 1, K * n).astype(np.float32)                     # K x n
    dcol, dW = to_dev(col), to_dev(W)
    out = dev_empty(co * n)
    gpu.gemm(dptr(dW), dptr(dcol), dptr(out), co, n, K, 1, 0, K, K, co, 1.0, 0.0)
    Wm, Cm = W.astype(np.float64).reshape(co, K), col.astype(np.float64).reshape(n, K)
    want = Cm @ Wm.T                                                    # (n, co) == column-major co x n
    got = to_host(out)
    assert rel_err(got, want.reshape(-1)) <= TOL_GEMM
    g = dev_empty(K * co)
    gpu.gemm(dptr(dcol), dptr(out), dptr(g), K, co, n, 0, 1, K, co, K, 1.0, 0.0)
    want_g = got.astype(np.float64).reshape(n, co).T @ Cm               # (co, K) == column-major K x co
    assert rel_err(to_host(g), want_g.reshape(-1)) <= TOL_GEMM


# (10, 128, 2560): the split-K form; (5, 300, 64): thin; (40, 50, 1): rank-1; (300, 1, 70): matrix-vector --
# the fused entry point keeps those forms and runs the tail as separate kernels
# (128, 256, 48) and (256, 256, 16): full tiles with an odd number of K stages (three, one)
@pytest.mark.parametrize("m,n,k", [(3, 5, 7), (64, 64, 64), (129, 127, 17), (256, 512, 128), (128, 1024, 96),
                                   (10, 128, 2560), (5, 300, 64), (40, 50, 1), (300, 1, 70),
                                   (128, 256, 48), (256, 256, 16)])
@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1)])
@pytest.mark.parametrize("act", [0, 1, 2, 3, 4])
def test_gemm_fused_epilogue(gpu, m, n, k, ta, tb, act):
    """bias / activation / residual fused into the store of C: bit-identical to
    jzhip_gemm followed by the separate kernels, and within the GEMM tolerance
    of the float64 closed form (erf-GELU from math.erf)."""
    import math
    r = rng(m * 31 + n * 7 + k + act)
    lda, ldb = (k if ta else m), (n if tb else k)
    A = (r.normal(0, 1, lda * (m if ta else k)) / np.sqrt(k)).astype(np.float32)
    B = r.normal(0, 1, ldb * (k if tb else n)).astype(np.float32)
    bias = r.normal(0, 1, m).astype(np.float32)
    res = r.normal(0, 1, m * n).astype(np.float32)
    pre = r.normal(0, 1, m * n).astype(np.float32)      # saved pre-activation for act 3/4
    dA, dB, dbias, dres = to_dev(A), to_dev(B), to_dev(bias), to_dev(res)
    # separate kernels
    dC = dev_empty(m * n)
    daux = to_dev(pre) if act in (3, 4) else dev_empty(m * n)
    gpu.gemm(dptr(dA), dptr(dB), dptr(dC), m, n, k, ta, tb, lda, ldb, m, 1.0, 0.0)
    gpu.add_bias(dptr(dC), dptr(dbias), m, n)
    want_aux = to_host(dC).copy()
    if act == 1:
        gpu.relu(dptr(dC), dptr(dC), m * n)
    elif act == 2:
        gpu.gelu(dptr(dC), dptr(dC), m * n)
    elif act == 3:
        gpu.drelu_mul(dptr(dC), dptr(daux), dptr(dC), m * n)
    elif act == 4:
        gpu.dgelu_mul(dptr(dC), dptr(daux), dptr(dC), m * n)
    gpu.axpby(dptr(dC), dptr(dC), dptr(dres), m * n, 1.0, 1.0)
    want = to_host(dC)
    # fused
    dF = dev_empty(m * n)
    daux2 = to_dev(pre) if act in (3, 4) else dev_empty(m * n)
    gpu.gemm_fused(dptr(dA), dptr(dB), dptr(dF), m, n, k, ta, tb, lda, ldb, m, 1.0, 0.0, dptr(dbias), act,
                   dptr(daux2) if act else None, m, dptr(dres), m)
    got = to_host(dF)
    assert np.array_equal(got, want)
    if act in (1, 2):
        assert np.array_equal(to_host(daux2), want_aux)
    # closed form in float64
    Am = A.astype(np.float64).reshape(-1, lda).T
    Bm = B.astype(np.float64).reshape(-1, ldb).T
    opA = Am.T if ta else Am
    opB = Bm.T if tb else Bm
    v = opA @ opB + bias.astype(np.float64)[:, None]
    erf = np.vectorize(math.erf)
    P = pre.astype(np.float64).reshape(n, m).T
    if act == 1:
        v = np.maximum(v, 0)
    elif act == 2:
        v = 0.5 * v * (1 + erf(v / math.sqrt(2)))
    elif act == 3:
        v = v * (P > 0)
    elif act == 4:
        v = v * (0.5 * (1 + erf(P / math.sqrt(2))) + P * np.exp(-0.5 * P * P) / math.sqrt(2 * math.pi))
    v = v + res.astype(np.float64).reshape(n, m).T
    assert rel_err(got, v.T.reshape(-1)) <= TOL_GEMM


# Products with more full 128 x 128 tiles than workgroups fit on the chip at once (768), so
# that tiles start while others are half way and the XCD-wise tile order wraps unevenly
# (7 x 111 tiles).  A tile's arithmetic does not depend on when or where it runs, so the
# result must equal, bit for bit, the same product computed in column blocks of at most
# half that many tiles.  k = 32 is the shortest contraction with two K stages.
@pytest.mark.parametrize("m,n,k", [(1536, 16384, 512), (896, 14208, 32), (2048, 8320, 64)])
@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
@pytest.mark.parametrize("fused", [False, True])
def test_gemm_more_tiles_than_workgroups(gpu, m, n, k, ta, tb, fused):
    import torch
    assert (m // 128) * (n // 128) > 768 and (k // 16) % 2 == 0
    g = torch.Generator(device="cuda")
    g.manual_seed(m + n + k + 2 * ta + tb)
    lda, ldb = (k if ta else m), (n if tb else k)
    A = torch.randn(lda * (m if ta else k), generator=g, device="cuda") / math.sqrt(k)
    B = torch.randn(ldb * (k if tb else n), generator=g, device="cuda")
    bias = torch.randn(m, generator=g, device="cuda")
    res = torch.randn(m * n, generator=g, device="cuda")
    old = torch.randn(m * n, generator=g, device="cuda")
    whole, pieces = old.clone(), old.clone()
    aux_w, aux_p = torch.zeros(m * n, device="cuda"), torch.zeros(m * n, device="cuda")
    beta = 0.0 if fused else 0.5

    def run(C_, aux_, col0, cols):
        # columns [col0, col0 + cols) of op(B) and C
        b_off = col0 if tb else col0 * ldb
        pb = C.c_void_p(B.data_ptr() + 4 * b_off)
        pc = C.c_void_p(C_.data_ptr() + 4 * col0 * m)
        if fused:
            gpu.gemm_fused(dptr(A), pb, pc, m, cols, k, ta, tb, lda, ldb, m, 1.0, beta, dptr(bias), 2,
                           C.c_void_p(aux_.data_ptr() + 4 * col0 * m), m,
                           C.c_void_p(res.data_ptr() + 4 * col0 * m), m)
        else:
            gpu.gemm(dptr(A), pb, pc, m, cols, k, ta, tb, lda, ldb, m, 1.0, beta)

    run(whole, aux_w, 0, n)
    step = 128 * (768 // (m // 128) // 2)          # at most half the tiles that would be walked
    for col0 in range(0, n, step):
        run(pieces, aux_p, col0, min(step, n - col0))
    torch.cuda.synchronize()
    assert torch.equal(whole, pieces)
    assert torch.equal(aux_w, aux_p)
    # and against float64 on the device
    Am = A.double().view(-1, lda).T
    Bm = B.double().view(-1, ldb).T
    v = (Am.T if ta else Am) @ (Bm.T if tb else Bm)            # m x n
    if fused:
        v = v + bias.double()[:, None]
        assert rel_err(to_host(aux_w), to_host(v.T.reshape(-1))) <= TOL_GEMM
        v = 0.5 * v * (1 + torch.erf(v / math.sqrt(2))) + res.double().view(n, m).T
    else:
        v = v + beta * old.double().view(n, m).T
    assert rel_err(to_host(whole), to_host(v.T.reshape(-1))) <= TOL_GEMM


# The fused store with the row sums of what it stores (upstream gradient times activation derivative and
# the bias gradient of the layer below): tiled forms of several tile shapes, ragged edges on the checked
# loaders, and the forms without a fused store (split-K, thin, matrix-vector), which run the sum kernel.
@pytest.mark.parametrize("m,n,k,ta", [(256, 512, 128, 1), (2048, 1024, 512, 1), (128, 1024, 96, 0), (129, 127, 17, 1),
                                      (64, 1216, 512, 1), (32, 512, 64, 0), (512, 64, 128, 1), (1024, 32, 64, 0),
                                      (10, 128, 2560, 1), (5, 300, 64, 0), (300, 1, 70, 0), (256, 128, 4096, 1)])
@pytest.mark.parametrize("act", [0, 3, 4])
def test_gemm_fused_rowsum(gpu, m, n, k, ta, act):
    r = rng(m + 3 * n + 5 * k + act)
    lda = k if ta else m
    A = r.normal(0, 1 / math.sqrt(k), m * k).astype(np.float32)
    B = r.normal(0, 1, k * n).astype(np.float32)
    pre = r.normal(0.2, 1, m * n).astype(np.float32)
    bias = r.normal(0.1, 0.5, m).astype(np.float32)
    dA, dB, dpre, dbias = to_dev(A), to_dev(B), to_dev(pre), to_dev(bias)
    want = to_dev(np.full(m * n, np.nan, np.float32))
    got = to_dev(np.full(m * n, np.nan, np.float32))
    rs = to_dev(np.full(m, np.nan, np.float32))
    aux = dptr(dpre) if act else None
    pb = dptr(dbias) if act == 0 else None
    gpu.gemm_fused(dptr(dA), dptr(dB), dptr(want), m, n, k, ta, 0, lda, k, m, 1.0, 0.0, pb, act, aux, m, None, m)
    gpu.gemm_fused_rowsum(dptr(dA), dptr(dB), dptr(got), dptr(rs), m, n, k, ta, 0, lda, k, m, 1.0, 0.0, pb, act, aux, m,
                          None, m)
    out = to_host(got)
    assert np.array_equal(out, to_host(want))
    O = out.reshape(n, m).astype(np.float64)
    assert np.linalg.norm(to_host(rs) - O.sum(0)) <= 1e-5 * np.linalg.norm(np.abs(O).sum(0))


def test_gemm_fused_rowsum_at_the_feed_forward_gradient_shape(gpu):
    """(W2^T dy) .* gelu'(F1) at 2048 x 16384 x 512 with the row sums: against the plain fused entry
    point bit for bit and jzhip_sum_rows over its result; twice (the partial sums live in the workspace)."""
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(11)
    d, ff, N = 512, 2048, 16384
    for _ in range(2):
        W2 = torch.randn(d * ff, generator=g, device="cuda") / math.sqrt(ff)
        dy = torch.randn(d * N, generator=g, device="cuda")
        F1 = torch.randn(ff * N, generator=g, device="cuda")
        a, b = torch.full((ff * N,), float("nan"), device="cuda"), torch.empty(ff * N, device="cuda")
        rs, rs2 = torch.full((ff,), float("nan"), device="cuda"), torch.empty(ff, device="cuda")
        gpu.gemm_fused_rowsum(dptr(W2), dptr(dy), dptr(a), dptr(rs), ff, N, d, 1, 0, d, d, ff, 1.0, 0.0, None, 4, dptr(F1), ff,
                              None, ff)
        gpu.gemm_fused(dptr(W2), dptr(dy), dptr(b), ff, N, d, 1, 0, d, d, ff, 1.0, 0.0, None, 4, dptr(F1), ff, None, ff)
        gpu.sum_rows(dptr(rs2), dptr(b), ff, N, ff)
        gpu.synchronize()
        assert torch.equal(a, b)
        want = b.view(N, ff).double().sum(dim=0)
        assert float((rs.double() - want).norm() / want.norm()) <= 1e-5
        assert float((rs - rs2).norm() / rs2.norm()) <= 1e-5


def test_gemm_fused_rejects_bad_arguments(gpu):
    from juzhen_amd import capi
    lib = capi.load()
    d = dev_empty(16)
    assert lib.jzhip_gemm_fused(dptr(d), dptr(d), dptr(d), 2, 2, 2, 0, 0, 2, 2, 2, 1.0, 0.0, None, 7, None, 2, None, 2) == -1
    assert lib.jzhip_gemm_fused(dptr(d), dptr(d), dptr(d), 2, 2, 2, 0, 0, 2, 2, 2, 1.0, 0.0, None, 3, None, 2, None, 2) == -1
    assert lib.jzhip_gemm_fused(dptr(d), dptr(d), dptr(d), 2, 2, 2, 0, 0, 2, 2, 2, 1.0, 0.0, None, 0, None, 2, dptr(d), 1) == -1


def test_gemm_known_answer(gpu):
    """tests/testRocmDeviceProof.cu:36-41: [[1,2],[3,4]]*[[5,6],[7,8]] = [[19,22],[43,50]]."""
    A = np.array([1, 3, 2, 4], np.float32)  # column-major
    B = np.array([5, 7, 6, 8], np.float32)
    dC = dev_empty(4)
    gpu.gemm_nn(dp(A), dp(B), dptr(dC), 2, 2, 2, 1.0, 0.0)
    assert np.array_equal(to_host(dC), np.array([19, 43, 22, 50], np.float32))


def test_gemm_rejects_bad_arguments(gpu):
    from juzhen_amd import capi
    lib = capi.load()
    d = dev_empty(16)
    assert lib.jzhip_gemm(dptr(d), dptr(d), dptr(d), 0, 2, 2, 0, 0, 2, 2, 2, 1.0, 0.0) == -1
    assert lib.jzhip_gemm(None, dptr(d), dptr(d), 2, 2, 2, 0, 0, 2, 2, 2, 1.0, 0.0) == -1
    assert lib.jzhip_gemv(dptr(d), dptr(d), dptr(d), 2, 2, 0, 2, 0, 1, 1.0, 0.0) == -1


@pytest.mark.parametrize("m,n,trans", [(1, 1, 0), (5, 3, 0), (5, 3, 1), (1000, 37, 0), (1000, 37, 1), (64, 5000, 0),
                                       (64, 5000, 1)])
def test_gemv(gpu, oracle_lib, m, n, trans):
    r = rng(m + n)
    lda = m + 2
    A = r.normal(0, 1, lda * n).astype(np.float32)
    lx, ly = (m, n) if trans else (n, m)
    x = r.normal(0, 1, lx).astype(np.float32)
    y0 = r.normal(0, 1, ly).astype(np.float32)
    ref = y0.copy()
    oracle_lib.jzo_gemv(trans, m, n, 0.5, hptr(A), lda, hptr(x), 1, 2.0, hptr(ref), 1)
    dy = to_dev(y0)
    gpu.gemv(dp(A), dp(x), dptr(dy), m, n, trans, lda, 1, 1, 0.5, 2.0)
    assert rel_err(to_host(dy), ref) <= TOL_GEMM


@pytest.mark.parametrize("m,n,trans,incx,incy", [
    (2048, 300, 1, 1, 1),      # long columns, A^T x: four columns per workgroup, rows split over its waves
    (2052, 7, 1, 1, 3),        # the same with a ragged last float4 step and a strided y
    (4096, 512, 0, 1, 1),      # A x through the thin-product kernel with one vector
    (4096, 512, 0, 2, 2),      # strided x and y on that path
    (256, 4096, 1, 1, 1),      # short columns, A^T x: the thin dot form, four columns per wavefront
    (512, 1030, 1, 3, 1),      # strided x on the dot form
    (1024, 1, 1, 1, 1), (1, 1024, 0, 1, 1),
])
def test_gemv_float4_forms(gpu, oracle_lib, m, n, trans, incx, incy):
    """Shapes with lda % 4 == 0 and aligned operands, which take the vector kernels (the
    cases of test_gemv have lda = m + 2 and stay on the scalar ones)."""
    r = rng(m + 3 * n + trans)
    lda = m
    A = r.normal(0, 1, lda * n).astype(np.float32)
    lx, ly = (m, n) if trans else (n, m)
    x = r.normal(0, 1, lx * incx).astype(np.float32)
    y0 = r.normal(0, 1, ly * incy).astype(np.float32)
    for alpha, beta in ((0.5, 2.0), (1.0, 0.0)):
        ref = y0.copy()
        oracle_lib.jzo_gemv(trans, m, n, alpha, hptr(A), lda, hptr(x), incx, beta, hptr(ref), incy)
        dy = to_dev(y0)
        gpu.gemv(dp(A), dp(x), dptr(dy), m, n, trans, lda, incx, incy, alpha, beta)
        got = to_host(dy)
        assert rel_err(got, ref) <= TOL_GEMM
        if incy > 1:   # the gaps of a strided y are untouched
            mask = np.ones(ly * incy, bool)
            mask[::incy] = False
            assert np.array_equal(got[mask], y0[mask])


@pytest.mark.parametrize("ta,tb", [(1, 0), (0, 1), (0, 0)])
def test_gemm_strided_batched(gpu, oracle_lib, ta, tb):
    """Attention-shaped batches: per (head, sequence) S x S scores from d_h x S slices."""
    r = rng(9)
    S, dh, dk, batch = 48, 16, 64, 5
    Q = r.normal(0, 1, dk * S * batch).astype(np.float32)
    K = r.normal(0, 1, dk * S * batch).astype(np.float32)
    if (ta, tb) == (1, 0):      # scores = Qi^T Ki
        m, n, k, lda, ldb, sa, sb = S, S, dh, dk, dk, dk * S, dk * S
    elif (ta, tb) == (0, 1):    # Hi = Vi * Ai^T with Ai (S x S): here B = K viewed (S x dh)
        m, n, k, lda, ldb, sa, sb = dh, dh, S, dk, dk, dk * S, dk * S
        tb = 1
    else:
        m, n, k, lda, ldb, sa, sb = dh, S, dh, dk, dk, dk * S, dk * S
    ldc = m
    out = np.zeros(m * n * batch, np.float32)
    for b in range(batch):
        Cb = np.zeros(m * n, np.float32)
        oracle_lib.jzo_gemm(ta, tb, m, n, k, 1.0, hp(Q[b * sa:]), lda, hp(K[b * sb:]), ldb, 0.0, hptr(Cb), ldc)
        out[b * m * n:(b + 1) * m * n] = Cb
    dC = dev_empty(m * n * batch)
    gpu.gemm_strided_batched(dp(Q), dp(K), dptr(dC), m, n, k, ta, tb, lda, ldb, ldc,
                             sa, sb, m * n, batch, 1.0, 0.0)
    assert rel_err(to_host(dC), out) <= TOL_GEMM


@pytest.mark.parametrize("m,n,k,batch,beta", [(128, 96, 8192, 3, 0.0), (64, 64, 4096, 5, 0.5), (192, 128, 16384, 3, 0.0)])
def test_gemm_batched_problems_with_a_long_contraction(gpu, m, n, k, batch, beta):
    """A few batched problems whose outputs cannot fill the chip and whose contraction is long
    (the weight gradients of three projections sharing their input): K is split over workgroups
    for every problem, each with its own run of partial sums.  B is shared (stride 0), as there.
    Checked against float64 products; alpha and beta apply once, in the reduction."""
    r = rng(m + n + k)
    A = r.normal(0, 1, (batch, k, m)).astype(np.float32)      # column-major m x k per problem
    B = r.normal(0, 1, (k, n)).astype(np.float32)             # column-major n x k, used transposed
    C0 = r.normal(0, 1, (batch, n, m)).astype(np.float32)     # column-major m x n per problem
    dA, dB, dC = to_dev(A.reshape(-1)), to_dev(B.reshape(-1)), to_dev(C0.reshape(-1))
    gpu.gemm_strided_batched(dptr(dA), dptr(dB), dptr(dC), m, n, k, 0, 1, m, n, m, m * k, 0, m * n, batch, 0.75, beta)
    got = to_host(dC).reshape(batch, n, m)
    for b in range(batch):
        want = 0.75 * (B.astype(np.float64).T @ A[b].astype(np.float64)) + beta * C0[b]
        assert np.max(np.abs(got[b] - want)) <= TOL_GEMM * np.sqrt(k)


def test_add_bias(gpu):
    r = rng(3)
    for rows, cols in ((512, 100), (10, 33), (1, 7)):
        y = r.normal(0, 1, rows * cols).astype(np.float32)
        b = r.normal(0, 1, rows).astype(np.float32)
        dy = to_dev(y)
        gpu.add_bias(dptr(dy), dp(b), rows, cols)
        assert np.array_equal(to_host(dy), (y.reshape(cols, rows) + b[None, :]).reshape(-1))


@pytest.mark.parametrize("k,n", [(10, 128), (7, 33), (256, 16384), (4, 1), (1, 5)])
def test_one_hot(gpu, oracle_lib, k, n):
    r = rng(k * 31 + n)
    lab = r.integers(0, k, n).astype(np.int32)
    if n > 4:
        lab[1], lab[n - 2] = -1, k                      # outside the range: zero column
    dl = to_dev(lab)
    out = to_dev(np.full(k * n, 7.0, np.float32))
    gpu.one_hot(dptr(out), dptr(dl), k, n)
    ref = np.empty(k * n, np.float32)
    oracle_lib.jzo_one_hot(hptr(ref), hptr(lab), k, n)
    assert np.array_equal(to_host(out), ref)


# ── softmax family ───────────────────────────────────────────────────────
@pytest.mark.parametrize("rows,cols", [(1, 1), (10, 128), (64, 9), (100, 300), (256, 2048), (1024, 64), (3000, 5),
                                       # every kernel of the family: register, wide-block, chunked rows;
                                       # wave, block and three-sweep columns
                                       (1024, 1024), (520, 700), (2048, 1500), (64, 9000), (600, 2500),
                                       (4096, 33), (6000, 4), (16384, 7), (20000, 3), (1028, 40), (1030, 12)])
def test_softmax_cols_rows(gpu, oracle_lib, rows, cols):
    x = rng(rows + cols).normal(0, 3, rows * cols).astype(np.float32)
    dx = to_dev(x)
    out = dev_empty(rows * cols)
    ref = np.empty_like(x)
    oracle_lib.jzo_softmax_cols(hptr(ref), hptr(x), rows, cols, rows)
    gpu.softmax_cols(dptr(out), dptr(dx), rows, cols, rows)
    got = to_host(out)
    assert rel_err(got, ref) <= TOL_RED
    assert np.allclose(got.reshape(cols, rows).sum(axis=1), 1.0, atol=1e-5)
    oracle_lib.jzo_softmax_rows(hptr(ref), hptr(x), rows, cols, rows)
    gpu.softmax_rows(dptr(out), dptr(dx), rows, cols, rows)
    got = to_host(out)
    assert rel_err(got, ref) <= TOL_RED
    assert np.allclose(got.reshape(cols, rows).sum(axis=0), 1.0, atol=1e-5)


@pytest.mark.parametrize("rows,cols,pad", [
    # rows of at most 2048 columns are held in the registers of one workgroup; the split of the
    # workgroup depends on the column count, the height and whether float4 access applies
    # (rows and leading dimension multiples of 4): one case per branch, ragged edges included
    (16384, 200, 0), (260, 100, 0), (301, 250, 3), (16388, 256, 4),
    (4096, 400, 0), (4099, 300, 1), (300, 500, 0), (4100, 512, 8),
    (4096, 1000, 0), (4097, 1024, 0), (2049, 700, 2), (1024, 1024, 0), (257, 900, 0),
    (8192, 2048, 0), (2048, 1500, 4), (8193, 1100, 0), (1001, 2047, 0), (8200, 1025, 0)])
def test_softmax_rows_single_read_forms(gpu, oracle_lib, rows, cols, pad):
    ld = rows + pad
    x = rng(rows + 3 * cols + pad).normal(0, 3, ld * cols).astype(np.float32)
    ref = x.copy()                                   # the padding rows must come back untouched
    oracle_lib.jzo_softmax_rows(hptr(ref), hptr(x), rows, cols, ld)
    out = to_dev(x)
    gpu.softmax_rows(dptr(out), dptr(out), rows, cols, ld)   # in place, as row_softmax of a view does
    got = to_host(out).reshape(cols, ld)
    ref = ref.reshape(cols, ld)
    assert rel_err(got[:, :rows], ref[:, :rows]) <= TOL_RED
    assert np.array_equal(got[:, rows:], x.reshape(cols, ld)[:, rows:])
    assert np.allclose(got[:, :rows].sum(axis=0), 1.0, atol=1e-5)


@pytest.mark.parametrize("S,nblk", [(8, 3), (64, 4), (100, 2), (256, 6)])
@pytest.mark.parametrize("causal", [0, 1])
@pytest.mark.parametrize("kar", [0, 1])
def test_attn_softmax_fwd_bwd(gpu, oracle_lib, S, nblk, causal, kar):
    r = rng(S * 10 + nblk + causal)
    n = S * S * nblk
    x = r.normal(0, 4, n).astype(np.float32)
    scale = 1.0 / np.sqrt(np.float32(64))
    ref = np.empty_like(x)
    oracle_lib.jzo_attn_softmax(hptr(ref), hptr(x), S, nblk, scale, causal, kar)
    out = dev_empty(n)
    gpu.attn_softmax(dptr(out), dp(x), S, nblk, scale, causal, kar)
    got = to_host(out)
    assert rel_err(got, ref) <= TOL_RED
    if causal:
        blk = got.reshape(nblk, S, S)  # [b, col, row]
        qi, ki = (np.arange(S)[:, None], np.arange(S)[None, :]) if kar else (np.arange(S)[None, :], np.arange(S)[:, None])
        assert np.all(blk[:, ki > qi] == 0.0)
    dA = r.normal(0, 1, n).astype(np.float32)
    refd = np.empty_like(x)
    oracle_lib.jzo_attn_softmax_bwd(hptr(refd), hptr(ref), hptr(dA), S, nblk, scale, kar)
    dS = dev_empty(n)
    gpu.attn_softmax_bwd(dptr(dS), dp(ref), dp(dA), S, nblk, scale, kar)
    assert rel_err(to_host(dS), refd) <= TOL_RED


@pytest.mark.parametrize("K,N", [(10, 128), (256, 4096), (2, 1), (77, 300), (1024, 9), (2000, 17)])
def test_softmax_xent(gpu, oracle_lib, K, N):
    r = rng(K + N)
    x = r.normal(0, 2, K * N).astype(np.float32)
    lab = r.integers(0, K, N).astype(np.int32)
    refd = np.empty_like(x)
    ref_loss = oracle_lib.jzo_softmax_xent(hptr(refd), hptr(x), hptr(lab), K, N, K)
    dl = dev_empty(1)
    dd = dev_empty(K * N)
    gpu.softmax_xent(dptr(dl), dptr(dd), dp(x), dp(lab), K, N, K)
    assert abs(to_host(dl)[0] - ref_loss) <= TOL_RED * (abs(ref_loss) + np.abs(x).max())
    assert rel_err(to_host(dd), refd) <= TOL_RED
    # closed form in float64
    X = x.reshape(N, K).astype(np.float64)
    lse = np.log(np.exp(X - X.max(1, keepdims=True)).sum(1)) + X.max(1)
    exact = -(X[np.arange(N), lab] - lse).mean()
    # x[label] - lse cancels when the label dominates, so the bound is relative
    # to the magnitude of the terms that are subtracted
    assert abs(to_host(dl)[0] - exact) <= TOL_RED * (abs(exact) + np.abs(lse).mean())


@pytest.mark.parametrize("K,N,nb", [(10, 128, 128), (1, 5, 5), (256, 1000, 1000), (1000, 33, 33), (1500, 40, 8), (65, 7, 7)])
def test_softmax_xent_dense_targets(gpu, oracle_lib, K, N, nb):
    """The head against a matrix of targets (ml/layer.hpp:252-283): with one-hot targets it agrees
    with the label form (checked against the oracle's), with soft targets with the closed form in
    float64; more than 1024 classes take the swept kernel; nb need not equal N."""
    r = rng(K * 3 + N)
    x = r.normal(0, 2, K * N).astype(np.float32)
    lab = r.integers(0, K, N).astype(np.int32)
    onehot = np.zeros((N, K), np.float32)
    onehot[np.arange(N), lab] = 1.0
    refd = np.empty_like(x)
    ref_loss = oracle_lib.jzo_softmax_xent(hptr(refd), hptr(x), hptr(lab), K, N, K)   # scaled by 1/N
    dl, dd = dev_empty(1), dev_empty(K * N)
    gpu.softmax_xent_dense(dptr(dl), dptr(dd), dp(x), dp(onehot.reshape(-1)), K, N, K, 1.0 / nb)
    assert abs(to_host(dl)[0] * nb / N - ref_loss) <= TOL_RED * (abs(ref_loss) + np.abs(x).max())
    assert rel_err(to_host(dd) * np.float32(nb / N), refd) <= TOL_RED
    # soft targets: closed form
    Y = r.random((N, K)); Y /= Y.sum(1, keepdims=True)
    y32 = Y.astype(np.float32)
    X = x.reshape(N, K).astype(np.float64)
    mx = X.max(1, keepdims=True)
    E = np.exp(X - mx)
    lse = np.log(E.sum(1)) + mx[:, 0]
    exact = -((X * y32).sum(1) - lse).sum() / nb
    grad = -(y32 - E / E.sum(1, keepdims=True)) / nb
    gpu.softmax_xent_dense(dptr(dl), dptr(dd), dp(x), dp(y32.reshape(-1)), K, N, K, 1.0 / nb)
    assert abs(to_host(dl)[0] - exact) <= TOL_RED * (abs(exact) + np.abs(lse).mean() * N / nb)
    assert rel_err(to_host(dd), grad.reshape(-1)) <= TOL_RED
    # either output alone
    only = dev_empty(K * N)
    gpu.softmax_xent_dense(None, dptr(only), dp(x), dp(y32.reshape(-1)), K, N, K, 1.0 / nb)
    assert np.array_equal(to_host(only), to_host(dd))


# ── LayerNorm ────────────────────────────────────────────────────────────
@pytest.mark.parametrize("dim,N", [(4, 3), (256, 512), (512, 1024), (1024, 33), (100, 77), (1030, 9), (513, 5)])
def test_layernorm(gpu, oracle_lib, dim, N):
    r = rng(dim + N)
    x = r.normal(0.3, 2, dim * N).astype(np.float32)
    gamma = r.normal(1, 0.2, dim).astype(np.float32)
    beta = r.normal(0, 0.2, dim).astype(np.float32)
    y, xh, inv = (np.empty(dim * N, np.float32), np.empty(dim * N, np.float32), np.empty(N, np.float32))
    oracle_lib.jzo_layernorm_fwd(hptr(y), hptr(xh), hptr(inv), hptr(x), hptr(gamma), hptr(beta), dim, N)
    dy_, dxh, dinv = dev_empty(dim * N), dev_empty(dim * N), dev_empty(N)
    dg, db = to_dev(gamma), to_dev(beta)
    gpu.layernorm_fwd(dptr(dy_), dptr(dxh), dptr(dinv), dp(x), dptr(dg), dptr(db), dim, N)
    assert rel_err(to_host(dy_), y) <= TOL_RED
    assert rel_err(to_host(dxh), xh) <= TOL_RED
    assert rel_err(to_host(dinv), inv) <= TOL_RED
    # float64 closed form
    X = x.reshape(N, dim).astype(np.float64)
    mu = X.mean(1, keepdims=True)
    var = ((X - mu) ** 2).mean(1, keepdims=True)
    exact = (X - mu) / np.sqrt(var + 1e-5) * gamma + beta
    assert rel_err(to_host(dy_), exact.reshape(-1)) <= TOL_RED

    g = r.normal(0, 1, dim * N).astype(np.float32)
    dx = np.empty(dim * N, np.float32)
    oracle_lib.jzo_layernorm_bwd(hptr(dx), hptr(g), hptr(gamma), hptr(xh), hptr(inv), dim, N)
    ddx = dev_empty(dim * N)
    gpu.layernorm_bwd(dptr(ddx), dp(g), dptr(dg), dp(xh), dp(inv), dim, N)
    assert rel_err(to_host(ddx), dx) <= TOL_RED
    # the fused skip-gradient add equals the separate add bit for bit
    res = r.normal(0, 1, dim * N).astype(np.float32)
    dres = to_dev(res)
    dfused = dev_empty(dim * N)
    gpu.layernorm_bwd_residual(dptr(dfused), dp(g), dptr(dg), dp(xh), dp(inv), dptr(dres), dim, N)
    gpu.axpby(dptr(ddx), dptr(ddx), dptr(dres), dim * N, 1.0, 1.0)
    assert np.array_equal(to_host(dfused), to_host(ddx))
    assert rel_err(to_host(dfused), dx.astype(np.float64) + res) <= TOL_RED

    # tangent through the same point (LayerNorm::jvp)
    jv = np.empty(dim * N, np.float32)
    oracle_lib.jzo_layernorm_jvp(hptr(jv), hptr(g), hptr(gamma), hptr(xh), hptr(inv), dim, N)
    djv = dev_empty(dim * N)
    gpu.layernorm_jvp(dptr(djv), dp(g), dptr(dg), dp(xh), dp(inv), dim, N)
    assert rel_err(to_host(djv), jv) <= TOL_RED

    rg, rb = np.empty(dim, np.float32), np.empty(dim, np.float32)
    oracle_lib.jzo_layernorm_param_grads(hptr(rg), hptr(rb), hptr(g), hptr(xh), dim, N)
    og, ob = dev_empty(dim), dev_empty(dim)
    gpu.layernorm_param_grads(dptr(og), dptr(ob), dp(g), dp(xh), dim, N)
    G = g.reshape(N, dim).astype(np.float64)
    XH = xh.reshape(N, dim).astype(np.float64)
    sg = np.linalg.norm(np.abs(G * XH).sum(0))
    sb = np.linalg.norm(np.abs(G).sum(0))
    assert np.linalg.norm(to_host(og) - (G * XH).sum(0)) <= TOL_RED * sg
    assert np.linalg.norm(to_host(ob) - G.sum(0)) <= TOL_RED * sb
    assert np.linalg.norm(to_host(og) - rg) <= TOL_RED * sg


# The backward sweep with the sums over tokens on the side (ml/layer.hpp:2674-2686 and the `sum(t, 1)`
# bias gradients of the dense layers around the residual add, :100).  (512, 16384) is the transformer
# configuration's shape; (300, 5000) leaves lanes without rows and waves with ragged runs of columns;
# the last four take the separate passes (dim > 512, few columns, dim not a multiple of 4).
@pytest.mark.parametrize("dim,N", [(512, 16384), (256, 2048), (512, 1027), (300, 5000), (64, 4096),
                                   (1024, 2048), (512, 100), (7, 3000), (513, 1500)])
@pytest.mark.parametrize("mode", ["res+sums", "res", "plain", "in place"])
def test_layernorm_backward_with_sums(gpu, oracle_lib, dim, N, mode):
    r = rng(dim * 3 + N)
    x = r.normal(0.3, 2, dim * N).astype(np.float32)
    gamma = r.normal(1, 0.2, dim).astype(np.float32)
    beta = r.normal(0, 0.2, dim).astype(np.float32)
    y, xh, inv = (np.empty(dim * N, np.float32), np.empty(dim * N, np.float32), np.empty(N, np.float32))
    oracle_lib.jzo_layernorm_fwd(hptr(y), hptr(xh), hptr(inv), hptr(x), hptr(gamma), hptr(beta), dim, N)
    g = r.normal(0.05, 1, dim * N).astype(np.float32)
    res = r.normal(0.02, 1, dim * N).astype(np.float32)
    with_res = mode != "plain"
    dg, dxh, dinv, dgam = to_dev(g), to_dev(xh), to_dev(inv), to_dev(gamma)
    dres = to_dev(res) if with_res else None
    pres = dptr(dres) if with_res else None
    # the separate entry points
    want_dx = dev_empty(dim * N)
    gpu.layernorm_bwd_residual(dptr(want_dx), dptr(dg), dptr(dgam), dptr(dxh), dptr(dinv), pres, dim, N)
    wg, wb = dev_empty(dim), dev_empty(dim)
    gpu.layernorm_param_grads(dptr(wg), dptr(wb), dptr(dg), dptr(dxh), dim, N)
    nan = lambda n: to_dev(np.full(n, np.nan, np.float32))
    og, ob, osx, osr = nan(dim), nan(dim), nan(dim), nan(dim)
    out = dres if mode == "in place" else nan(dim * N)
    gpu.layernorm_bwd_residual_sums(dptr(out), dptr(dg), dptr(dgam), dptr(dxh), dptr(dinv), pres, dptr(og), dptr(ob),
                                    dptr(osx) if mode != "res" else None,
                                    dptr(osr) if mode in ("res+sums", "in place") else None, dim, N)
    got = to_host(out)
    assert np.array_equal(got, to_host(want_dx))
    G = g.reshape(N, dim).astype(np.float64)
    XH = xh.reshape(N, dim).astype(np.float64)
    sg = np.linalg.norm(np.abs(G * XH).sum(0))
    sb = np.linalg.norm(np.abs(G).sum(0))
    assert np.linalg.norm(to_host(og) - (G * XH).sum(0)) <= TOL_RED * sg
    assert np.linalg.norm(to_host(ob) - G.sum(0)) <= TOL_RED * sb
    assert np.linalg.norm(to_host(og) - to_host(wg)) <= 1e-5 * sg
    assert np.linalg.norm(to_host(ob) - to_host(wb)) <= 1e-5 * sb
    if mode != "res":
        D = got.reshape(N, dim).astype(np.float64)
        assert np.linalg.norm(to_host(osx) - D.sum(0)) <= 1e-5 * np.linalg.norm(np.abs(D).sum(0))
    if mode in ("res+sums", "in place"):
        R = res.reshape(N, dim).astype(np.float64)
        assert np.linalg.norm(to_host(osr) - R.sum(0)) <= 1e-5 * np.linalg.norm(np.abs(R).sum(0))
    else:
        assert np.isnan(to_host(osr)).all()          # not asked for: not written


def test_layernorm_backward_with_sums_rejects_bad_arguments(gpu):
    from juzhen_amd import capi
    lib = capi.load()
    d = dev_empty(64)
    P = dptr(d)
    assert lib.jzhip_layernorm_bwd_residual_sums(P, P, P, P, P, None, P, P, None, P, 4, 4) == -1   # sum_res without res
    assert lib.jzhip_layernorm_bwd_residual_sums(P, P, P, P, P, None, None, P, None, None, 4, 4) == -1
    assert lib.jzhip_layernorm_bwd_residual_sums(P, P, P, P, P, None, P, P, None, None, 0, 4) == -1


# ── Adam ─────────────────────────────────────────────────────────────────
@pytest.mark.parametrize("n", [1, 5, 4096, 1 << 20])
def test_adam_bit_exact(gpu, oracle_lib, n):
    r = rng(n)
    g0 = r.normal(0, 1, n).astype(np.float32)
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    dm, dv = to_dev(m), to_dev(v)
    for it in range(1, 6):
        g = (g0 * np.float32(1.0 / it)).astype(np.float32)
        dg = to_dev(g)
        oracle_lib.jzo_adam_update(hptr(g), hptr(m), hptr(v), n, 1e-3, 0.9, 0.999, 1e-8, it)
        gpu.adam_update(dptr(dg), dptr(dm), dptr(dv), n, 1e-3, 0.9, 0.999, 1e-8, it)
        assert np.array_equal(to_host(dg), g)
        assert np.array_equal(to_host(dm), m)
        assert np.array_equal(to_host(dv), v)
    # step 1 closed form: update = alpha * g/(|g| + eps*...) ~ alpha*sign(g)
    g = g0.copy()
    m[:] = 0
    v[:] = 0
    oracle_lib.jzo_adam_update(hptr(g), hptr(m), hptr(v), n, 1e-3, 0.9, 0.999, 1e-8, 1)
    big = np.abs(g0) > 1e-3
    assert np.allclose(g[big], 1e-3 * np.sign(g0[big]), rtol=1e-4)


@pytest.mark.parametrize("wd", [0.0, 0.01])
def test_adamw_step(gpu, oracle_lib, wd):
    n = 10007
    r = rng(11)
    w = r.normal(0, 1, n).astype(np.float32)
    g = r.normal(0, 1, n).astype(np.float32)
    m = r.normal(0, 0.1, n).astype(np.float32)
    v = r.uniform(0, 0.1, n).astype(np.float32)
    dw, dg, dm, dv = to_dev(w), to_dev(g), to_dev(m), to_dev(v)
    oracle_lib.jzo_adamw_step(hptr(w), hptr(g), hptr(m), hptr(v), n, 3e-4, 0.9, 0.999, 1e-8, wd, 7)
    gpu.adamw_step(dptr(dw), dptr(dg), dptr(dm), dptr(dv), n, 3e-4, 0.9, 0.999, 1e-8, wd, 7)
    assert np.array_equal(to_host(dw), w)
    assert np.array_equal(to_host(dm), m)
    assert np.array_equal(to_host(dv), v)
    assert np.array_equal(to_host(dg), g)


def test_adamw_step_multi_equals_single_tensor_steps(gpu):
    """Seven tensors of awkward sizes (one unaligned, one empty, different
    hyper-parameters and step counters) in one launch against jzhip_adamw_step per
    tensor: parameters and both moments bit for bit, over three steps."""
    from juzhen_amd.capi import AdamTensor
    r = rng(31)
    sizes = [1, 5, 1024, 4099, 0, 256 * 256, 70001]
    hyper = [(1e-3, 0.9, 0.999, 1e-8, 0.0, 1), (3e-4, 0.8, 0.99, 1e-6, 0.01, 4), (1e-2, 0.9, 0.999, 1e-8, 0.0, 2),
             (1e-3, 0.9, 0.999, 1e-8, 0.1, 1), (1e-3, 0.9, 0.999, 1e-8, 0.0, 1), (2e-4, 0.95, 0.999, 1e-8, 0.0, 7),
             (1e-3, 0.9, 0.98, 1e-7, 0.02, 3)]
    import torch
    def fresh():
        rr = rng(5)
        out = []
        for n in sizes:
            pad = 1 if n == 4099 else 0          # a view that is not 16-byte aligned
            w = to_dev(rr.normal(0, 1, n + pad).astype(np.float32))
            m = to_dev(rr.normal(0, 0.1, n + pad).astype(np.float32))
            v = to_dev(rr.uniform(0, 0.1, n + pad).astype(np.float32))
            out.append((w, m, v, pad))
        return out
    A, B = fresh(), fresh()
    for step in range(3):
        grads = [to_dev(r.normal(0, 1, n + (1 if n == 4099 else 0)).astype(np.float32)) for n in sizes]
        arr = (AdamTensor * len(sizes))()
        for i, n in enumerate(sizes):
            w, m, v, pad = A[i]
            al, b1, b2, eps, wd, it = hyper[i]
            o = 4 * pad
            gpu.adamw_step(C.c_void_p(w.data_ptr() + o), C.c_void_p(grads[i].data_ptr() + o),
                           C.c_void_p(m.data_ptr() + o), C.c_void_p(v.data_ptr() + o), n, al, b1, b2, eps, wd, it + step)
            w2, m2, v2, _ = B[i]
            arr[i] = AdamTensor(w2.data_ptr() + o, grads[i].data_ptr() + o, m2.data_ptr() + o, v2.data_ptr() + o, n,
                                al, b1, b2, eps, wd, it + step)
        gpu.adamw_step_multi(arr, len(sizes))
        gpu.synchronize()
        for i in range(len(sizes)):
            for a, b in zip(A[i][:3], B[i][:3]):
                assert torch.equal(a, b), (step, i)
    from juzhen_amd import capi
    lib = capi.load()
    assert lib.jzhip_adamw_step_multi(None, 0) == 0
    assert lib.jzhip_adamw_step_multi(None, 2) == -1


# ── convolution data movement (bit-exact) ────────────────────────────────
CONV_CASES = [
    # N, C, H, W, kH, kW, pad, stride
    (2, 1, 5, 5, 3, 3, 1, 1),
    (3, 2, 7, 6, 3, 3, 0, 1),
    (2, 3, 8, 8, 3, 3, 1, 2),
    (2, 4, 9, 7, 2, 2, 0, 2),
    (1, 2, 6, 6, 5, 5, 2, 1),
    (4, 1, 28, 28, 3, 3, 1, 1),
    (2, 32, 28, 28, 3, 3, 1, 2),
    (2, 3, 10, 10, 4, 4, 1, 2),
    (2, 5, 7, 9, 3, 2, 1, 3),
    # layer-sized: the row-tiled kernels (K % 4 == 0, K >= 64), chunk edges inside a channel
    (2, 64, 32, 32, 3, 3, 1, 1),
    (3, 128, 16, 16, 3, 3, 1, 2),
    (2, 36, 13, 11, 3, 3, 1, 1),
    (2, 20, 9, 10, 5, 5, 2, 2),
    (1, 16, 8, 8, 2, 2, 0, 1),
    (2, 256, 8, 8, 3, 3, 1, 1),
    (2, 8, 9, 7, 3, 3, 0, 1),
    (2, 4, 6, 6, 3, 3, 2, 1),
    (2, 8, 12, 12, 5, 5, 2, 1),
    (2, 4, 10, 10, 4, 4, 0, 2),
    (2, 8, 11, 11, 3, 3, 0, 2),
    (1, 16, 37, 20, 3, 3, 1, 1),
    # 64 MB of patches and more, where the scatter walks down the patch rows with a ring in LDS:
    # no padding, more padding than the kernel needs, 5x5, 4x4 stride 2, whole images per
    # workgroup (many samples) and ragged row segments (few samples of tall images)
    (7000, 8, 9, 7, 3, 3, 0, 1),
    (7400, 4, 6, 6, 3, 3, 2, 1),
    (600, 8, 12, 12, 5, 5, 2, 1),
    (16500, 4, 10, 10, 4, 4, 0, 2),
    (9400, 8, 11, 11, 3, 3, 0, 2),
    (160, 16, 37, 20, 3, 3, 1, 1),
    (5, 64, 151, 48, 3, 3, 1, 1),
    (18, 64, 101, 64, 3, 3, 1, 2),
    (32, 64, 32, 32, 3, 3, 1, 1),
]


def conv_dims(H, W, kH, kW, pad, stride):
    return (H + 2 * pad - kH) // stride + 1, (W + 2 * pad - kW) // stride + 1


@pytest.mark.parametrize("case", CONV_CASES)
def test_im2col_col2im(gpu, oracle_lib, case):
    N, Cc, H, W, kH, kW, pad, stride = case
    Ho, Wo = conv_dims(H, W, kH, kW, pad, stride)
    K, P = Cc * kH * kW, Ho * Wo
    r = rng(sum(case))
    x = r.normal(0, 1, Cc * H * W * N).astype(np.float32)
    col = np.empty(K * P * N, np.float32)
    args = (Cc, H, W, kH, kW, pad, pad, stride, stride, Ho, Wo, N)
    oracle_lib.jzo_im2col(hptr(x), hptr(col), *args)
    dcol = dev_empty(K * P * N)
    gpu.im2col(dp(x), dptr(dcol), *args)
    assert np.array_equal(to_host(dcol), col)

    c2 = r.normal(0, 1, K * P * N).astype(np.float32)
    dx = np.empty(Cc * H * W * N, np.float32)
    oracle_lib.jzo_col2im(hptr(c2), hptr(dx), *args)
    ddx = dev_empty(Cc * H * W * N)
    gpu.col2im(dp(c2), dptr(ddx), *args)
    assert np.array_equal(to_host(ddx), dx)
    # adjoint identity <im2col(x), c> == <x, col2im(c)>
    lhs = np.dot(col.astype(np.float64), c2.astype(np.float64))
    rhs = np.dot(x.astype(np.float64), dx.astype(np.float64))
    assert abs(lhs - rhs) <= 1e-4 * max(1.0, abs(lhs))


@pytest.mark.parametrize("C_out,P,N", [(1, 1, 1), (32, 784, 4), (3, 50, 7), (64, 196, 2), (33, 65, 3)])
def test_conv_reshapes(gpu, oracle_lib, C_out, P, N):
    r = rng(C_out + P + N)
    n = C_out * P * N
    y2d = r.normal(0, 1, n).astype(np.float32)
    bias = r.normal(0, 1, C_out).astype(np.float32)
    ref = np.empty(n, np.float32)
    oracle_lib.jzo_conv_forward_reshape_bias(hptr(y2d), hptr(ref), hptr(bias), C_out, P, N)
    out = dev_empty(n)
    gpu.conv_forward_reshape_bias(dp(y2d), dptr(out), dp(bias), C_out, P, N)
    assert np.array_equal(to_host(out), ref)
    back = np.empty(n, np.float32)
    oracle_lib.jzo_conv_backward_reshape(hptr(ref), hptr(back), C_out, P, N)
    dback = dev_empty(n)
    gpu.conv_backward_reshape(dptr(out), dptr(dback), C_out, P, N)
    assert np.array_equal(to_host(dback), back)
    for direction in (0, 1):
        oracle_lib.jzo_convtrans_reshape(hptr(y2d), hptr(ref), C_out, P, N, direction)
        gpu.convtrans_reshape(dp(y2d), dptr(out), C_out, P, N, direction)
        assert np.array_equal(to_host(out), ref)


CT_CASES = [
    # N, C_out, H_in, W_in, kH, kW, pad, stride
    (2, 3, 4, 4, 4, 4, 1, 2),
    (1, 2, 5, 3, 3, 3, 0, 1),
    (2, 4, 8, 8, 4, 4, 1, 2),
    (3, 1, 3, 5, 2, 2, 0, 2),
    (2, 2, 4, 4, 3, 3, 1, 3),
    (2, 64, 16, 16, 4, 4, 1, 2),
    (2, 128, 8, 8, 4, 4, 1, 2),
    (3, 12, 7, 5, 3, 3, 1, 2),
    # 64 MB of patches and more (the streamed scatter): whole images and row segments
    (64, 64, 16, 16, 4, 4, 1, 2),
    (26, 32, 40, 32, 4, 4, 1, 2),
]


@pytest.mark.parametrize("case", CT_CASES)
def test_convtrans_scatter_gather(gpu, oracle_lib, case):
    N, Co, Hi, Wi, kH, kW, pad, stride = case
    Ho = (Hi - 1) * stride - 2 * pad + kH
    Wo = (Wi - 1) * stride - 2 * pad + kW
    R, Pin = Co * kH * kW, Hi * Wi
    r = rng(sum(case))
    patches = r.normal(0, 1, R * Pin * N).astype(np.float32)
    bias = r.normal(0, 1, Co).astype(np.float32)
    args = (Co, Ho, Wo, Hi, Wi, kH, kW, pad, pad, stride, stride, N)
    ref = np.empty(Co * Ho * Wo * N, np.float32)
    oracle_lib.jzo_convtrans_scatter(hptr(patches), hptr(ref), hptr(bias), *args)
    out = dev_empty(ref.size)
    gpu.convtrans_scatter(dp(patches), dptr(out), dp(bias), *args)
    assert np.array_equal(to_host(out), ref)
    t = r.normal(0, 1, ref.size).astype(np.float32)
    tp = np.empty(R * Pin * N, np.float32)
    oracle_lib.jzo_convtrans_gather(hptr(t), hptr(tp), *args)
    dtp = dev_empty(tp.size)
    gpu.convtrans_gather(dp(t), dptr(dtp), *args)
    assert np.array_equal(to_host(dtp), tp)


# ── random numbers: range / moments only (tests/testRocmCpuParity.cu:214-224) ──
def test_rand(gpu):
    n = 1 << 20
    d = dev_empty(n)
    gpu.rand_uniform(dptr(d), n, 123)
    u = to_host(d)
    assert np.all(np.isfinite(u)) and u.min() >= 0.0 and u.max() < 1.0
    assert abs(u.mean() - 0.5) < 5e-3 and abs(u.var() - 1 / 12) < 5e-3
    gpu.rand_normal(dptr(d), n, 1.0, 2.0, 0)
    z = to_host(d)
    assert np.all(np.isfinite(z))
    assert abs(z.mean() - 1.0) < 2e-2 and abs(z.std() - 2.0) < 2e-2
    # seed != 0 restarts the stream, seed == 0 continues it
    gpu.rand_uniform(dptr(d), 1000, 123)
    assert np.array_equal(to_host(d)[:1000], u[:1000])
    gpu.rand_uniform(dptr(d), 1000, 0)
    assert not np.array_equal(to_host(d)[:1000], u[:1000])


# ── batched attention core ───────────────────────────────────────────────
@pytest.mark.parametrize("d_k,heads,S,B,causal", [(8, 4, 3, 2, 1), (16, 2, 5, 3, 0), (64, 1, 17, 2, 1), (128, 2, 64, 3, 1),
                                                  (512, 8, 32, 2, 1), (512, 8, 256, 2, 1), (256, 4, 128, 1, 0),
                                                  (64, 2, 96, 2, 1), (128, 2, 160, 1, 1), (128, 4, 224, 1, 0)])
def test_attention_fwd_bwd(gpu, d_k, heads, S, B, causal):
    """Against a float64 restatement of the per-(head, sequence) loop of
    ml/layer.hpp:2967-3006 and 3329-3363 (the method of tests/testTransformerRef.cu:102-141)."""
    r = rng(d_k + S + B)
    N, dh = S * B, d_k // heads
    Q, K, V, dH = (r.normal(0, 1, (N, d_k)).astype(np.float32) for _ in range(4))   # [col, row]
    H = np.zeros((N, d_k)); A = np.zeros((heads * B, S, S))                           # A[blk][key][query]
    dQ, dK, dV = np.zeros((N, d_k)), np.zeros((N, d_k)), np.zeros((N, d_k))
    scale = 1.0 / np.sqrt(np.float32(dh))
    for hh in range(heads):
        for b in range(B):
            rs, cs = slice(hh * dh, (hh + 1) * dh), slice(b * S, (b + 1) * S)
            q, k, v, g = (X[cs, rs].astype(np.float64).T for X in (Q, K, V, dH))       # (dh, S)
            s = (q.T @ k) * scale                                                      # [query, key]
            if causal:
                s[np.triu_indices(S, 1)] = -1e9
            a = np.exp(s - s.max(1, keepdims=True))
            a /= a.sum(1, keepdims=True)
            H[cs, rs] = (v @ a.T).T
            A[hh * B + b] = a.T
            da = g.T @ v                                                               # [query, key]
            ds = a * (da - (a * da).sum(1, keepdims=True)) * scale
            dV[cs, rs] = (g @ a).T
            dQ[cs, rs] = (k @ ds.T).T
            dK[cs, rs] = (q @ ds).T
    dHm, dAm = dev_empty(N * d_k), dev_empty(S * S * B * heads)
    dq, dk, dv = to_dev(Q.reshape(-1)), to_dev(K.reshape(-1)), to_dev(V.reshape(-1))
    gpu.attention_fwd(dptr(dHm), dptr(dAm), dptr(dq), dptr(dk), dptr(dv), d_k, heads, S, B, causal)
    assert rel_err(to_host(dHm), H.reshape(-1)) <= TOL_GEMM
    assert rel_err(to_host(dAm), A.reshape(-1)) <= TOL_RED
    oq, ok_, ov, scratch = dev_empty(N * d_k), dev_empty(N * d_k), dev_empty(N * d_k), dev_empty(S * S * B * heads)
    gpu.attention_bwd(dptr(oq), dptr(ok_), dptr(ov), dptr(scratch), dp(dH.reshape(-1)), dptr(dq), dptr(dk), dptr(dv),
                      dptr(dAm), d_k, heads, S, B)
    assert rel_err(to_host(ov), dV.reshape(-1)) <= TOL_GEMM
    assert rel_err(to_host(oq), dQ.reshape(-1)) <= TOL_GEMM
    assert rel_err(to_host(ok_), dK.reshape(-1)) <= TOL_GEMM
    # the same operands as row blocks of stacked (3*d_k, N) buffers give the same bits
    import torch
    ld = 3 * d_k
    qkv = torch.stack([dq.view(N, d_k), dk.view(N, d_k), dv.view(N, d_k)], dim=1).contiguous().view(-1)
    base = qkv.data_ptr()
    Hs, As = dev_empty(N * d_k), dev_empty(S * S * B * heads)
    pq, pk, pv = (C.c_void_p(base + 4 * i * d_k) for i in range(3))
    gpu.attention_fwd_ld(dptr(Hs), d_k, dptr(As), pq, pk, pv, ld, d_k, heads, S, B, causal)
    assert np.array_equal(to_host(Hs), to_host(dHm)) and np.array_equal(to_host(As), to_host(dAm))
    dqkv = dev_empty(3 * N * d_k)
    ob = dqkv.data_ptr()
    gpu.attention_bwd_ld(C.c_void_p(ob), C.c_void_p(ob + 4 * d_k), C.c_void_p(ob + 8 * d_k), ld, dptr(scratch),
                         dp(dH.reshape(-1)), d_k, pq, pk, pv, ld, dptr(As), d_k, heads, S, B, causal)
    got = to_host(dqkv).reshape(N, 3, d_k)
    assert np.array_equal(got[:, 0].reshape(-1), to_host(oq))
    assert np.array_equal(got[:, 1].reshape(-1), to_host(ok_))
    assert np.array_equal(got[:, 2].reshape(-1), to_host(ov))
    if causal:
        # causal == 2: a second call on the same score buffers (new operands) leaves the
        # entries above the diagonal, zeros since the first call, unwritten: same bits as
        # a first call on fresh buffers
        q2 = to_dev(rng(5).normal(0, 1, 3 * N * d_k).astype(np.float32))
        b2 = q2.data_ptr()
        p2 = [C.c_void_p(b2 + 4 * i * d_k) for i in range(3)]
        g2 = to_dev(rng(6).normal(0, 1, N * d_k).astype(np.float32))
        Hf, Af, sf, of = dev_empty(N * d_k), dev_empty(S * S * B * heads), dev_empty(S * S * B * heads), dev_empty(3 * N * d_k)
        gpu.attention_fwd_ld(dptr(Hf), d_k, dptr(Af), *p2, ld, d_k, heads, S, B, 1)
        gpu.attention_bwd_ld(C.c_void_p(of.data_ptr()), C.c_void_p(of.data_ptr() + 4 * d_k),
                             C.c_void_p(of.data_ptr() + 8 * d_k), ld, dptr(sf), dptr(g2), d_k, *p2, ld, dptr(Af),
                             d_k, heads, S, B, 1)
        gpu.attention_fwd_ld(dptr(Hs), d_k, dptr(As), *p2, ld, d_k, heads, S, B, 2)
        gpu.attention_bwd_ld(C.c_void_p(ob), C.c_void_p(ob + 4 * d_k), C.c_void_p(ob + 8 * d_k), ld, dptr(scratch),
                             dptr(g2), d_k, *p2, ld, dptr(As), d_k, heads, S, B, 2)
        assert np.array_equal(to_host(Hs), to_host(Hf)) and np.array_equal(to_host(As), to_host(Af))
        assert np.array_equal(to_host(scratch), to_host(sf)) and np.array_equal(to_host(dqkv), to_host(of))


def test_second_stream_workspace_and_event_order(gpu):
    """Calls on two streams with no host synchronisation between them: each stream
    has its own split-K / reduction workspace, so concurrent launches give the
    one-stream results to the bit, and an event recorded on one stream orders a
    consumer on the other."""
    from juzhen_amd import capi
    lib = capi.load()
    r = rng(77)
    m, n, k = 256, 128, 8192              # two tiles: K is split, partials go to the workspace
    A = to_dev(r.normal(size=m * k).astype(np.float32))
    B = to_dev(r.normal(size=k * n).astype(np.float32))
    X = to_dev(r.normal(size=512 * 16384).astype(np.float32))   # row sums in chunks: workspace again
    want_c, want_r = dev_empty(m * n), dev_empty(512)
    gpu.gemm(dptr(A), dptr(B), dptr(want_c), m, n, k, 0, 1, m, n, m, 1.0, 0.0)
    gpu.sum_rows(dptr(want_r), dptr(X), 512, 16384, 512)
    gpu.synchronize()
    want_c, want_r = to_host(want_c), to_host(want_r)

    main = lib.jzhip_get_stream()
    side, ev = C.c_void_p(), C.c_void_p()
    assert lib.jzhip_stream_create(C.byref(side)) == 0 and side.value
    assert lib.jzhip_event_create(C.byref(ev)) == 0 and ev.value
    before = lib.jzhip_workspace_bytes()
    c_main = [dev_empty(m * n) for _ in range(8)]
    c_side = [dev_empty(m * n) for _ in range(8)]
    r_side = [dev_empty(512) for _ in range(8)]
    try:
        for i in range(8):
            gpu.gemm(dptr(A), dptr(B), dptr(c_main[i]), m, n, k, 0, 1, m, n, m, 1.0, 0.0)
            gpu.set_stream(side)
            gpu.sum_rows(dptr(r_side[i]), dptr(X), 512, 16384, 512)
            gpu.gemm(dptr(A), dptr(B), dptr(c_side[i]), m, n, k, 0, 1, m, n, m, 1.0, 0.0)
            gpu.set_stream(main)
        # producer on the side stream, consumer on the main stream behind an event
        buf, out = dev_empty(1 << 20), dev_empty(1 << 20)
        gpu.fill(dptr(out), 1 << 20, -1.0)
        gpu.set_stream(side)
        gpu.fill(dptr(buf), 1 << 20, 3.0)
        gpu.event_record(ev)
        gpu.set_stream(main)
        gpu.stream_wait_event(ev)
        gpu.affine(dptr(out), dptr(buf), 1 << 20, 2.0, 1.0)
        gpu.set_stream(side)
        gpu.synchronize()
        gpu.set_stream(main)
        gpu.synchronize()
    finally:
        lib.jzhip_set_stream(main)
    during = lib.jzhip_workspace_bytes()
    assert during == before + (64 << 20)   # the side stream's own
    for i in range(8):
        assert np.array_equal(to_host(c_main[i]), want_c)
        assert np.array_equal(to_host(c_side[i]), want_c)
        assert np.array_equal(to_host(r_side[i]), want_r)
    assert np.array_equal(to_host(out), np.full(1 << 20, 7.0, np.float32))
    assert lib.jzhip_event_record(None) == -1
    assert lib.jzhip_stream_wait_event(None) == -1
    assert lib.jzhip_stream_create(None) == -1 and lib.jzhip_event_create(None) == -1
    assert lib.jzhip_event_destroy(ev) == 0
    assert lib.jzhip_stream_destroy(side) == 0
    assert lib.jzhip_workspace_bytes() == before   # given back with the stream


@pytest.mark.parametrize("d,V,S,B,with_bias", [(512, 256, 256, 4, 0), (64, 13, 8, 3, 1), (30, 5, 7, 2, 1), (4, 3, 1, 9, 0)])
def test_embedding_fwd(gpu, oracle_lib, d, V, S, B, with_bias):
    """Lookup against the oracle (bit-exact: one addition or two per element) and
    against the one-hot products it replaces, through the library's own GEMM."""
    r = rng(d + V)
    N = S * B
    E = r.normal(size=V * d).astype(np.float32)
    Pm = r.normal(size=S * d).astype(np.float32)
    bias = r.normal(size=d).astype(np.float32)
    tok = r.integers(0, V, N).astype(np.int32)
    if N > 2:
        tok[1], tok[2] = -3, V + 5
    want = np.empty(N * d, np.float32)
    oracle_lib.jzo_embedding_fwd(hptr(want), hptr(E), hptr(Pm), hptr(bias) if with_bias else None, hptr(tok), d, V, S, N)
    import torch
    dtok = torch.from_numpy(tok).cuda()
    dE, dP, db = to_dev(E), to_dev(Pm), to_dev(bias)
    out = dev_empty(N * d)
    gpu.embedding_fwd(dptr(out), dptr(dE), dptr(dP), dptr(db) if with_bias else None, dptr(dtok), d, V, S, N)
    got = to_host(out)
    assert np.array_equal(got, want)
    # the two one-hot products (+ bias broadcast) on the GPU
    oh = np.zeros((N, V), np.float32)
    for n, t in enumerate(tok):
        if 0 <= t < V:
            oh[n, t] = 1.0
    op = np.zeros((N, S), np.float32)
    op[np.arange(N), np.arange(N) % S] = 1.0
    x0 = dev_empty(N * d)
    gpu.gemm(dptr(dE), dp(oh.ravel()), dptr(x0), d, N, V, 0, 0, d, V, d, 1.0, 0.0)
    gpu.gemm(dptr(dP), dp(op.ravel()), dptr(x0), d, N, S, 0, 0, d, S, d, 1.0, 1.0)
    if with_bias:
        gpu.add_bias(dptr(x0), dptr(db), d, N)
    assert np.array_equal(to_host(x0), got)
    from juzhen_amd import capi
    assert capi.load().jzhip_embedding_fwd(dptr(out), None, dptr(dP), None, dptr(dtok), d, V, S, N) == -1
    assert capi.load().jzhip_embedding_fwd(dptr(out), dptr(dE), dptr(dP), None, dptr(dtok), 0, V, S, N) == -1


def test_page_locked_host_memory_and_asynchronous_copies(gpu):
    """jzhip_host_alloc / jzhip_memcpy_h2d_async / _d2h_async / jzhip_event_synchronize:
    a round trip through the device behind a kernel on the same stream, with the
    host waiting on an event instead of draining the stream."""
    from juzhen_amd import capi
    lib = capi.load()
    n = 1 << 20
    src, dst, ev = C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert lib.jzhip_host_alloc(C.byref(src), 4 * n) == 0 and src.value
    assert lib.jzhip_host_alloc(C.byref(dst), 4 * n) == 0 and dst.value
    assert lib.jzhip_event_create(C.byref(ev)) == 0
    try:
        a = np.ctypeslib.as_array(C.cast(src, C.POINTER(C.c_float)), shape=(n,))
        b = np.ctypeslib.as_array(C.cast(dst, C.POINTER(C.c_float)), shape=(n,))
        a[:] = rng(1).normal(size=n).astype(np.float32)
        b[:] = 0
        d_in, d_out = dev_empty(n), dev_empty(n)
        gpu.memcpy_h2d_async(dptr(d_in), src, 4 * n)
        gpu.affine(dptr(d_out), dptr(d_in), n, 2.0, 1.0)          # 2*x + 1 behind the copy
        gpu.memcpy_d2h_async(dst, dptr(d_out), 4 * n)
        gpu.event_record(ev)
        gpu.event_synchronize(ev)
        assert np.array_equal(b, a * np.float32(2.0) + np.float32(1.0))
        assert lib.jzhip_memcpy_h2d_async(None, src, 16) == -1
        assert lib.jzhip_memcpy_h2d_async(dptr(d_in), src, 0) == 0
        assert lib.jzhip_event_synchronize(None) == -1
    finally:
        gpu.synchronize()
        lib.jzhip_event_destroy(ev)
        assert lib.jzhip_host_free(src) == 0 and lib.jzhip_host_free(dst) == 0
    assert lib.jzhip_host_alloc(None, 16) == -1 and lib.jzhip_host_free(None) == 0

