"""GEMM parity at the shapes the benchmark configurations and the 4096^3
target actually run, through the C ABI.

The operands are too large for the scalar CPU oracle, so each product is
checked on >= 4096 sampled entries of C against float64 dot products of the
same operand rows/columns (the method of tests/testCpuLinalg.cu:54-66 on a
sample; tolerance 1e-3 relative to the entry scale sqrt(k)), plus properties
that hold at any size: the whole result is finite, and a fused tail equals
jzhip_gemm followed by the separate kernels bit for bit.  torch is used as
device-memory plumbing only (random operands, gathers of the sampled rows).
"""
import ctypes as C
import math

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOL_GEMM = 1e-3
SAMPLES = 4096


def dptr(t):
    return C.c_void_p(t.data_ptr())


def operands(m, n, k, ta, tb, seed):
    """Device operands: A physically (k x m if ta else m x k), B (n x k if tb
    else k x n), column-major dense; entries N(0,1)."""
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    # torch tensors are row-major: a column-major (r x c) buffer is a (c, r) tensor
    A = torch.randn((m, k) if ta else (k, m), generator=g, device="cuda")
    B = torch.randn((k, n) if tb else (n, k), generator=g, device="cuda")
    return A, B


def op_rows_cols(A, B, ta, tb, ii, jj):
    """float64 rows ii of op(A) (len(ii) x k) and columns jj of op(B) (len(jj) x k) on the host."""
    import torch
    ii_t = torch.as_tensor(ii, device="cuda")
    jj_t = torch.as_tensor(jj, device="cuda")
    # A tensor is (k, m) for N (col-major m x k): op(A)[i, :] = A[:, i]; for T it is (m, k): row i
    rows = (A[ii_t, :] if ta else A[:, ii_t].T).double().cpu().numpy()
    # B tensor is (n, k) for N: op(B)[:, j] = B[j, :]; for T it is (k, n): column j
    cols = (B[:, jj_t].T if tb else B[jj_t, :]).double().cpu().numpy()
    return rows, cols


def check_sampled(Cdev, A, B, m, n, k, ta, tb, seed, ldc=None, extra=None):
    """Compare SAMPLES entries of C (column-major, ld = ldc) with float64 dot products.
    `extra(i, j, v)` maps the float64 product to the expected stored value."""
    import torch
    ldc = ldc or m
    r = np.random.default_rng(seed)
    ii = r.integers(0, m, SAMPLES)
    jj = r.integers(0, n, SAMPLES)
    # corners and tile edges are where a wrong bound shows
    edge_i = np.array([0, m - 1, min(m - 1, 127), min(m - 1, 128), m // 2])
    edge_j = np.array([0, n - 1, min(n - 1, 127), min(n - 1, 128), n // 2])
    ii[:25] = np.repeat(edge_i, 5)
    jj[:25] = np.tile(edge_j, 5)
    want = np.empty(SAMPLES)
    for s in range(0, SAMPLES, 512):
        rows, cols = op_rows_cols(A, B, ta, tb, ii[s:s + 512], jj[s:s + 512])
        want[s:s + 512] = np.einsum("sk,sk->s", rows, cols)
    if extra is not None:
        want = extra(ii, jj, want)
    flat = torch.as_tensor(jj.astype(np.int64) * ldc + ii, device="cuda")
    got = Cdev.reshape(-1)[flat].double().cpu().numpy()
    err = np.max(np.abs(got - want)) / math.sqrt(k)
    assert err <= TOL_GEMM, (err, m, n, k, ta, tb)
    rel = np.linalg.norm(got - want) / np.linalg.norm(want)
    assert rel <= TOL_GEMM, rel
    return rel


def run_gemm(gpu, m, n, k, ta, tb, seed, alpha=1.0):
    import torch
    A, B = operands(m, n, k, ta, tb, seed)
    Cd = torch.full((n * m,), float("nan"), device="cuda")
    lda, ldb = (k if ta else m), (n if tb else k)
    gpu.gemm(dptr(A), dptr(B), dptr(Cd), m, n, k, ta, tb, lda, ldb, m, alpha, 0.0)
    gpu.synchronize()
    assert bool(torch.isfinite(Cd).all())
    rel = check_sampled(Cd, A, B, m, n, k, ta, tb, seed + 1,
                        extra=(lambda i, j, v: alpha * v) if alpha != 1.0 else None)
    return rel


# ── the 4096^3 target point, all four transpose variants ─────────────────
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_4096_cubed(gpu, ta, tb):
    run_gemm(gpu, 4096, 4096, 4096, ta, tb, 40 + 2 * ta + tb)


# ── transformer configuration (d 512, ff 2048, 16384 tokens, 6 blocks) ────
C4_SHAPES = [
    # forward NN: Q/K/V/O projections, stacked QKV, FFN up and down, tied head
    (512, 16384, 512, 0, 0), (1536, 16384, 512, 0, 0), (2048, 16384, 512, 0, 0), (512, 16384, 2048, 0, 0),
    (256, 16384, 512, 1, 0),
    # weight gradients NT, K = 16384 tokens (split along K)
    (512, 512, 16384, 0, 1), (1536, 512, 16384, 0, 1), (2048, 512, 16384, 0, 1), (512, 2048, 16384, 0, 1),
    (512, 256, 16384, 0, 1),
    # input gradients TN
    (512, 16384, 512, 1, 0), (512, 16384, 1536, 1, 0), (512, 16384, 2048, 1, 0), (2048, 16384, 512, 1, 0),
    (512, 16384, 256, 0, 0),
]


@pytest.mark.parametrize("m,n,k,ta,tb", C4_SHAPES)
def test_gemm_transformer_shapes(gpu, m, n, k, ta, tb):
    run_gemm(gpu, m, n, k, ta, tb, m + n + k + ta * 3 + tb * 5)


# ── CNN and UNet configurations: im2col products (forward TN C_out x n x K,
#    weight gradient NT K x C_out x n, input gradient NN K x n x C_out) and
#    transposed convolutions (forward NN R x n x C_in, weight gradient NT
#    R x C_in x n, input gradient TN C_in x n x R) ─────────────────────────
CONV_LAYERS = [  # (C_out, n, K)
    (32, 100352, 9), (64, 25088, 288),                                       # CNN conv1, conv2
    (64, 131072, 99), (128, 32768, 576), (256, 8192, 1152), (256, 8192, 2304),  # UNet enc1-3, mid
    (128, 32768, 2304), (64, 131072, 1152), (3, 131072, 576),                # dec2, dec1, head
    (64, 131072, 27), (64, 131072, 576), (128, 32768, 1152),                 # two-conv-per-level variant
]
CONVT_LAYERS = [(2048, 8192, 256), (1024, 32768, 128)]                       # (R, n, C_in): up2, up1


def conv_products():
    out = []
    for co, n, K in CONV_LAYERS:
        out += [(co, n, K, 1, 0), (K, co, n, 0, 1), (K, n, co, 0, 0)]
    for R, n, ci in CONVT_LAYERS:
        out += [(R, n, ci, 0, 0), (R, ci, n, 0, 1), (ci, n, R, 1, 0)]
    out += [(10, 128, 12544, 0, 0), (10, 12544, 128, 0, 1), (12544, 128, 10, 1, 0)]   # CNN classifier
    return out


@pytest.mark.parametrize("m,n,k,ta,tb", conv_products())
def test_gemm_conv_shapes(gpu, m, n, k, ta, tb):
    run_gemm(gpu, m, n, k, ta, tb, (m * 31 + n * 7 + k) % 100000)


# ── fused tails at the FFN shapes ────────────────────────────────────────
def gelu64(v):
    from scipy.special import erf
    return 0.5 * v * (1 + erf(v / math.sqrt(2)))


def dgelu64(p):
    from scipy.special import erf
    return 0.5 * (1 + erf(p / math.sqrt(2))) + p * np.exp(-0.5 * p * p) / math.sqrt(2 * math.pi)


@pytest.mark.parametrize("m,n,k,ta,act", [
    (2048, 16384, 512, 0, 2),     # FFN up: bias + GELU, pre-activation saved
    (2048, 16384, 512, 1, 4),     # FFN backward: W2^T dy times GELU'(saved pre-activation)
    (2048, 16384, 512, 0, 1),     # the reference's ReLU FFN
    (2048, 16384, 512, 1, 3),
    (512, 16384, 2048, 0, 0),     # FFN down: bias + residual
    (512, 16384, 512, 0, 0),      # attention output projection: bias + residual
])
def test_gemm_fused_tails_at_ffn_shapes(gpu, m, n, k, ta, act):
    import torch
    seed = m + k + act
    A, B = operands(m, n, k, ta, 0, seed)
    A *= 1.0 / math.sqrt(k)                         # pre-activations of order one
    g = torch.Generator(device="cuda")
    g.manual_seed(seed + 7)
    bias = torch.randn(m, generator=g, device="cuda")
    res = torch.randn(n * m, generator=g, device="cuda")
    pre = torch.randn(n * m, generator=g, device="cuda")
    lda, ldb = (k if ta else m), k
    use_bias = act in (0, 1, 2)
    use_res = act == 0
    # separate kernels
    sep = torch.empty(n * m, device="cuda")
    gpu.gemm(dptr(A), dptr(B), dptr(sep), m, n, k, ta, 0, lda, ldb, m, 1.0, 0.0)
    if use_bias:
        gpu.add_bias(dptr(sep), dptr(bias), m, n)
    want_aux = sep.clone()
    if act == 1:
        gpu.relu(dptr(sep), dptr(sep), m * n)
    elif act == 2:
        gpu.gelu(dptr(sep), dptr(sep), m * n)
    elif act == 3:
        gpu.drelu_mul(dptr(sep), dptr(pre), dptr(sep), m * n)
    elif act == 4:
        gpu.dgelu_mul(dptr(sep), dptr(pre), dptr(sep), m * n)
    if use_res:
        gpu.axpby(dptr(sep), dptr(sep), dptr(res), m * n, 1.0, 1.0)
    # fused
    fused = torch.full((n * m,), float("nan"), device="cuda")
    aux = pre.clone() if act in (3, 4) else torch.full((n * m,), float("nan"), device="cuda")
    gpu.gemm_fused(dptr(A), dptr(B), dptr(fused), m, n, k, ta, 0, lda, ldb, m, 1.0, 0.0,
                   dptr(bias) if use_bias else None, act, dptr(aux) if act else None, m,
                   dptr(res) if use_res else None, m)
    gpu.synchronize()
    assert torch.equal(fused, sep)
    if act in (1, 2):
        assert torch.equal(aux, want_aux)
    bias_h = bias.double().cpu().numpy()
    res_h, pre_h = res, pre

    def tail(ii, jj, v):
        flat = torch.as_tensor(jj.astype(np.int64) * m + ii, device="cuda")
        if use_bias:
            v = v + bias_h[ii]
        if act == 1:
            v = np.maximum(v, 0)
        elif act == 2:
            v = gelu64(v)
        elif act == 3:
            v = v * (pre_h[flat].double().cpu().numpy() > 0)
        elif act == 4:
            v = v * dgelu64(pre_h[flat].double().cpu().numpy())
        if use_res:
            v = v + res_h[flat].double().cpu().numpy()
        return v

    import torch  # noqa: F811  (closure above uses it)
    # entries are O(1): the sampled check's sqrt(k) scale would be too lenient, use the plain relative norm
    r = np.random.default_rng(seed)
    ii = r.integers(0, m, SAMPLES)
    jj = r.integers(0, n, SAMPLES)
    rows, cols = [], []
    want = np.empty(SAMPLES)
    for s in range(0, SAMPLES, 512):
        rows, cols = op_rows_cols(A, B, ta, 0, ii[s:s + 512], jj[s:s + 512])
        want[s:s + 512] = np.einsum("sk,sk->s", rows, cols)
    want = tail(ii, jj, want)
    flat = torch.as_tensor(jj.astype(np.int64) * m + ii, device="cuda")
    got = fused[flat].double().cpu().numpy()
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= TOL_GEMM
    assert np.max(np.abs(got - want)) <= TOL_GEMM * (1 + np.max(np.abs(want)))


# ── strided batches at the attention shapes (d_h 64, S 256, 512 blocks) ───
@pytest.mark.parametrize("m,n,k,ta,tb", [(256, 256, 64, 1, 0), (64, 256, 256, 0, 1), (64, 256, 256, 0, 0)])
def test_gemm_strided_batched_attention_shapes(gpu, m, n, k, ta, tb):
    import torch
    batch = 512
    g = torch.Generator(device="cuda")
    g.manual_seed(m + k)
    A = torch.randn((batch, m, k) if ta else (batch, k, m), generator=g, device="cuda")
    B = torch.randn((batch, k, n) if tb else (batch, n, k), generator=g, device="cuda")
    Cd = torch.full((batch, n, m), float("nan"), device="cuda")
    lda, ldb = (k if ta else m), (n if tb else k)
    gpu.gemm_strided_batched(dptr(A), dptr(B), dptr(Cd), m, n, k, ta, tb, lda, ldb, m, m * k, k * n, m * n,
                             batch, 0.125, 0.0)
    gpu.synchronize()
    opA = A.double() if ta else A.double().transpose(1, 2)            # (batch, m, k)
    opB = B.double().transpose(1, 2) if tb else B.double()            # (batch, n, k)
    for b in (0, 1, 255, 511):
        want = 0.125 * (opA[b] @ opB[b].T).T                          # (n, m) == column-major m x n
        got = Cd[b].double()
        rel = float((got - want).norm() / want.norm())
        assert rel <= TOL_GEMM, (b, rel)
    assert bool(torch.isfinite(Cd).all())
