"""Attention without the S x S matrices (jzhip_attention_flash_fwd / _bwd) through the C ABI.

Checked against a float64 restatement of the per-(head, sequence) loop of
ml/layer.hpp:2967-3006 and 3329-3363 (the method of tests/testTransformerRef.cu:102-141)
and against the materialising pair jzhip_attention_fwd_ld / _bwd_ld on the same operands,
both within 1e-4 (relative, norm-wise), at the shapes of the materialising pair's own test
that the kernels cover; the other shapes must be refused."""
import ctypes as C

import numpy as np
import pytest

from util import dev_empty, dptr, rel_err, to_dev, to_host

pytestmark = pytest.mark.gpu
TOL = 1e-4

SHAPES = [(8, 4, 3, 2, 1), (16, 2, 5, 3, 0), (64, 1, 17, 2, 1), (128, 2, 64, 3, 1), (512, 8, 32, 2, 1),
          (512, 8, 256, 2, 1), (256, 4, 128, 1, 0), (64, 2, 96, 2, 1), (128, 2, 160, 1, 1), (128, 4, 224, 1, 0),
          (512, 8, 256, 3, 0), (128, 4, 256, 2, 1)]


def float64_attention(Q, K, V, dH, d_k, heads, S, B, causal):
    """Q, K, V, dH as (N, d_k) arrays [column, row]; returns H, dQ, dK, dV likewise and the
    row maxima / reciprocal sums per block."""
    N, dh = S * B, d_k // heads
    H, dQ, dK, dV = (np.zeros((N, d_k)) for _ in range(4))
    mx, inv = np.zeros((heads * B, S)), np.zeros((heads * B, S))
    scale = 1.0 / np.sqrt(np.float32(dh))
    for hh in range(heads):
        for b in range(B):
            rs, cs = slice(hh * dh, (hh + 1) * dh), slice(b * S, (b + 1) * S)
            q, k, v, g = (X[cs, rs].astype(np.float64).T for X in (Q, K, V, dH))       # (dh, S)
            s = (q.T @ k) * scale                                                      # [query, key]
            if causal:
                s[np.triu_indices(S, 1)] = -1e9
            e = np.exp(s - s.max(1, keepdims=True))
            mx[hh * B + b], inv[hh * B + b] = s.max(1), 1.0 / e.sum(1)
            a = e / e.sum(1, keepdims=True)
            H[cs, rs] = (v @ a.T).T
            da = g.T @ v
            ds = a * (da - (a * da).sum(1, keepdims=True)) * scale
            dV[cs, rs] = (g @ a).T
            dQ[cs, rs] = (k @ ds.T).T
            dK[cs, rs] = (q @ ds).T
    return H, dQ, dK, dV, mx, inv


@pytest.mark.parametrize("d_k,heads,S,B,causal", SHAPES)
def test_flash_attention_against_float64_and_the_materialising_path(gpu, d_k, heads, S, B, causal):
    from juzhen_amd import capi
    lib = capi.load()
    N, dh = S * B, d_k // heads
    r = np.random.default_rng(d_k + 3 * S + B + causal)
    Q, K, V, dH = (r.normal(0, 1, (N, d_k)).astype(np.float32) for _ in range(4))
    dq, dk, dv, dg = (to_dev(X.reshape(-1)) for X in (Q, K, V, dH))
    Hf, stats = dev_empty(N * d_k), dev_empty(2 * S * heads * B)
    oq, ok_, ov = (to_dev(np.full(N * d_k, np.nan, np.float32)) for _ in range(3))
    supported = dh in (32, 64) and S % 32 == 0 and S <= 256
    assert lib.jzhip_attention_flash_supported(d_k, heads, S, B) == int(supported)
    if not supported:
        assert lib.jzhip_attention_flash_fwd(dptr(Hf), d_k, dptr(stats), dptr(dq), dptr(dk), dptr(dv), d_k, d_k, heads,
                                             S, B, causal) == -1
        assert lib.jzhip_attention_flash_bwd(dptr(oq), dptr(ok_), dptr(ov), d_k, dptr(dg), d_k, dptr(dq), dptr(dk),
                                             dptr(dv), d_k, dptr(Hf), d_k, dptr(stats), d_k, heads, S, B, causal) == -1
        return
    H, dQ, dK, dV, mx, inv = float64_attention(Q, K, V, dH, d_k, heads, S, B, causal)
    print(f"flash attention d_k {d_k} heads {heads} S {S} B {B} causal {causal}", flush=True)
    gpu.attention_flash_fwd(dptr(Hf), d_k, dptr(stats), dptr(dq), dptr(dk), dptr(dv), d_k, d_k, heads, S, B, causal)
    assert rel_err(to_host(Hf), H.reshape(-1)) <= TOL
    st = to_host(stats).reshape(heads * B, 2, S)
    assert np.allclose(st[:, 0], mx, rtol=1e-5, atol=1e-5)
    assert np.allclose(st[:, 1], inv, rtol=1e-4)
    gpu.attention_flash_bwd(dptr(oq), dptr(ok_), dptr(ov), d_k, dptr(dg), d_k, dptr(dq), dptr(dk), dptr(dv), d_k,
                            dptr(Hf), d_k, dptr(stats), d_k, heads, S, B, causal)
    gq, gk, gv = to_host(oq), to_host(ok_), to_host(ov)
    assert np.isfinite(gq).all() and np.isfinite(gk).all() and np.isfinite(gv).all()
    errs = {n: rel_err(g, w.reshape(-1)) for n, g, w in (("dQ", gq, dQ), ("dK", gk, dK), ("dV", gv, dV))}
    print("   against float64:", {n: f"{e:.1e}" for n, e in errs.items()})
    assert max(errs.values()) <= TOL, errs

    # the materialising pair on the same operands
    Hm, A, scratch = dev_empty(N * d_k), dev_empty(S * S * heads * B), dev_empty(S * S * heads * B)
    mq, mk, mv = dev_empty(N * d_k), dev_empty(N * d_k), dev_empty(N * d_k)
    gpu.attention_fwd_ld(dptr(Hm), d_k, dptr(A), dptr(dq), dptr(dk), dptr(dv), d_k, d_k, heads, S, B, causal)
    gpu.attention_bwd_ld(dptr(mq), dptr(mk), dptr(mv), d_k, dptr(scratch), dptr(dg), d_k, dptr(dq), dptr(dk), dptr(dv),
                         d_k, dptr(A), d_k, heads, S, B, causal)
    assert np.array_equal(to_host(Hm), to_host(Hf))                # the forward kernel is the same code
    for n, g, m in (("dQ", gq, mq), ("dK", gk, mk), ("dV", gv, mv)):
        assert rel_err(g, to_host(m)) <= TOL, n

    # operands as row blocks of stacked (3*d_k, N) buffers, output likewise: same bits; and a second
    # run gives the same bits as the first (every sum has one fixed order)
    import torch
    ld = 3 * d_k
    qkv = torch.stack([dq.view(N, d_k), dk.view(N, d_k), dv.view(N, d_k)], dim=1).contiguous().view(-1)
    base = qkv.data_ptr()
    pq, pk, pv = (C.c_void_p(base + 4 * i * d_k) for i in range(3))
    Hs, st2 = dev_empty(N * d_k), dev_empty(2 * S * heads * B)
    gpu.attention_flash_fwd(dptr(Hs), d_k, dptr(st2), pq, pk, pv, ld, d_k, heads, S, B, causal)
    assert np.array_equal(to_host(Hs), to_host(Hf)) and np.array_equal(to_host(st2), to_host(stats))
    for _ in range(2):
        out = to_dev(np.full(3 * N * d_k, np.nan, np.float32))
        ob = out.data_ptr()
        gpu.attention_flash_bwd(C.c_void_p(ob), C.c_void_p(ob + 4 * d_k), C.c_void_p(ob + 8 * d_k), ld, dptr(dg), d_k,
                                pq, pk, pv, ld, dptr(Hs), d_k, dptr(st2), d_k, heads, S, B, causal)
        got = to_host(out).reshape(N, 3, d_k)
        assert np.array_equal(got[:, 0].reshape(-1), gq)
        assert np.array_equal(got[:, 1].reshape(-1), gk)
        assert np.array_equal(got[:, 2].reshape(-1), gv)


def test_flash_attention_rejects_bad_arguments(gpu):
    from juzhen_amd import capi
    lib = capi.load()
    d = dev_empty(64 * 64 * 4)
    p = dptr(d)
    ok = (p, 64, p, p, p, p, 64, 64, 1, 64, 1, 1)
    assert lib.jzhip_attention_flash_fwd(None, *ok[1:]) == -1
    assert lib.jzhip_attention_flash_fwd(p, 64, p, p, p, p, 64, 64, 1, 64, 1, 2) == -1      # causal is 0 or 1
    assert lib.jzhip_attention_flash_fwd(p, 32, p, p, p, p, 64, 64, 1, 64, 1, 1) == -1      # ld below d_k
    assert lib.jzhip_attention_flash_bwd(p, p, p, 64, p, 64, p, p, p, 64, p, 64, None, 64, 1, 64, 1, 1) == -1
    assert lib.jzhip_attention_flash_bwd(p, p, p, 66, p, 64, p, p, p, 64, p, 64, p, 64, 1, 64, 1, 1) == -1   # ld % 4
    off = C.c_void_p(d.data_ptr() + 4)
    assert lib.jzhip_attention_flash_bwd(off, p, p, 64, p, 64, p, p, p, 64, p, 64, p, 64, 1, 64, 1, 1) == -1  # alignment
