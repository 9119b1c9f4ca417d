#!/usr/bin/env python3
"""Per-kernel roofline report for the MI355X backend.

    python -m juzhen_amd.opbench [--groups gemm,ew,reduce,fused,conv,broadcast,conv_implicit] [--out FILE]

Every line is one C-ABI entry point at one shape: median and p95 launch time
over 20 samples after 3 warm-ups (the reference's convention,
tests/benchmarkCoreOps.cu:35-54 and tests/benchmarkTrainingStep.cu:73-74),
the algorithmic bytes or flops of the call, and the fraction of the bound that
applies (HBM 8 TB/s for streaming kernels, 157.3 TFLOP/s fp32 MFMA for GEMM).
A sample is a HIP-event pair around enough back-to-back launches to last
about 100 us, so short kernels are not priced at event resolution.

The report is a Markdown table on stdout (or --out).
"""
from __future__ import annotations

import argparse
import ctypes as C
import sys
from pathlib import Path

import torch

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))

from juzhen_amd import capi  # noqa: E402

HBM_GBS = 8000.0
MFMA_TFLOPS = 157.3


class _Events:
    def __init__(self):
        h = self.hip = C.CDLL("libamdhip64.so")
        h.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        h.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        h.hipEventSynchronize.argtypes = [C.c_void_p]
        h.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.a, self.b = C.c_void_p(), C.c_void_p()
        assert h.hipEventCreate(C.byref(self.a)) == 0 and h.hipEventCreate(C.byref(self.b)) == 0

    def time_ms(self, fn, reps, stream):
        h = self.hip
        assert h.hipEventRecord(self.a, stream) == 0
        for _ in range(reps):
            fn()
        assert h.hipEventRecord(self.b, stream) == 0
        assert h.hipEventSynchronize(self.b) == 0
        ms = C.c_float()
        assert h.hipEventElapsedTime(C.byref(ms), self.a, self.b) == 0
        return ms.value / reps


class Report:
    def __init__(self):
        self.lib = capi.load()
        self.jz = capi.jz
        self.ev = _Events()
        self.stream = C.c_void_p(self.lib.jzhip_get_stream())
        self.rows = []

    def run(self, group, name, shape, fn, *, bytes_=None, flops=None, samples=20, warm=3):
        for _ in range(warm):
            fn()
        first = self.ev.time_ms(fn, 1, self.stream)
        reps = max(1, min(64, int(0.1 / max(first, 1e-4))))
        ts = sorted(self.ev.time_ms(fn, reps, self.stream) for _ in range(samples))
        med = ts[len(ts) // 2]
        p95 = ts[min(len(ts) - 1, int(round(0.95 * (len(ts) - 1))))]
        if flops is not None:
            ach = flops / (med * 1e-3) / 1e12
            self.rows.append((group, name, shape, med, p95, f"{flops / 1e9:.2f} GF", f"{ach:.1f} TFLOP/s", ach / MFMA_TFLOPS, "mfma"))
        else:
            ach = bytes_ / (med * 1e-3) / 1e9
            self.rows.append((group, name, shape, med, p95, f"{bytes_ / 1e6:.2f} MB", f"{ach:.0f} GB/s", ach / HBM_GBS, "hbm"))
        print(f"{group} {name} {shape}: {med * 1e3:.1f} us  {self.rows[-1][6]}", file=sys.stderr, flush=True)

    def markdown(self):
        out = ["| group | entry point | shape | median us | p95 us | algorithmic | achieved | bound | frac |",
               "|---|---|---|---:|---:|---:|---:|---|---:|"]
        for g, n, s, med, p95, alg, ach, frac, bound in self.rows:
            out.append(f"| {g} | {n} | {s} | {med * 1e3:.1f} | {p95 * 1e3:.1f} | {alg} | {ach} | {bound} | {frac:.2f} |")
        return "\n".join(out) + "\n"


def P(t):
    return C.c_void_p(t.data_ptr())


def dev(n, fill=None):
    if fill is None:
        return torch.randn(n, device="cuda")
    return torch.full((n,), float(fill), device="cuda")


def bench_gemm(r):
    jz = r.jz
    shapes = [
        # (label, m, n, k, ta, tb)
        ("C1 chain NN", 1024, 1024, 1024, 0, 0),
        ("C2 fwd NN", 256, 4096, 256, 0, 0), ("C2 dW NT", 256, 256, 4096, 0, 1), ("C2 dx TN", 256, 4096, 256, 1, 0),
        ("C3 conv2 fwd TN", 64, 25088, 288, 1, 0), ("C3 conv2 dW NT", 288, 64, 25088, 0, 1),
        ("C3 conv2 dcol NN", 288, 25088, 64, 0, 0),
        ("C4 proj NN", 512, 16384, 512, 0, 0), ("C4 ffn1 NN", 2048, 16384, 512, 0, 0),
        ("C4 ffn2 NN", 512, 16384, 2048, 0, 0), ("C4 dx TN", 512, 16384, 2048, 1, 0),
        ("C4 dx TN", 2048, 16384, 512, 1, 0), ("C4 dW NT", 512, 512, 16384, 0, 1),
        ("C4 dW NT", 2048, 512, 16384, 0, 1), ("C4 dW NT", 512, 2048, 16384, 0, 1),
        ("C4 logits TN", 256, 16384, 512, 1, 0),
        # C5 (UNet, 128 images of 32 x 32): 3x3 convolutions 64 -> 64, 128 -> 64 and the 64 -> 3 output layer
        ("C5 conv 64>64 fwd TN", 64, 131072, 576, 1, 0), ("C5 conv 64>64 dW NT", 576, 64, 131072, 0, 1),
        ("C5 conv 64>64 dcol NN", 576, 131072, 64, 0, 0), ("C5 conv 128>64 fwd TN", 64, 131072, 1152, 1, 0),
        ("C5 conv 128>64 dW NT", 1152, 64, 131072, 0, 1), ("C5 conv 128>64 dcol NN", 1152, 131072, 64, 0, 0),
        ("C5 conv 128>128 fwd TN", 128, 32768, 1152, 1, 0), ("C5 conv 128>128 dW NT", 1152, 128, 32768, 0, 1),
        ("C5 up 256>128 fwd NN", 2048, 8192, 256, 0, 0),
        ("square NN", 4096, 4096, 4096, 0, 0), ("square NT", 4096, 4096, 4096, 0, 1),
        ("square TN", 4096, 4096, 4096, 1, 0), ("square TT", 4096, 4096, 4096, 1, 1),
        ("square NN", 8192, 8192, 8192, 0, 0), ("square TN", 8192, 8192, 8192, 1, 0),
    ]
    for label, m, n, k, ta, tb in shapes:
        A, B, Cm = dev(m * k), dev(k * n), dev(m * n, 0)
        lda, ldb = (k if ta else m), (n if tb else k)
        r.run("gemm", f"jzhip_gemm {label}", f"{m}x{n}x{k}",
              lambda: jz.gemm(P(A), P(B), P(Cm), m, n, k, ta, tb, lda, ldb, m, 1.0, 0.0), flops=2.0 * m * n * k)
    # thin products (m or n <= 8) are bound by reading the big operand once
    for label, m, n, k, ta, tb in (("C5 output conv fwd TN (thin)", 3, 131072, 576, 1, 0),
                                   ("C5 output conv dW NT (thin)", 576, 3, 131072, 0, 1)):
        A, B, Cm = dev(m * k), dev(k * n), dev(m * n, 0)
        lda, ldb = (k if ta else m), (n if tb else k)
        r.run("gemm", f"jzhip_gemm {label}", f"{m}x{n}x{k}",
              lambda: jz.gemm(P(A), P(B), P(Cm), m, n, k, ta, tb, lda, ldb, m, 1.0, 0.0),
              bytes_=4.0 * (m * k + k * n + m * n))
    # products with the layer's elementwise tail fused into the store (C4 shapes)
    for label, m, n, k, ta, act, use_res in (("C4 Wo: bias+residual NN", 512, 16384, 512, 0, 0, 1),
                                             ("C4 W2: bias+residual NN", 512, 16384, 2048, 0, 0, 1),
                                             ("C4 W1: bias+gelu(+pre) NN", 2048, 16384, 512, 0, 2, 0),
                                             ("C4 dF1: .*gelu'(pre) TN", 2048, 16384, 512, 1, 4, 0)):
        A, B, Cm = dev(m * k), dev(k * n), dev(m * n, 0)
        bias, aux, res = dev(m), dev(m * n), dev(m * n)
        lda = k if ta else m
        r.run("gemm", f"jzhip_gemm_fused {label}", f"{m}x{n}x{k}",
              lambda: jz.gemm_fused(P(A), P(B), P(Cm), m, n, k, ta, 0, lda, k, m, 1.0, 0.0,
                                    P(bias) if act != 4 else None, act, P(aux) if act else None, m,
                                    P(res) if use_res else None, m), flops=2.0 * m * n * k)
    # the same store with the row sums of the result (the bias gradient of the layer below) on the side
    m, n, k = 2048, 16384, 512
    A, B, Cm, aux, rs = dev(m * k), dev(k * n), dev(m * n, 0), dev(m * n), dev(m, 0)
    r.run("gemm", "jzhip_gemm_fused_rowsum C4 dF1: .*gelu'(pre) TN + row sums", f"{m}x{n}x{k}",
          lambda: jz.gemm_fused_rowsum(P(A), P(B), P(Cm), P(rs), m, n, k, 1, 0, k, k, m, 1.0, 0.0, None, 4, P(aux), m, None, m),
          flops=2.0 * m * n * k)
    # a dense layer's weight and bias gradients from one pass over the upstream gradient
    for label, m, n, k in (("C2 dW + db NT", 256, 256, 4096), ("C4 dW1 + db1 NT", 2048, 512, 16384)):
        A, B, Cm, rs = dev(m * k), dev(n * k), dev(m * n, 0), dev(m, 0)
        r.run("gemm", f"jzhip_gemm_rowsum {label}", f"{m}x{n}x{k}",
              lambda: jz.gemm_rowsum(P(A), P(B), P(Cm), P(rs), m, n, k, 0, 1, m, n, m, 1.0, 0.0), flops=2.0 * m * n * k)
        r.run("gemm", f"jzhip_gemm + jzhip_sum_rows {label}", f"{m}x{n}x{k}",
              lambda: (jz.gemm(P(A), P(B), P(Cm), m, n, k, 0, 1, m, n, m, 1.0, 0.0), jz.sum_rows(P(rs), P(A), m, k, m)),
              flops=2.0 * m * n * k)
    # attention-shaped strided batches (C4: 512 blocks of 256x256x64)
    S, dk, nb = 256, 64, 512
    Q, K, A_ = dev(S * dk * nb), dev(S * dk * nb), dev(S * S * nb, 0)
    r.run("gemm", "jzhip_gemm_strided_batched QK^T", f"{S}x{S}x{dk} x{nb}",
          lambda: jz.gemm_strided_batched(P(Q), P(K), P(A_), S, S, dk, 1, 0, dk, dk, S, dk * S, dk * S, S * S, nb, 1.0, 0.0),
          flops=2.0 * S * S * dk * nb)
    r.run("gemm", "jzhip_gemm_strided_batched AV", f"{dk}x{S}x{S} x{nb}",
          lambda: jz.gemm_strided_batched(P(Q), P(A_), P(K), dk, S, S, 0, 0, dk, S, dk, dk * S, S * S, dk * S, nb, 1.0, 0.0),
          flops=2.0 * S * S * dk * nb)


def bench_ew(r):
    jz = r.jz
    for lg in (20, 22, 24, 26, 28):
        n = 1 << lg
        a, b, o = dev(n), dev(n), dev(n, 0)
        a.abs_().add_(0.5)
        tag = f"2^{lg}"
        for name, fn, bpe in [
            ("jzhip_copy", lambda: jz.copy(P(o), P(a), n), 8), ("jzhip_fill", lambda: jz.fill(P(o), n, 1.0), 4),
            ("jzhip_exp", lambda: jz.exp(P(o), P(a), n), 8), ("jzhip_log", lambda: jz.log(P(o), P(a), n), 8),
            ("jzhip_tanh", lambda: jz.tanh(P(o), P(a), n), 8), ("jzhip_affine", lambda: jz.affine(P(o), P(a), n, 0.2, 1.0), 8),
            ("jzhip_eleminv", lambda: jz.eleminv(P(o), P(a), n, 1.0), 8),
            ("jzhip_axpby", lambda: jz.axpby(P(o), P(a), P(b), n, 1.0, 2.0), 12),
            ("jzhip_hadamard", lambda: jz.hadamard(P(o), P(a), P(b), n), 12),
            ("jzhip_gelu", lambda: jz.gelu(P(o), P(a), n), 8),
        ]:
            r.run("elementwise", name, tag, fn, bytes_=bpe * n)
    # logical-transpose forms (one operand stored transposed): C1 size and a large one
    for rows, cols in ((1024, 1024), (8192, 8192)):
        n = rows * cols
        a, b, o = dev(n), dev(n), dev(n, 0)
        r.run("elementwise", "jzhip_axpby2d (B transposed)", f"{rows}x{cols}",
              lambda: jz.axpby2d(P(o), rows, 0, P(a), rows, 0, P(b), cols, 1, rows, cols, 1.0, 1.0), bytes_=12 * n)
        r.run("elementwise", "jzhip_copy2d (transpose)", f"{rows}x{cols}",
              lambda: jz.copy2d(P(o), rows, 0, 0, 0, P(a), cols, 1, 0, 0, rows, cols), bytes_=8 * n)


def bench_reduce(r):
    jz = r.jz
    for rows, cols in ((1024, 1024), (256, 4096), (512, 16384), (2048, 16384), (64, 25088), (16384, 16384)):
        a, o = dev(rows * cols), dev(max(rows, cols) * 2, 0)
        s = f"{rows}x{cols}"
        r.run("reduce", "jzhip_sum_cols", s, lambda: jz.sum_cols(P(o), P(a), rows, cols, rows), bytes_=4 * (rows * cols + cols))
        r.run("reduce", "jzhip_sum_rows", s, lambda: jz.sum_rows(P(o), P(a), rows, cols, rows), bytes_=4 * (rows * cols + rows))
        r.run("reduce", "jzhip_max_cols", s, lambda: jz.max_cols(P(o), P(a), rows, cols, rows), bytes_=4 * (rows * cols + cols))
        r.run("reduce", "jzhip_nrm2", s, lambda: jz.nrm2(P(o), P(a), rows * cols), bytes_=4 * rows * cols)
        r.run("reduce", "jzhip_softmax_cols", s, lambda: jz.softmax_cols(P(a), P(a), rows, cols, rows), bytes_=8 * rows * cols)
        r.run("reduce", "jzhip_softmax_rows", s, lambda: jz.softmax_rows(P(a), P(a), rows, cols, rows), bytes_=8 * rows * cols)
    # row softmax on rows of at most 2048 columns (whole rows in registers, one read)
    for rows, cols in ((131072, 256), (16384, 512), (16384, 2048), (65536, 2048)):
        a = dev(rows * cols)
        r.run("reduce", "jzhip_softmax_rows (single read)", f"{rows}x{cols}",
              lambda: jz.softmax_rows(P(a), P(a), rows, cols, rows), bytes_=8 * rows * cols)
        del a
    a, o = dev(10 * 16384), dev(10 * 16384, 0)
    r.run("reduce", "jzhip_predict_one_hot", "10x16384", lambda: jz.predict_one_hot(P(o), P(a), 10, 16384, 10), bytes_=8 * 10 * 16384)
    a, o = dev(1024 * 16384), dev(1024 * 16384, 0)
    r.run("reduce", "jzhip_predict_one_hot", "1024x16384", lambda: jz.predict_one_hot(P(o), P(a), 1024, 16384, 1024),
          bytes_=8 * 1024 * 16384)
    del a, o
    # loss of C3 and C4: softmax cross-entropy over columns
    for k, nb in ((10, 128), (256, 16384)):
        z, g, loss = dev(k * nb), dev(k * nb, 0), dev(1, 0)
        lab = torch.randint(0, k, (nb,), device="cuda", dtype=torch.int32)
        r.run("reduce", "jzhip_softmax_xent", f"{k}x{nb}", lambda: jz.softmax_xent(P(loss), P(g), P(z), P(lab), k, nb, k),
              bytes_=8 * k * nb + 4 * nb)
        y = dev(k * nb, 0)
        r.run("reduce", "jzhip_softmax_xent_dense (value)", f"{k}x{nb}",
              lambda: jz.softmax_xent_dense(P(loss), None, P(z), P(y), k, nb, k, 1.0 / nb), bytes_=8 * k * nb)
        r.run("reduce", "jzhip_softmax_xent_dense (gradient)", f"{k}x{nb}",
              lambda: jz.softmax_xent_dense(None, P(g), P(z), P(y), k, nb, k, 1.0 / nb), bytes_=12 * k * nb)
    for n in (4096, 1 << 26):
        a, b, g, loss = dev(n), dev(n), dev(n, 0), dev(1, 0)
        r.run("reduce", "jzhip_mse_loss", f"{n}", lambda: jz.mse_loss(P(loss), P(a), P(b), n, 1.0 / 128), bytes_=8 * n)
        r.run("reduce", "jzhip_mse_grad", f"{n}", lambda: jz.mse_grad(P(g), P(a), P(b), n, 1.0 / 128), bytes_=12 * n)


def bench_fused(r):
    jz = r.jz
    for dim, N in ((512, 16384), (512, 262144)):
        x, y, xh = dev(dim * N), dev(dim * N, 0), dev(dim * N, 0)
        inv, g, b, dg, db = dev(N, 1), dev(dim, 1), dev(dim, 0), dev(dim, 0), dev(dim, 0)
        s = f"{dim}x{N}"
        r.run("fused", "jzhip_layernorm_fwd", s, lambda: jz.layernorm_fwd(P(y), P(xh), P(inv), P(x), P(g), P(b), dim, N),
              bytes_=4 * (3 * dim * N + N + 2 * dim))
        r.run("fused", "jzhip_layernorm_bwd", s, lambda: jz.layernorm_bwd(P(y), P(x), P(g), P(xh), P(inv), dim, N),
              bytes_=4 * (3 * dim * N + N + dim))
        r.run("fused", "jzhip_layernorm_param_grads", s, lambda: jz.layernorm_param_grads(P(dg), P(db), P(x), P(xh), dim, N),
              bytes_=4 * (2 * dim * N + 2 * dim))
        # the backward sweep with the parameter gradients and two row sums on the side: dy, xhat, res in, dx out
        res, sx, sr = dev(dim * N), dev(dim, 0), dev(dim, 0)
        r.run("fused", "jzhip_layernorm_bwd_residual_sums", s,
              lambda: jz.layernorm_bwd_residual_sums(P(y), P(x), P(g), P(xh), P(inv), P(res), P(dg), P(db), P(sx), P(sr), dim, N),
              bytes_=4 * (4 * dim * N + N + 5 * dim))
        r.run("fused", "the same as separate launches (bwd_residual, param_grads, 2 x sum_rows)", s,
              lambda: (jz.layernorm_bwd_residual(P(y), P(x), P(g), P(xh), P(inv), P(res), dim, N),
                       jz.layernorm_param_grads(P(dg), P(db), P(x), P(xh), dim, N),
                       jz.sum_rows(P(sx), P(y), dim, N, dim), jz.sum_rows(P(sr), P(res), dim, N, dim)),
              bytes_=4 * (4 * dim * N + N + 5 * dim))
        del res, sx, sr
    for n in (1 << 20, 19_000_000, 1 << 27):
        w, g, m, v = dev(n), dev(n), dev(n, 0), dev(n, 0)
        r.run("fused", "jzhip_adam_update", f"{n}", lambda: jz.adam_update(P(g), P(m), P(v), n, 1e-3, 0.9, 0.999, 1e-8, 3), bytes_=24 * n)
        r.run("fused", "jzhip_adamw_step", f"{n}", lambda: jz.adamw_step(P(w), P(g), P(m), P(v), n, 1e-3, 0.9, 0.999, 1e-8, 0.01, 3),
              bytes_=28 * n)
    S, nblk = 256, 512
    a, o, da = dev(S * S * nblk), dev(S * S * nblk, 0), dev(S * S * nblk)
    for kar in (0, 1):
        s = f"{S}x{S} x{nblk} keys_along_rows={kar}"
        r.run("fused", "jzhip_attn_softmax (causal)", s, lambda: jz.attn_softmax(P(o), P(a), S, nblk, 0.125, 1, kar), bytes_=8 * a.numel())
        r.run("fused", "jzhip_attn_softmax_bwd", s, lambda: jz.attn_softmax_bwd(P(da), P(o), P(da), S, nblk, 0.125, kar), bytes_=12 * a.numel())
    # attention core of C4 (QK^T, mask+softmax, AV and their backward)
    dk, heads, B = 512, 8, 64
    N = S * B
    Q, K, V, H = (dev(dk * heads * N) for _ in range(4))
    A = dev(S * S * heads * B, 0)
    dQ, dK, dV, dA = dev(dk * heads * N, 0), dev(dk * heads * N, 0), dev(dk * heads * N, 0), dev(S * S * heads * B, 0)
    fl = 4.0 * S * S * dk * B
    r.run("fused", "jzhip_attention_fwd", f"S{S} d_k{dk} h{heads} B{B}",
          lambda: jz.attention_fwd(P(H), P(A), P(Q), P(K), P(V), dk, heads, S, B, 1), flops=fl)
    r.run("fused", "jzhip_attention_bwd", f"S{S} d_k{dk} h{heads} B{B}",
          lambda: jz.attention_bwd(P(dQ), P(dK), P(dV), P(dA), P(H), P(Q), P(K), P(V), P(A), dk, heads, S, B), flops=2 * fl)
    # the same core without the score matrices: forward keeps (max, 1/sum) per query, backward recomputes
    stats = dev(2 * S * heads * B, 0)
    dH = dev(dk * heads * N)
    for causal in (1, 0):
        tag = f"S{S} d_k{dk} h{heads} B{B} causal={causal}"
        r.run("fused", "jzhip_attention_flash_fwd", tag,
              lambda: jz.attention_flash_fwd(P(H), dk, P(stats), P(Q), P(K), P(V), dk, dk, heads, S, B, causal),
              flops=fl)
        r.run("fused", "jzhip_attention_flash_bwd", tag,
              lambda: jz.attention_flash_bwd(P(dQ), P(dK), P(dV), dk, P(dH), dk, P(Q), P(K), P(V), dk, P(H), dk, P(stats),
                                             dk, heads, S, B, causal), flops=2 * fl)
    # token embedding and one-hot construction of C4 (vocab 256, d_model 512, 16384 tokens)
    import torch
    Vc, dm = 256, 512
    tok = torch.randint(0, Vc, (N,), dtype=torch.int32, device="cuda")
    E, Pt, x0, oh = dev(dm * Vc), dev(dm * S), dev(dm * N, 0), dev(Vc * N, 0)
    r.run("fused", "jzhip_embedding_fwd", f"{dm}x{N} vocab {Vc}",
          lambda: jz.embedding_fwd(P(x0), P(E), P(Pt), None, P(tok), dm, Vc, S, N), bytes_=4.0 * (dm * N + N))
    r.run("fused", "jzhip_one_hot", f"{Vc}x{N}", lambda: jz.one_hot(P(oh), P(tok), Vc, N), bytes_=4.0 * (Vc * N + N))


def bench_conv(r):
    jz = r.jz
    for label, N, Cc, H, W, k, pad, s in (("C3 conv1", 128, 1, 28, 28, 3, 1, 1), ("C3 conv2", 128, 32, 28, 28, 3, 1, 2),
                                          ("C5 enc", 128, 64, 32, 32, 3, 1, 2), ("C5 dec1", 128, 128, 32, 32, 3, 1, 1)):
        Ho = (H + 2 * pad - k) // s + 1
        K, Pp = Cc * k * k, Ho * Ho
        x, col = dev(Cc * H * W * N), dev(K * Pp * N, 0)
        args = (Cc, H, W, k, k, pad, pad, s, s, Ho, Ho, N)
        byt = 4 * (x.numel() + col.numel())
        shape = f"{label} N{N} C{Cc} {H}x{W} k{k} s{s}"
        r.run("conv", "jzhip_im2col", shape, lambda: jz.im2col(P(x), P(col), *args), bytes_=byt)
        r.run("conv", "jzhip_col2im", shape, lambda: jz.col2im(P(col), P(x), *args), bytes_=byt)
        Co = 64
        y2d, out, bias = dev(Co * Pp * N), dev(Co * Pp * N, 0), dev(Co, 0)
        r.run("conv", "jzhip_conv_forward_reshape_bias", f"{label} C_out{Co} P{Pp} N{N}",
              lambda: jz.conv_forward_reshape_bias(P(y2d), P(out), P(bias), Co, Pp, N), bytes_=8 * y2d.numel())
        r.run("conv", "jzhip_conv_backward_reshape", f"{label} C_out{Co} P{Pp} N{N}",
              lambda: jz.conv_backward_reshape(P(out), P(y2d), Co, Pp, N), bytes_=8 * y2d.numel())


def bench_broadcast(r):
    """Bandwidth-bound members of the product family (rank-1 products and bias
    broadcasts, matrix-vector products) and the copy kernels behind slices and stacks."""
    jz = r.jz
    for m, n in ((256, 4096), (512, 16384), (2048, 16384), (16384, 16384)):
        a, b, c = dev(m), dev(n), dev(m * n, 0)
        s = f"{m}x{n}"
        # bias * ones(1, n): the layers' broadcast idiom (ml/layer.hpp:79,120,2797)
        r.run("broadcast", "jzhip_gemm k=1 (rank-1)", s, lambda: jz.gemm(P(a), P(b), P(c), m, n, 1, 0, 0, m, 1, m, 1.0, 0.0),
              bytes_=4.0 * (m * n + m + n))
        r.run("broadcast", "jzhip_add_bias", s, lambda: jz.add_bias(P(c), P(a), m, n), bytes_=8.0 * m * n + 4.0 * m)
    for m, n in ((4096, 4096), (16384, 16384), (256, 1 << 20)):
        A, x, y = dev(m * n), dev(max(m, n)), dev(max(m, n), 0)
        s = f"{m}x{n}"
        r.run("broadcast", "jzhip_gemv N", s, lambda: jz.gemv(P(A), P(x), P(y), m, n, 0, m, 1, 1, 1.0, 0.0),
              bytes_=4.0 * (m * n + m + n))
        r.run("broadcast", "jzhip_gemv T", s, lambda: jz.gemv(P(A), P(x), P(y), m, n, 1, m, 1, 1, 1.0, 0.0),
              bytes_=4.0 * (m * n + m + n))
    # slices and stacks: UNet skip concat / split (131072 + 65536 rows x 128 columns) and an attention-sized block
    for rows, cols in ((131072, 128), (8192, 8192)):
        src, dst = dev(rows * cols), dev(2 * rows * cols, 0)
        s = f"{rows}x{cols}"
        half = rows // 2
        r.run("broadcast", "jzhip_slice_extract (rows)", s,
              lambda: jz.slice_extract(P(dst), half, P(src), rows, 0, rows // 4, 0, half, cols), bytes_=8.0 * half * cols)
        r.run("broadcast", "jzhip_slice_extract (transposed source)", s,
              lambda: jz.slice_extract(P(dst), cols, P(src), rows, 1, 0, rows // 4, cols, half), bytes_=8.0 * half * cols)
        r.run("broadcast", "jzhip_slice_assign", s,
              lambda: jz.slice_assign(P(dst), rows, 0, rows // 4, 0, P(src), half, 0, half, cols), bytes_=8.0 * half * cols)
        r.run("broadcast", "jzhip_stack_copy_rows (vstack)", s,
              lambda: jz.stack_copy_rows(P(dst), 2 * rows, rows, P(src), rows, cols, 0), bytes_=8.0 * rows * cols)
        r.run("broadcast", "jzhip_stack_copy_cols (hstack)", s,
              lambda: jz.stack_copy_cols(P(dst), rows, cols, P(src), rows, cols, 0), bytes_=8.0 * rows * cols)
    a = dev(512 * 16384)
    o = dev(512, 0)
    r.run("broadcast", "jzhip_sum_rows_noalloc", "512x16384", lambda: jz.sum_rows_noalloc(P(o), P(a), 512, 16384, 512),
          bytes_=4.0 * (512 * 16384 + 512))
    x, xh, inv, g, out = dev(512 * 16384), dev(512 * 16384), dev(16384, 1), dev(512, 1), dev(512 * 16384, 0)
    r.run("broadcast", "jzhip_layernorm_jvp", "512x16384", lambda: jz.layernorm_jvp(P(out), P(x), P(g), P(xh), P(inv), 512, 16384),
          bytes_=4.0 * (3 * 512 * 16384 + 16384 + 512))
    from juzhen_amd.capi import AdamTensor
    sizes = [512 * 512] * 4 + [2048 * 512] * 2 + [512, 2048, 512]      # one transformer block
    bufs = [(dev(n), dev(n), dev(n, 0), dev(n, 0)) for n in sizes]
    arr = (AdamTensor * len(sizes))()
    for i, (n, (w, gr, m, v)) in enumerate(zip(sizes, bufs)):
        arr[i] = AdamTensor(w.data_ptr(), gr.data_ptr(), m.data_ptr(), v.data_ptr(), n, 1e-3, 0.9, 0.999, 1e-8, 0.0, 3)
    r.run("broadcast", "jzhip_adamw_step_multi", "9 tensors of one transformer block (3.15 M parameters)",
          lambda: jz.adamw_step_multi(arr, len(sizes)), bytes_=28.0 * sum(sizes))


def bench_conv_implicit(r):
    """The three products of a convolution layer without the patch matrix against the
    patch-matrix route (im2col, product, reshape / col2im), per layer of the CNN and UNet
    configurations.  flops = 2*K*C_out*P*N for each product."""
    jz = r.jz
    layers = (("C3 conv1", 128, 1, 28, 32, 1), ("C3 conv2", 128, 32, 28, 64, 2), ("C5 in", 128, 3, 32, 64, 1),
              ("C5 e1b", 128, 64, 32, 64, 1), ("C5 e2a", 128, 64, 32, 128, 2), ("C5 e2b", 128, 128, 16, 128, 1),
              ("C5 mid", 128, 256, 8, 256, 1), ("C5 d2a", 128, 256, 16, 128, 1), ("C5 d1a", 128, 128, 32, 64, 1))
    for label, N, Ci, H, Co, s in layers:
        k, pad = 3, 1
        Ho = (H + 2 * pad - k) // s + 1
        K, Pp = Ci * k * k, Ho * Ho
        x, w, b, t = dev(N * Ci * H * H), dev(K * Co), dev(Co), dev(Co * Pp * N)
        col, y2d, out, dW, dx = dev(K * Pp * N, 0), dev(Co * Pp * N, 0), dev(Co * Pp * N, 0), dev(K * Co, 0), dev(N * Ci * H * H, 0)
        dims = (Ci, H, H, Co, k, k, pad, pad, s, s, Ho, Ho, N)
        cargs = (Ci, H, H, k, k, pad, pad, s, s, Ho, Ho, N)
        fl = 2.0 * K * Co * Pp * N
        shape = f"{label} N{N} {Ci}>{Co} {H}x{H} s{s}"

        def fwd_patch():
            jz.im2col(P(x), P(col), *cargs)
            jz.gemm(P(w), P(col), P(y2d), Co, Pp * N, K, 1, 0, K, K, Co, 1.0, 0.0)
            jz.conv_forward_reshape_bias(P(y2d), P(out), P(b), Co, Pp, N)
            jz.relu(P(out), P(out), Co * Pp * N)

        def dw_patch():
            jz.conv_backward_reshape(P(t), P(y2d), Co, Pp, N)
            jz.im2col(P(x), P(col), *cargs)
            jz.gemm(P(col), P(y2d), P(dW), K, Co, Pp * N, 0, 1, K, Co, K, 1.0, 0.0)

        def dx_patch():
            jz.gemm(P(w), P(y2d), P(col), K, Pp * N, Co, 0, 0, K, Co, K, 1.0, 0.0)
            jz.col2im(P(col), P(dx), *cargs)

        r.run("conv", "forward, patch-matrix route (4 launches)", shape, fwd_patch, flops=fl)
        # with at most four input channels the products are bound by the output (forward) or the upstream
        # gradient (weight gradients) passing through memory once: those rows are priced in bytes
        few = Ci <= 4 and s == 1
        io = 4.0 * (N * Ci * H * H + Co * Pp * N)
        price = dict(bytes_=io) if few else dict(flops=fl)
        r.run("conv", "jzhip_conv2d_forward", shape, lambda: jz.conv2d_forward(P(x), P(w), P(b), P(out), *dims, 1), **price)
        r.run("conv", "weight gradients, patch-matrix route (3 launches)", shape, dw_patch, flops=fl)
        r.run("conv", "jzhip_conv2d_backward_weights", shape, lambda: jz.conv2d_backward_weights(P(x), P(t), P(dW), *dims), **price)
        r.run("conv", "input gradients, patch-matrix route (2 launches)", shape, dx_patch, flops=fl)
        if s == 1:
            r.run("conv", "jzhip_conv2d_backward_data", shape, lambda: jz.conv2d_backward_data(P(t), P(w), P(dx), *dims), flops=fl)
        else:
            r.run("conv", "jzhip_conv2d_transposed (input gradients of the strided layer)", shape,
                  lambda: jz.conv2d_transposed(P(t), P(w), None, P(dx), Co, Ho, Ho, Ci, k, k, pad, pad, s, s, H, H, N, 0), flops=fl)
        del x, w, b, t, col, y2d, out, dW, dx
        torch.cuda.empty_cache()
    # the UNet's up-sampling layers: 4x4, stride 2, pad 1
    for label, N, Ci, H, Co in (("C5 up2", 128, 256, 8, 128), ("C5 up1", 128, 128, 16, 64)):
        k, pad, s = 4, 1, 2
        Ho = (H - 1) * s - 2 * pad + k
        R, Pin = Co * k * k, H * H
        x, w, b = dev(N * Ci * Pin), dev(R * Ci), dev(Co)
        x2d, patches, out = dev(N * Ci * Pin, 0), dev(R * Pin * N, 0), dev(Co * Ho * Ho * N, 0)
        fl = 2.0 * N * Pin * Ci * R
        shape = f"{label} N{N} {Ci}>{Co} {H}x{H}>{Ho}x{Ho} k4 s2"

        def up_patch():
            jz.convtrans_reshape(P(x), P(x2d), Ci, Pin, N, 0)
            jz.gemm(P(w), P(x2d), P(patches), R, Pin * N, Ci, 0, 0, R, Ci, R, 1.0, 0.0)
            jz.convtrans_scatter(P(patches), P(out), P(b), Co, Ho, Ho, H, H, k, k, pad, pad, s, s, N)
            jz.relu(P(out), P(out), Co * Ho * Ho * N)

        r.run("conv", "transposed forward, patch-matrix route (4 launches)", shape, up_patch, flops=fl)
        r.run("conv", "jzhip_conv2d_transposed", shape,
              lambda: jz.conv2d_transposed(P(x), P(w), P(b), P(out), Ci, H, H, Co, k, k, pad, pad, s, s, Ho, Ho, N, 1), flops=fl)
        del x, w, b, x2d, patches, out
        torch.cuda.empty_cache()


GROUPS = {"gemm": bench_gemm, "ew": bench_ew, "reduce": bench_reduce, "fused": bench_fused, "conv": bench_conv,
          "broadcast": bench_broadcast, "conv_implicit": bench_conv_implicit}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--groups", default=",".join(GROUPS))
    ap.add_argument("--out", default=None)
    args = ap.parse_args()
    if not torch.cuda.is_available():
        sys.exit("opbench needs a GPU")
    r = Report()
    for g in args.groups.split(","):
        GROUPS[g](r)
        torch.cuda.empty_cache()
    text = r.markdown()
    if args.out:
        Path(args.out).write_text(text)
    else:
        print(text)


if __name__ == "__main__":
    main()
