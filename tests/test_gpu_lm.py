"""Train-step parity of the transformer LM harness.

(a) In the reference's own configuration (ReLU FFN, Adam, untied head with
    biases) the harness must track a model assembled from the reference's own
    classes on the CPU (LinearLayer + TransformerLayer<float> + LogisticLayer,
    examples/demo_transformer.cu:285-340, through oracle/_ref) for 100 steps:
    relative loss error <= 1e-3.
(b) The pieces the reference does not contain (GELU, tied embeddings, AdamW)
    are not pinned by it; they are checked against an independent float64
    PyTorch autograd model on the CPU (closed-form definitions only).
"""
import ctypes as C

import numpy as np
import pytest

import oracle
from oracle.lm_check import track_reference_lm
from util import hptr, need_ref_binary

pytestmark = pytest.mark.gpu

BLOCK_PARAMS = ["Wq", "Wk", "Wv", "Wo", "bo", "W1", "b1", "W2", "b2", "ln1_gamma", "ln1_beta", "ln2_gamma",
                "ln2_beta"]


def make_tokens(rng, vocab, batch, seq):
    p = 1.0 / np.arange(1, vocab + 1) ** 1.1     # Zipf(s=1.1) over the vocabulary
    p /= p.sum()
    return rng.choice(vocab, size=(batch, seq + 1), p=p).astype(np.int32)


def cm(a):
    """(rows, cols) array -> dense column-major float32 vector"""
    return np.ascontiguousarray(np.asarray(a, np.float32).T).reshape(-1)


def test_reference_configuration_tracks_the_reference_cpu_model(gpu):
    ref = oracle.load_ref()
    if ref is None:
        need_ref_binary(oracle.REF_LIB)
    from juzhen_amd.lm import CharLM
    V, d, heads, ff, L, S, B = 13, 16, 4, 32, 2, 8, 3
    N = S * B
    lr = 2e-3
    rng = np.random.default_rng(0)
    m = CharLM(V, d, heads, ff, L, S, B, gelu=False, tied=False, adamw=False, lr=lr)
    m.init_random(1)
    m.set("embed_bias", rng.normal(0, 0.1, (d, 1)))
    m.set("head_bias", rng.normal(0, 0.1, (V, 1)))
    tokens = make_tokens(rng, V, B, S)
    want, got, h = track_reference_lm(ref, m, (V, d, heads, ff, L, S, B), tokens, 100, lr)
    worst = float(np.max(np.abs(got - want) / np.abs(want)))
    first, last = want[0], want[-1]
    print(f"reference-configuration LM: loss {first:.4f} -> {last:.4f}, worst rel err {worst:.2e}")
    assert last < first                      # it trains
    assert worst <= 1e-3
    # parameters after 100 steps
    buf = np.empty(d * d, np.float32)
    ref.jzref_lm_param(h, 4, L - 1, 0, hptr(buf), 0)
    got = cm(m.get(f"block{L - 1}.Wq"))
    assert np.linalg.norm(got - buf) <= 1e-3 * np.linalg.norm(buf)
    ref.jzref_lm_destroy(h)
    m.close()


def test_full_size_reference_configuration_two_steps(gpu):
    """The benchmark's width, depth, context and batch (d 512, 8 heads, ff 2048,
    6 blocks, 256 x 64 tokens) in the reference's own configuration (ReLU FFN,
    Adam, untied head), two train steps beside the reference's CPU classes
    built against OpenBLAS (examples/demo_transformer.cu:285-340): losses within
    1e-3, two weight tensors within 1e-3, and the Adam updates themselves (what
    the step changed) in agreement."""
    got_ref = oracle.load_ref_openblas()
    if got_ref is None:
        need_ref_binary(oracle.REF_LIB_OPENBLAS)
    ref, cores = got_ref
    from juzhen_amd.lm import CharLM
    V, d, heads, ff, L, S, B = 256, 512, 8, 2048, 6, 256, 64
    lr = 3e-4
    rng = np.random.default_rng(21)
    m = CharLM(V, d, heads, ff, L, S, B, gelu=False, tied=False, adamw=False, lr=lr)
    m.init_random(6)
    m.set("embed_bias", rng.normal(0, 0.1, (d, 1)))
    m.set("head_bias", rng.normal(0, 0.1, (V, 1)))
    watch = ["block0.Wq", f"block{L - 1}.W2"]
    before = {n: m.get(n).copy() for n in watch}
    tokens = make_tokens(rng, V, B, S)
    want, got, h = track_reference_lm(ref, m, (V, d, heads, ff, L, S, B), tokens, 2, lr)
    worst = float(np.max(np.abs(got - want) / np.abs(want)))
    print(f"full-size reference-configuration LM ({cores} BLAS threads): reference losses {want}, ours {got}, "
          f"worst rel err {worst:.2e}")
    assert worst <= 1e-3
    for which, n in ((0, watch[0]), (7, watch[1])):
        r, c = m.shape(n)
        buf = np.empty(r * c, np.float32)
        layer = 0 if n.startswith("block0") else L - 1
        assert ref.jzref_lm_param(h, 4, layer, which, hptr(buf), 0) == 0
        ours = cm(m.get(n))
        assert np.linalg.norm(ours - buf) <= 1e-3 * np.linalg.norm(buf), n
        # what two Adam steps changed: first steps are close to lr*sign(g), so a
        # gradient of the wrong sign or scale shows here although the weights barely move
        upd_ref, upd_ours = buf - cm(before[n]), ours - cm(before[n])
        rel = np.linalg.norm(upd_ours - upd_ref) / np.linalg.norm(upd_ref)
        print(f"  {n}: update agreement {rel:.2e}")
        assert rel <= 5e-2, (n, rel)
    ref.jzref_lm_destroy(h)
    m.close()


def torch_twin(cfg, params, tokens, steps, lr, wd):
    """float64 autograd restatement: pre-LN blocks, exact-erf GELU, tied head, AdamW."""
    import torch
    V, d, heads, ff, L, S, B = cfg
    dh = d // heads
    P = {k: torch.tensor(v, dtype=torch.float64, requires_grad=True) for k, v in params.items()}
    opt_decay = [v for k, v in P.items() if v.shape[1] > 1]
    opt_plain = [v for k, v in P.items() if v.shape[1] == 1]
    opt = torch.optim.AdamW([{"params": opt_decay, "weight_decay": wd}, {"params": opt_plain, "weight_decay": 0.0}],
                            lr=lr, betas=(0.9, 0.999), eps=1e-8)
    tok = torch.tensor(tokens[:, :-1].reshape(-1), dtype=torch.long)
    tgt = torch.tensor(tokens[:, 1:].reshape(-1), dtype=torch.long)
    pos = torch.arange(S).repeat(B)
    mask = torch.triu(torch.ones(S, S, dtype=torch.bool), 1)          # [query, key] key > query
    losses = []
    first_grads = {}

    def ln(x, g, b):
        mu = x.mean(0, keepdim=True)
        var = ((x - mu) ** 2).mean(0, keepdim=True)
        return (x - mu) / torch.sqrt(var + 1e-5) * g + b

    for _ in range(steps):
        x = P["embed"][:, tok] + P["pos"][:, pos]                       # (d, N)
        for l in range(L):
            p = lambda n: P[f"block{l}.{n}"]
            x1 = ln(x, p("ln1_gamma"), p("ln1_beta"))
            # head hh owns rows [hh*dh, (hh+1)*dh), sequence b columns [b*S, (b+1)*S): all
            # (head, sequence) blocks at once as (heads, dh, B, S) views
            q, k, v = (t.reshape(heads, dh, B, S) for t in (p("Wq") @ x1, p("Wk") @ x1, p("Wv") @ x1))
            s = torch.einsum("hdbq,hdbk->hbqk", q, k) / np.sqrt(dh)
            a = torch.softmax(s.masked_fill(mask, -1e9), dim=3)
            H = torch.einsum("hdbk,hbqk->hdbq", v, a).reshape(d, B * S)
            R = x + p("Wo") @ H + p("bo")
            x2 = ln(R, p("ln2_gamma"), p("ln2_beta"))
            f1 = p("W1") @ x2 + p("b1")
            x = R + p("W2") @ torch.nn.functional.gelu(f1) + p("b2")
        logits = P["embed"].T @ x                                       # (V, N)
        loss = torch.nn.functional.cross_entropy(logits.T, tgt)
        losses.append(float(loss.detach()))
        opt.zero_grad()
        loss.backward()
        if not first_grads:
            first_grads.update({k: v.grad.detach().numpy().copy() for k, v in P.items()})
        opt.step()
    return losses, {k: v.detach().numpy() for k, v in P.items()}, first_grads


def test_gelu_tied_adamw_against_float64_autograd(gpu):
    from juzhen_amd.lm import CharLM
    V, d, heads, ff, L, S, B = 17, 32, 4, 64, 2, 12, 4
    lr, wd = 3e-3, 0.01
    rng = np.random.default_rng(5)
    m = CharLM(V, d, heads, ff, L, S, B, gelu=True, tied=True, adamw=True, lr=lr, weight_decay=wd)
    m.init_random(2)
    for n in m.names:                      # non-trivial biases / gains so every gradient path is live
        r, c = m.shape(n)
        if c == 1:
            m.set(n, m.get(n) + rng.normal(0, 0.05, (r, 1)).astype(np.float32))
    params = {n: m.get(n).astype(np.float64) for n in m.names}
    tokens = make_tokens(rng, V, B, S)
    m.set_batch(tokens)
    steps = 100
    want, final, _ = torch_twin((V, d, heads, ff, L, S, B), params, tokens, steps, lr, wd)
    worst = 0.0
    for i in range(steps):
        m.step()
        got = m.loss()
        worst = max(worst, abs(got - want[i]) / abs(want[i]))
    print(f"GELU/tied/AdamW LM: loss {want[0]:.4f} -> {want[-1]:.4f}, worst rel err {worst:.2e}")
    assert want[-1] < want[0]
    assert worst <= 1e-3                   # train-step losses after 100 steps
    for n in ("embed", "pos", "block0.W1", "block1.Wq", "block1.ln2_gamma", "block0.b1"):
        a, b = m.get(n), final[n]
        assert np.linalg.norm(a - b) <= 2e-3 * np.linalg.norm(b), n
    m.close()


def test_headline_variant_at_full_width_against_float64_autograd(gpu):
    """The benchmark's own variant (exact-erf GELU, tied embeddings, AdamW with the decay
    group) at the benchmark's width, depth, context and batch (d 512, 8 heads, ff 2048,
    6 blocks, 256 x 64 tokens) beside the float64 autograd statement of the same model:
    the loss and the gradients of the token table, the position table and one FFN weight
    before any update, then the losses of two optimiser steps, all within 1e-3."""
    import torch
    from juzhen_amd.lm import CharLM
    V, d, heads, ff, L, S, B = 256, 512, 8, 2048, 6, 256, 64
    lr, wd = 3e-4, 0.01
    rng = np.random.default_rng(31)
    m = CharLM(V, d, heads, ff, L, S, B, gelu=True, tied=True, adamw=True, lr=lr, weight_decay=wd)
    m.init_random(8)
    for n in m.names:                      # live biases and gains
        r, c = m.shape(n)
        if c == 1:
            m.set(n, m.get(n) + rng.normal(0, 0.05, (r, 1)).astype(np.float32))
    params = {n: m.get(n).astype(np.float64) for n in m.names}
    tokens = make_tokens(rng, V, B, S)
    m.set_batch(tokens)
    m.forward()
    m.backward(update=False)
    loss0 = m.loss()
    grads = {n: m.get(n, which=1) for n in ("embed", "pos", "block0.W1", f"block{L - 1}.Wq", "block2.ln1_gamma")}
    got = []
    for _ in range(2):
        m.step()
        got.append(m.loss())
    m.close()
    print("float64 twin of the full-size model: two steps on the CPU ...", flush=True)
    want, _, first = torch_twin((V, d, heads, ff, L, S, B), params, tokens, 2, lr, wd)
    print(f"headline variant, full size: float64 losses {want}, ours {[loss0] + got[1:]}")
    assert abs(loss0 - want[0]) <= 1e-3 * abs(want[0])
    assert abs(got[0] - want[0]) <= 1e-3 * abs(want[0])
    assert abs(got[1] - want[1]) <= 1e-3 * abs(want[1])
    for n, g in grads.items():
        rel = np.linalg.norm(g - first[n]) / np.linalg.norm(first[n])
        print(f"  gradient of {n}: rel err {rel:.2e}")
        assert rel <= 1e-3, (n, rel)


def test_full_size_properties_of_the_headline_variant(gpu):
    """Size-independent properties at the benchmark's full size: every parameter stays
    finite over 20 steps and the loss falls; the gradient of the tied token table is the
    sum of the head product's gradient and the lookup's gradient, which an untied model on
    the same weights (head = table transposed, zero biases) yields separately."""
    from juzhen_amd.lm import CharLM
    V, d, heads, ff, L, S, B = 256, 512, 8, 2048, 6, 256, 64
    rng = np.random.default_rng(77)
    tokens = make_tokens(rng, V, B, S)
    tied = CharLM(V, d, heads, ff, L, S, B, gelu=True, tied=True, adamw=True, lr=3e-4, weight_decay=0.01)
    tied.init_random(9)
    tied.set_batch(tokens)
    tied.forward()
    tied.backward(update=False)
    g_tied = tied.get("embed", which=1)
    untied = CharLM(V, d, heads, ff, L, S, B, gelu=True, tied=False, adamw=True, lr=3e-4, weight_decay=0.01)
    for n in untied.names:
        if n == "head":
            untied.set(n, tied.get("embed").T)
        elif n in ("embed_bias", "head_bias"):
            r, c = untied.shape(n)
            untied.set(n, np.zeros((r, c), np.float32))
        else:
            untied.set(n, tied.get(n))
    untied.set_batch(tokens)
    untied.forward()
    untied.backward(update=False)
    assert abs(untied.loss() - tied.loss()) <= 1e-6 * abs(tied.loss())
    parts = untied.get("embed", which=1).astype(np.float64) + untied.get("head", which=1).astype(np.float64).T
    rel = np.linalg.norm(g_tied - parts) / np.linalg.norm(parts)
    print(f"tied-table gradient against lookup part + head part: rel err {rel:.2e}")
    assert rel <= 1e-5
    untied.close()
    first = None
    for i in range(20):
        tied.step()
        if i == 0:
            first = tied.loss()
    last = tied.loss()
    assert np.isfinite(last) and last < first
    for n in tied.names:
        assert np.isfinite(tied.get(n)).all(), n
        assert np.isfinite(tied.get(n, which=1)).all(), n
    tied.close()


def test_zero_gradient_adamw_step_is_the_decay_alone(gpu):
    """With zero gradients and zero moments the update term is exactly 0, so a step of the
    fused AdamW leaves w * (1 - lr*wd), the factor formed in fp32 as the kernel forms it,
    bit for bit, on as many elements as the headline model has parameters; with wd = 0 the
    weights do not move at all."""
    import torch
    n = 19_000_000 + 3
    lr, wd = 3e-4, 0.01
    w0 = torch.randn(n, device="cuda")
    for decay in (wd, 0.0):
        w, g, mm, vv = w0.clone(), torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
        gpu.adamw_step(C.c_void_p(w.data_ptr()), C.c_void_p(g.data_ptr()), C.c_void_p(mm.data_ptr()),
                       C.c_void_p(vv.data_ptr()), n, lr, 0.9, 0.999, 1e-8, decay, 1)
        gpu.synchronize()
        factor = np.float32(1.0) - np.float32(lr) * np.float32(decay)
        want = w0.cpu().numpy() * factor if decay else w0.cpu().numpy()
        assert np.array_equal(w.cpu().numpy(), want)
        assert not mm.any() and not vv.any()


def test_attention_without_the_score_matrices_trains_like_the_materialising_path(gpu, monkeypatch):
    """The harness keeps two floats per query instead of the S x S probabilities whenever
    the shape allows it.  Same model, same batches, both ways (JZLM_MATERIALISE_ATTENTION=1
    selects the buffers of the reference's layout): the two runs differ only in the order of
    a few sums, so losses agree to 1e-5 over ten steps and gradients to 1e-5."""
    from juzhen_amd.lm import CharLM
    V, d, heads, ff, L, S, B = 64, 128, 4, 256, 3, 96, 5          # head width 32, six key tiles
    rng = np.random.default_rng(12)
    tokens = make_tokens(rng, V, B, S)
    runs = []
    for keep in ("1", "0"):
        monkeypatch.setenv("JZLM_MATERIALISE_ATTENTION", keep)
        m = CharLM(V, d, heads, ff, L, S, B, gelu=True, tied=True, adamw=True, lr=1e-3)
        assert m.flash_attention == (keep == "0")
        m.init_random(5)
        m.set_batch(tokens)
        m.forward()
        m.backward(update=False)
        grads = {n: m.get(n, which=1) for n in ("embed", "block0.Wq", "block2.Wv", "block1.ln1_gamma")}
        losses = []
        for _ in range(10):
            m.step()
            losses.append(m.loss())
        runs.append((losses, grads))
        m.close()
    (l0, g0), (l1, g1) = runs
    assert np.allclose(l0, l1, rtol=1e-5)
    for n in g0:
        assert np.linalg.norm(g0[n] - g1[n]) <= 1e-5 * np.linalg.norm(g0[n]), n
    # a shape the kernels do not cover (head width 8) keeps the probabilities
    monkeypatch.delenv("JZLM_MATERIALISE_ATTENTION")
    m = CharLM(17, 32, 4, 64, 1, 12, 2)
    assert not m.flash_attention
    m.close()


def test_gradients_against_float64_autograd(gpu):
    """One backward pass: every parameter gradient against autograd (no optimiser)."""
    from juzhen_amd.lm import CharLM
    V, d, heads, ff, L, S, B = 11, 16, 2, 48, 1, 9, 3
    rng = np.random.default_rng(7)
    m = CharLM(V, d, heads, ff, L, S, B, gelu=True, tied=True, adamw=True, lr=0.0, weight_decay=0.0)
    m.init_random(3)
    for n in m.names:
        r, c = m.shape(n)
        if c == 1:
            m.set(n, m.get(n) + rng.normal(0, 0.1, (r, 1)).astype(np.float32))
    params = {n: m.get(n).astype(np.float64) for n in m.names}
    tokens = make_tokens(rng, V, B, S)
    m.set_batch(tokens)
    m.forward()
    m.backward(update=False)
    losses, _, grads = torch_twin((V, d, heads, ff, L, S, B), params, tokens, 1, 0.0, 0.0)
    assert abs(m.loss() - losses[0]) <= 1e-4 * abs(losses[0])
    for name in m.names:
        got, want = m.get(name, which=1), grads[name]
        assert np.linalg.norm(got - want) <= 1e-3 * np.linalg.norm(want), name
    m.close()


@pytest.mark.parametrize("tied", [True, False])
def test_two_stream_backward_is_bit_identical_to_program_order(gpu, tied):
    """The backward pass issues weight, bias and LayerNorm-parameter gradients on a
    second stream; every kernel and every accumulation order is the same as on one
    stream, so losses, gradients and parameters must agree to the bit.  Four blocks
    exercise the alternating scratch sets and the wait on the block two above."""
    from juzhen_amd.lm import CharLM
    V, d, heads, ff, L, S, B = 64, 128, 4, 512, 4, 64, 8
    rng = np.random.default_rng(5)
    tokens = make_tokens(rng, V, B, S)
    runs = []
    for overlap in (False, True):
        m = CharLM(V, d, heads, ff, L, S, B, gelu=True, tied=tied, adamw=True, lr=1e-3, overlap=overlap)
        m.init_random(3)
        m.set_batch(tokens)
        losses = []
        for _ in range(6):
            m.step()
            losses.append(m.loss())
        m.forward()
        m.backward(update=False)
        grads = {n: m.get(n, which=1) for n in m.names}
        params = {n: m.get(n) for n in m.names}
        runs.append((losses, grads, params))
        m.close()
    (l0, g0, p0), (l1, g1, p1) = runs
    assert l0 == l1
    for n in g0:
        assert np.array_equal(g0[n], g1[n]), n
        assert np.array_equal(p0[n], p1[n]), n


def test_fresh_batch_every_step_without_waiting_for_the_step_in_flight(gpu):
    """Batches go through two page-locked staging buffers and asynchronous copies:
    handing over batch i+1 while step i is still running must not disturb step i,
    and a buffer is reused only after its copies have run.  Five different batches
    handed over back to back give the losses of the same five batches handed over
    with a full synchronisation before each."""
    from juzhen_amd.lm import CharLM
    V, d, heads, ff, L, S, B = 64, 128, 4, 512, 2, 64, 8
    rng = np.random.default_rng(9)
    batches = [make_tokens(rng, V, B, S) for _ in range(5)]
    out = []
    for drain in (True, False):
        m = CharLM(V, d, heads, ff, L, S, B, gelu=True, tied=True, adamw=True, lr=1e-3)
        m.init_random(4)
        losses = []
        for t in batches:
            if drain:
                gpu.synchronize()
            m.set_batch(t)
            m.step()
            if drain:
                losses.append(m.loss())
        params = {n: m.get(n) for n in m.names}
        out.append((losses, params, m.loss()))
        m.close()
    (l0, p0, last0), (_, p1, last1) = out
    assert last0 == last1 == l0[-1]
    for n in p0:
        assert np.array_equal(p0[n], p1[n]), n
    assert len(set(l0)) == len(l0)          # the batches really differ

