"""Test infrastructure: drives the reference's own CPU transformer LM
(oracle/_ref, assembled as examples/demo_transformer.cu:285-340 does) beside a
model under test and reports the loss trajectory of both.  Only tests and the
smoke check use this; nothing in the product imports it."""
from __future__ import annotations

import ctypes as C

import numpy as np

BLOCK_PARAMS = ["Wq", "Wk", "Wv", "Wo", "bo", "W1", "b1", "W2", "b2", "ln1_gamma", "ln1_beta", "ln2_gamma",
                "ln2_beta"]


def _cm(a):
    """(rows, cols) array -> dense column-major float32 vector"""
    return np.ascontiguousarray(np.asarray(a, np.float32).T).reshape(-1)


def _hp(a):
    return C.c_void_p(a.ctypes.data)


def zipf_tokens(rng, vocab, batch, seq, s=1.1):
    p = 1.0 / np.arange(1, vocab + 1) ** s
    p /= p.sum()
    return rng.choice(vocab, size=(batch, seq + 1), p=p).astype(np.int32)


def track_reference_lm(ref, model, cfg, tokens, steps, lr):
    """Copy `model`'s parameters (ReLU FFN, Adam, untied head with biases) into a
    reference CPU model, run `steps` train steps on both with the same batch and
    return (reference losses, model losses, reference handle).  The caller
    destroys the handle with ref.jzref_lm_destroy."""
    V, d, heads, ff, L, S, B = cfg
    N = S * B
    h = ref.jzref_lm_create(V, d, heads, ff, L, S, B)
    keep = []

    def give(kind, layer, which, arr):
        buf = _cm(arr)
        keep.append(buf)
        assert ref.jzref_lm_param(h, kind, layer, which, _hp(buf), 1) == 0

    give(0, 0, 0, np.hstack([model.get("embed"), model.get("pos")]))
    give(1, 0, 0, model.get("embed_bias"))
    give(2, 0, 0, model.get("head"))
    give(3, 0, 0, model.get("head_bias"))
    for l in range(L):
        for w, name in enumerate(BLOCK_PARAMS):
            give(4, l, w, model.get(f"block{l}.{name}"))
    ref.jzref_lm_set_lr(h, lr)

    model.set_batch(tokens)
    X = np.zeros((V + S, N), np.float32)
    Y = np.zeros((V, N), np.float32)
    for b in range(B):
        for s in range(S):
            n = b * S + s
            X[tokens[b, s], n] = 1
            X[V + s, n] = 1
            Y[tokens[b, s + 1], n] = 1
    Xc, Yc = _cm(X), _cm(Y)
    want, got = [], []
    for _ in range(steps):
        want.append(float(ref.jzref_lm_step(h, _hp(Xc), _hp(Yc))))
        model.step()
        got.append(float(model.loss()))
    return np.array(want), np.array(got), h
