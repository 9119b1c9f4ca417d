"""ctypes binding of the train-step harness (juzhen_amd/harness/lm.cpp).

Host arrays are numpy (rows, cols) matrices; the library stores them
column-major, so they are transposed on the way in and out.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import numpy as np

from . import capi

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libjzlm.so"


class Config(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("vocab", "d_model", "heads", "d_ff", "layers", "seq", "batch",
                                         "gelu", "tied", "adamw")] + \
               [(n, C.c_float) for n in ("lr", "weight_decay", "beta1", "beta2", "eps")]


_lib = None


def load():
    global _lib
    if _lib is None:
        capi.load()
        if not LIB_PATH.exists():
            raise FileNotFoundError(f"{LIB_PATH} is missing: run `python -m juzhen_amd.build`")
        lib = C.CDLL(str(LIB_PATH))
        lib.jzlm_create.restype = C.c_void_p
        lib.jzlm_create.argtypes = [C.POINTER(Config)]
        lib.jzlm_destroy.argtypes = [C.c_void_p]
        for name in ("jzlm_status", "jzlm_num_tensors", "jzlm_forward", "jzlm_step", "jzlm_tokens_per_step"):
            getattr(lib, name).restype = C.c_int
            getattr(lib, name).argtypes = [C.c_void_p]
        lib.jzlm_backward.restype = C.c_int
        lib.jzlm_backward.argtypes = [C.c_void_p, C.c_int]
        lib.jzlm_param_count.restype = C.c_size_t
        lib.jzlm_param_count.argtypes = [C.c_void_p]
        lib.jzlm_tensor_name.restype = C.c_char_p
        lib.jzlm_tensor_name.argtypes = [C.c_void_p, C.c_int]
        for name in ("jzlm_tensor_rows", "jzlm_tensor_cols"):
            getattr(lib, name).restype = C.c_int
            getattr(lib, name).argtypes = [C.c_void_p, C.c_int]
        for name in ("jzlm_get", "jzlm_set"):
            getattr(lib, name).restype = C.c_int
            getattr(lib, name).argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p]
        lib.jzlm_set_batch.restype = C.c_int
        lib.jzlm_set_batch.argtypes = [C.c_void_p, C.c_void_p]
        lib.jzlm_loss.restype = C.c_float
        lib.jzlm_loss.argtypes = [C.c_void_p]
        lib.jzlm_logits.restype = C.c_int
        lib.jzlm_logits.argtypes = [C.c_void_p, C.c_void_p]
        lib.jzlm_set_iteration.argtypes = [C.c_void_p, C.c_int]
        lib.jzlm_set_overlap.argtypes = [C.c_void_p, C.c_int]
        lib.jzlm_set_overlap.restype = None
        lib.jzlm_flash_attention.restype = C.c_int
        lib.jzlm_flash_attention.argtypes = [C.c_void_p]
        _lib = lib
    return _lib


class CharLM:
    """Pre-LN decoder-only character LM trained with hand-written gfx950 kernels."""

    def __init__(self, vocab=256, d_model=512, heads=8, d_ff=2048, layers=6, seq=256, batch=64,
                 gelu=True, tied=True, adamw=True, lr=3e-4, weight_decay=0.01, beta1=0.9, beta2=0.999,
                 eps=1e-8, overlap=None):
        self.lib = load()
        self.cfg = Config(vocab, d_model, heads, d_ff, layers, seq, batch, int(gelu), int(tied), int(adamw),
                          lr, weight_decay, beta1, beta2, eps)
        self.h = self.lib.jzlm_create(C.byref(self.cfg))
        if not self.h:
            raise ValueError("invalid model configuration")
        self._check("create", self.lib.jzlm_status(self.h))
        self.names = [self.lib.jzlm_tensor_name(self.h, i).decode() for i in range(self.lib.jzlm_num_tensors(self.h))]
        self.index = {n: i for i, n in enumerate(self.names)}
        if overlap is not None:
            self.set_overlap(overlap)

    def set_overlap(self, on):
        """Weight-gradient work of the backward pass on a second stream, or everything
        on one stream in program order (the default)."""
        self.lib.jzlm_set_overlap(self.h, int(bool(on)))

    @property
    def flash_attention(self):
        """True when the attention core keeps two floats per query instead of the S x S
        probabilities (head width 32 or 64, context a multiple of 32 up to 256)."""
        return bool(self.lib.jzlm_flash_attention(self.h))

    def _check(self, what, rc):
        if rc != 0:
            raise capi.JzhipError("jzlm_" + what, rc, capi.load().jzhip_error_string(rc).decode())

    def close(self):
        if self.h:
            self.lib.jzlm_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def shape(self, name):
        i = self.index[name]
        return self.lib.jzlm_tensor_rows(self.h, i), self.lib.jzlm_tensor_cols(self.h, i)

    @property
    def param_count(self):
        return self.lib.jzlm_param_count(self.h)

    @property
    def tokens_per_step(self):
        return self.lib.jzlm_tokens_per_step(self.h)

    def set(self, name, value, which=0):
        r, c = self.shape(name)
        a = np.ascontiguousarray(np.asarray(value, dtype=np.float32).reshape(r, c).T)
        self._check("set", self.lib.jzlm_set(self.h, self.index[name], which, a.ctypes.data))

    def get(self, name, which=0):
        r, c = self.shape(name)
        a = np.empty((c, r), np.float32)
        self._check("get", self.lib.jzlm_get(self.h, self.index[name], which, a.ctypes.data))
        return a.T.copy()

    def init_random(self, seed=0):
        """N(0,1)/sqrt(fan_in) matrices, zero biases, unit LayerNorm gains (ml/layer.hpp:2822-2834)."""
        rng = np.random.default_rng(seed)
        for n in self.names:
            r, c = self.shape(n)
            if c == 1:
                v = np.ones((r, 1), np.float32) if n.endswith("gamma") else np.zeros((r, 1), np.float32)
            elif n in ("embed", "pos"):
                v = (rng.standard_normal((r, c)) * 0.02).astype(np.float32)
            else:
                v = (rng.standard_normal((r, c)) / np.sqrt(c)).astype(np.float32)
            self.set(n, v)

    def set_batch(self, tokens):
        t = np.ascontiguousarray(tokens, dtype=np.int32).reshape(self.cfg.batch, self.cfg.seq + 1)
        self._check("set_batch", self.lib.jzlm_set_batch(self.h, t.ctypes.data))

    def forward(self):
        self._check("forward", self.lib.jzlm_forward(self.h))

    def backward(self, update=False):
        self._check("backward", self.lib.jzlm_backward(self.h, int(update)))

    def step(self):
        self._check("step", self.lib.jzlm_step(self.h))

    def loss(self):
        return float(self.lib.jzlm_loss(self.h))

    def logits(self):
        a = np.empty((self.tokens_per_step, self.cfg.vocab), np.float32)
        self._check("logits", self.lib.jzlm_logits(self.h, a.ctypes.data))
        return a.T.copy()
