"""Parity oracle loader — TEST INFRASTRUCTURE ONLY.

Only tests/, the smoke check and the benchmark's cpu_baseline leg may import
this package.  It builds and binds

* ``liboracle.so``  — oracle/jz_oracle.c, the C restatement of the reference's
  CPU ``Matrix<float>`` path, and
* ``_ref/libjzref.so`` — the reference's own CPU path compiled from
  /root/reference through oracle/ref_shim.cpp (only where that tree exists;
  the built library travels with the working tree).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB = HERE / "liboracle.so"
REF_DIR = HERE / "_ref"
REF_LIB = REF_DIR / "libjzref.so"
REFERENCE_ROOT = Path(os.environ.get("JUZHEN_REFERENCE", "/root/reference"))

P, Z, I, F, D = C.c_void_p, C.c_size_t, C.c_int, C.c_float, C.c_double

SIGNATURES = {
    "jzo_gemm": (None, [I, I, I, I, I, F, P, I, P, I, F, P, I]),
    "jzo_gemv": (None, [I, I, I, F, P, I, P, I, F, P, I]),
    "jzo_dot": (None, [P, P, I, I, P, I, I, I, I, I]),
    "jzo_axpby2d": (None, [P, I, I, P, I, I, P, I, I, I, I, F, F]),
    "jzo_hadamard2d": (None, [P, I, I, P, I, I, P, I, I, I, I]),
    "jzo_copy2d": (None, [P, I, I, Z, Z, P, I, I, Z, Z, Z, Z]),
    "jzo_affine": (None, [P, P, Z, F, F]),
    "jzo_eleminv": (None, [P, P, Z, D]),
    "jzo_exp": (None, [P, P, Z]),
    "jzo_log": (None, [P, P, Z]),
    "jzo_tanh": (None, [P, P, Z]),
    "jzo_dtanh": (None, [P, P, Z]),
    "jzo_square": (None, [P, P, Z]),
    "jzo_relu": (None, [P, P, Z]),
    "jzo_drelu": (None, [P, P, Z]),
    "jzo_sqrt": (None, [P, P, Z]),
    "jzo_clamp": (None, [P, P, Z, F, F]),
    "jzo_drelu_mul": (None, [P, P, P, Z]),
    "jzo_gelu": (None, [P, P, Z]),
    "jzo_dgelu_mul": (None, [P, P, P, Z]),
    "jzo_embedding_fwd": (None, [P, P, P, P, P, I, I, I, I]),
    "jzo_one_hot": (None, [P, P, I, Z]),
    "jzo_sum_phys": (None, [P, P, I, I, I, I]),
    "jzo_norm": (F, [P, Z]),
    "jzo_max_cols": (None, [P, P, I, I, I]),
    "jzo_argmax_cols": (None, [P, P, I, I, I]),
    "jzo_softmax_cols": (None, [P, P, I, I, I]),
    "jzo_softmax_rows": (None, [P, P, I, I, I]),
    "jzo_attn_softmax": (None, [P, P, I, I, F, I, I]),
    "jzo_attn_softmax_bwd": (None, [P, P, P, I, I, F, I]),
    "jzo_softmax_xent": (F, [P, P, P, I, I, I]),
    "jzo_layernorm_fwd": (None, [P, P, P, P, P, P, I, I]),
    "jzo_layernorm_bwd": (None, [P, P, P, P, P, I, I]),
    "jzo_layernorm_jvp": (None, [P, P, P, P, P, I, I]),
    "jzo_layernorm_param_grads": (None, [P, P, P, P, I, I]),
    "jzo_adam_update": (None, [P, P, P, Z, F, F, F, F, I]),
    "jzo_adamw_step": (None, [P, P, P, P, Z, F, F, F, F, F, I]),
    "jzo_im2col": (None, [P, P] + [I] * 12),
    "jzo_col2im": (None, [P, P] + [I] * 12),
    "jzo_conv_forward_reshape_bias": (None, [P, P, P, I, I, I]),
    "jzo_conv_backward_reshape": (None, [P, P, I, I, I]),
    "jzo_convtrans_scatter": (None, [P, P, P] + [I] * 12),
    "jzo_convtrans_gather": (None, [P, P] + [I] * 12),
    "jzo_convtrans_reshape": (None, [P, P, I, I, I, I]),
}


def build(force: bool = False) -> Path:
    """Compile the C restatement with gcc (seconds)."""
    src = HERE / "jz_oracle.c"
    if force or not LIB.exists() or LIB.stat().st_mtime < src.stat().st_mtime:
        cmd = ["gcc", "-O2", "-ffp-contract=off", "-fPIC", "-shared", "-fvisibility=hidden",
               "-o", str(LIB), str(src), "-lm"]
        subprocess.run(cmd, check=True)
    return LIB


def build_ref(force: bool = False):
    """Compile the reference CPU path (oracle/_ref); None if the tree is absent."""
    if not REFERENCE_ROOT.exists():
        return REF_LIB if REF_LIB.exists() else None
    r = subprocess.run(["make", "-C", str(HERE), "-s", f"REF={REFERENCE_ROOT}"] + (["-B"] if force else []),
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("reference CPU path failed to build:\n" + r.stdout + r.stderr)
    return REF_LIB


_lib = None


def load() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        lib = C.CDLL(str(LIB))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def ptr(a: np.ndarray) -> C.c_void_p:
    assert a.flags["C_CONTIGUOUS"] or a.flags["F_CONTIGUOUS"], "oracle needs contiguous arrays"
    return C.c_void_p(a.ctypes.data)


def f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


PP = C.POINTER(C.c_void_p)
REF_SIGNATURES = {
    "jzref_init": (None, []),
    "jzref_dot": (None, [P, P, I, I, I, P, I, I, I]),
    "jzref_add": (I, [P, P, I, I, I, P, I, I, I, F, F]),
    "jzref_add_inplace": (None, [P, I, I, I, P, I, I, I, F, F]),
    "jzref_hadmd": (I, [P, P, I, I, I, P, I, I, I]),
    "jzref_unary": (I, [I, P, P, I, D, D]),
    "jzref_chain": (None, [P, P, I, I, P, I]),
    "jzref_sum": (None, [P, P, I, I, I, I]),
    "jzref_norm": (F, [P, I]),
    "jzref_slice": (None, [P, P, I, I, I, I, I, I, I]),
    "jzref_slice_assign": (None, [P, I, I, I, I, I, I, I, P, I, I, I]),
    "jzref_stack2": (None, [P, I, P, I, I, I, P, I, I, I]),
    "jzref_softmax": (None, [P, P, I, I, I, I]),
    "jzref_max_cols": (None, [P, P, I, I]),
    "jzref_adam_update": (None, [P, P, P, I, F, F, F, F, I]),
    "jzref_layernorm_fwd": (None, [P, P, P, P, P, P, I, I]),
    "jzref_layernorm_bwd": (None, [P, P, P, P, P, P, P, I, I]),
    "jzref_layernorm_jvp": (None, [P, P, P, P, P, I, I]),
    "jzref_logistic": (F, [P, P, P, I, I]),
    "jzref_conv_eval": (None, [P, P, P, P] + [I] * 10),
    "jzref_conv_backward": (None, [P, P, P, P, P] + [I] * 10),
    "jzref_convtrans_eval": (None, [P, P, P, P] + [I] * 10),
    "jzref_convtrans_backward": (None, [P, P, P, P, P] + [I] * 10),
    "jzref_block_create": (P, [I, I, I, I, I, I, I]),
    "jzref_block_destroy": (None, [P]),
    "jzref_block_param": (I, [P, I, P, I]),
    "jzref_block_set_lr": (None, [P, F]),
    "jzref_block_eval": (None, [P, P, P]),
    "jzref_block_backward": (None, [P, P, P, P, I]),
    "jzref_mlp_step": (F, [I, P, P, PP, PP, PP, PP, PP, PP, P, P, I, F, I]),
    "jzref_lm_create": (P, [I, I, I, I, I, I, I]),
    "jzref_lm_destroy": (None, [P]),
    "jzref_lm_param": (I, [P, I, I, I, P, I]),
    "jzref_lm_set_lr": (None, [P, F]),
    "jzref_lm_step": (F, [P, P, P]),
}

_ref = None


def load_ref():
    """The reference CPU path (oracle/_ref/libjzref.so), or None if it was never built."""
    global _ref
    if _ref is None:
        if not REF_LIB.exists():
            return None
        lib = C.CDLL(str(REF_LIB))
        for name, (res, args) in REF_SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        lib.jzref_init()
        _ref = lib
    return _ref


REF_LIB_OPENBLAS = REF_DIR / "libjzref_openblas.so"
_ref_blas = None


def load_ref_openblas(threads: int | None = None):
    """The same reference CPU path linked against OpenBLAS (the reference's default
    configuration, cpp/helper.hpp:190-250), for model-sized checks the BLAS-free
    build would take minutes over.  None if it was never built.  Returns
    (library, BLAS thread count)."""
    global _ref_blas
    if _ref_blas is None:
        if not REF_LIB_OPENBLAS.exists():
            return None
        lib = C.CDLL(str(REF_LIB_OPENBLAS))
        for name, (res, args) in REF_SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        lib.jzref_init()
        cores = 1
        for dep in sorted(Path("/usr/local/lib").glob("python3*/dist-packages/scipy.libs/libscipy_openblas*.so")):
            blas = C.CDLL(str(dep))
            want = threads or min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
            blas.scipy_openblas_set_num_threads(C.c_int(want))
            blas.scipy_openblas_get_num_threads.restype = C.c_int
            cores = int(blas.scipy_openblas_get_num_threads())
            break
        _ref_blas = (lib, cores)
    return _ref_blas
