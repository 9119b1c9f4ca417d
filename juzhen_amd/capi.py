"""ctypes binding of the C ABI declared in include/jzhip.h.

Loading fails loudly: there is no CPU or PyTorch fallback behind these calls.
Device memory is passed as raw addresses (``tensor.data_ptr()`` of a torch
CUDA tensor, or any ``hipMalloc`` pointer).
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

_PKG = Path(__file__).resolve().parent
LIB_PATH = _PKG / "lib" / "libjzhip.so"

P = C.c_void_p          # float* / int32_t* device or host pointer
Z = C.c_size_t
I = C.c_int
F = C.c_float
D = C.c_double
U64 = C.c_uint64
LL = C.c_longlong

class AdamTensor(C.Structure):
    """struct jzhip_adam_tensor of include/jzhip.h"""
    _fields_ = [("w", C.c_void_p), ("g", C.c_void_p), ("m", C.c_void_p), ("v", C.c_void_p), ("count", C.c_size_t),
                ("alpha", C.c_float), ("beta1", C.c_float), ("beta2", C.c_float), ("eps", C.c_float),
                ("weight_decay", C.c_float), ("iteration", C.c_int)]


# name -> (restype, argtypes); mirrors include/jzhip.h one to one
SIGNATURES: dict[str, tuple] = {
    "jzhip_runtime_available": (I, []),
    "jzhip_version": (I, []),
    "jzhip_error_string": (C.c_char_p, [I]),
    "jzhip_num_compute_units": (I, []),
    "jzhip_malloc": (I, [C.POINTER(P), Z]),
    "jzhip_free": (I, [P]),
    "jzhip_memcpy_h2d": (I, [P, P, Z]),
    "jzhip_memcpy_d2h": (I, [P, P, Z]),
    "jzhip_memcpy_d2d": (I, [P, P, Z]),
    "jzhip_set_stream": (I, [P]),
    "jzhip_get_stream": (P, []),
    "jzhip_synchronize": (I, []),
    "jzhip_workspace_bytes": (Z, []),
    "jzhip_stream_create": (I, [P]),
    "jzhip_stream_destroy": (I, [P]),
    "jzhip_event_create": (I, [P]),
    "jzhip_event_destroy": (I, [P]),
    "jzhip_event_record": (I, [P]),
    "jzhip_stream_wait_event": (I, [P]),
    "jzhip_event_synchronize": (I, [P]),
    "jzhip_graph_begin": (I, []),
    "jzhip_graph_end": (I, [C.POINTER(P)]),
    "jzhip_graph_recording": (I, []),
    "jzhip_graph_launch": (I, [P]),
    "jzhip_graph_destroy": (I, [P]),
    "jzhip_host_alloc": (I, [P, Z]),
    "jzhip_host_free": (I, [P]),
    "jzhip_memcpy_h2d_async": (I, [P, P, Z]),
    "jzhip_memcpy_d2h_async": (I, [P, P, Z]),
    "jzhip_rand_uniform": (I, [P, Z, U64]),
    "jzhip_rand_normal": (I, [P, Z, F, F, U64]),
    "jzhip_fill": (I, [P, Z, F]),
    "jzhip_exp_inplace": (I, [P, Z]),
    "jzhip_log_inplace": (I, [P, Z]),
    "jzhip_exp": (I, [P, P, Z]),
    "jzhip_log": (I, [P, P, Z]),
    "jzhip_axpby": (I, [P, P, P, Z, F, F]),
    "jzhip_affine_inplace": (I, [P, Z, F, F]),
    "jzhip_affine": (I, [P, P, Z, F, F]),
    "jzhip_hadamard": (I, [P, P, P, Z]),
    "jzhip_hadamard_inplace": (I, [P, P, Z]),
    "jzhip_eleminv_inplace": (I, [P, Z, F]),
    "jzhip_eleminv": (I, [P, P, Z, D]),
    "jzhip_copy": (I, [P, P, Z]),
    "jzhip_square": (I, [P, P, Z]),
    "jzhip_square_inplace": (I, [P, Z]),
    "jzhip_tanh": (I, [P, P, Z]),
    "jzhip_tanh_inplace": (I, [P, Z]),
    "jzhip_dtanh": (I, [P, P, Z]),
    "jzhip_dtanh_inplace": (I, [P, Z]),
    "jzhip_relu": (I, [P, P, Z]),
    "jzhip_drelu": (I, [P, P, Z]),
    "jzhip_sqrt": (I, [P, P, Z]),
    "jzhip_clamp": (I, [P, P, Z, F, F]),
    "jzhip_drelu_mul": (I, [P, P, P, Z]),
    "jzhip_mse_loss": (I, [P, P, P, Z, F]),
    "jzhip_mse_grad": (I, [P, P, P, Z, F]),
    "jzhip_gelu": (I, [P, P, Z]),
    "jzhip_dgelu_mul": (I, [P, P, P, Z]),
    "jzhip_axpby2d": (I, [P, I, I, P, I, I, P, I, I, I, I, F, F]),
    "jzhip_hadamard2d": (I, [P, I, I, P, I, I, P, I, I, I, I]),
    "jzhip_copy2d": (I, [P, I, I, Z, Z, P, I, I, Z, Z, Z, Z]),
    "jzhip_stack_copy_cols": (I, [P, Z, Z, P, Z, Z, I]),
    "jzhip_stack_copy_rows": (I, [P, Z, Z, P, Z, Z, I]),
    "jzhip_slice_extract": (I, [P, Z, P, Z, I, Z, Z, Z, Z]),
    "jzhip_slice_assign": (I, [P, Z, I, Z, Z, P, Z, I, Z, Z]),
    "jzhip_sum_cols": (I, [P, P, I, I, I]),
    "jzhip_sum_rows": (I, [P, P, I, I, I]),
    "jzhip_sum_rows_noalloc": (I, [P, P, I, I, I]),
    "jzhip_embedding_fwd": (I, [P, P, P, P, P, I, I, I, I]),
    "jzhip_one_hot": (I, [P, P, I, Z]),
    "jzhip_nrm2": (I, [P, P, Z]),
    "jzhip_max_cols": (I, [P, P, I, I, I]),
    "jzhip_argmax_cols": (I, [P, P, I, I, I]),
    "jzhip_predict_one_hot": (I, [P, P, I, I, I]),
    "jzhip_gemm": (I, [P, P, P, I, I, I, I, I, I, I, I, F, F]),
    "jzhip_gemm_nn": (I, [P, P, P, I, I, I, F, F]),
    "jzhip_gemv": (I, [P, P, P, I, I, I, I, I, I, F, F]),
    "jzhip_gemm_fused": (I, [P, P, P, I, I, I, I, I, I, I, I, F, F, P, I, P, I, P, I]),
    "jzhip_gemm_rowsum": (I, [P, P, P, P, I, I, I, I, I, I, I, I, F, F]),
    "jzhip_gemm_fused_rowsum": (I, [P, P, P, P, I, I, I, I, I, I, I, I, F, F, P, I, P, I, P, I]),
    "jzhip_gemm_strided_batched": (I, [P, P, P, I, I, I, I, I, I, I, I, LL, LL, LL, I, F, F]),
    "jzhip_profile_gemm": (I, [I]),
    "jzhip_profile_gemm_report": (I, [C.c_char_p, Z]),
    "jzhip_add_bias": (I, [P, P, I, I]),
    "jzhip_softmax_cols": (I, [P, P, I, I, I]),
    "jzhip_softmax_rows": (I, [P, P, I, I, I]),
    "jzhip_attn_softmax": (I, [P, P, I, I, F, I, I]),
    "jzhip_attn_softmax_bwd": (I, [P, P, P, I, I, F, I]),
    "jzhip_softmax_xent": (I, [P, P, P, P, I, I, I]),
    "jzhip_softmax_xent_dense": (I, [P, P, P, P, I, I, I, F]),
    "jzhip_attention_fwd_ld": (I, [P, I, P, P, P, P, I, I, I, I, I, I]),
    "jzhip_attention_bwd_ld": (I, [P, P, P, I, P, P, I, P, P, P, I, P, I, I, I, I, I]),
    "jzhip_attention_flash_supported": (I, [I, I, I, I]),
    "jzhip_attention_flash_order": (I, [I, I, P, I]),
    "jzhip_attention_flash_fwd": (I, [P, I, P, P, P, P, I, I, I, I, I, I]),
    "jzhip_attention_flash_bwd": (I, [P, P, P, I, P, I, P, P, P, I, P, I, P, I, I, I, I, I]),
    "jzhip_attention_fwd": (I, [P, P, P, P, P, I, I, I, I, I]),
    "jzhip_attention_bwd": (I, [P, P, P, P, P, P, P, P, P, I, I, I, I]),
    "jzhip_layernorm_fwd": (I, [P, P, P, P, P, P, I, I]),
    "jzhip_layernorm_bwd": (I, [P, P, P, P, P, I, I]),
    "jzhip_layernorm_bwd_residual": (I, [P, P, P, P, P, P, I, I]),
    "jzhip_layernorm_jvp": (I, [P, P, P, P, P, I, I]),
    "jzhip_layernorm_param_grads": (I, [P, P, P, P, I, I]),
    "jzhip_layernorm_bwd_residual_sums": (I, [P, P, P, P, P, P, P, P, P, P, I, I]),
    "jzhip_adam_update": (I, [P, P, P, Z, F, F, F, F, I]),
    "jzhip_adamw_step": (I, [P, P, P, P, Z, F, F, F, F, F, I]),
    "jzhip_adamw_step_multi": (I, [C.POINTER(AdamTensor), I]),
    "jzhip_adamw_step_multi_counted": (I, [C.POINTER(AdamTensor), I, P]),
    "jzhip_counter_add": (I, [P, I]),
    "jzhip_im2col": (I, [P, P] + [I] * 12),
    "jzhip_col2im": (I, [P, P] + [I] * 12),
    "jzhip_conv_forward_reshape_bias": (I, [P, P, P, I, I, I]),
    "jzhip_conv_backward_reshape": (I, [P, P, I, I, I]),
    "jzhip_convtrans_scatter": (I, [P, P, P] + [I] * 12),
    "jzhip_convtrans_gather": (I, [P, P] + [I] * 12),
    "jzhip_convtrans_reshape": (I, [P, P, I, I, I, I]),
    "jzhip_conv2d_forward": (I, [P, P, P, P] + [I] * 14),
    "jzhip_conv2d_backward_weights": (I, [P, P, P] + [I] * 13),
    "jzhip_conv2d_backward_data": (I, [P, P, P] + [I] * 13),
    "jzhip_conv2d_check": (I, [I] * 14),
    "jzhip_conv2d_transposed": (I, [P, P, P, P] + [I] * 14),
}


class JzhipError(RuntimeError):
    def __init__(self, name: str, rc: int, text: str):
        super().__init__(f"{name} failed with rc={rc}: {text}")
        self.rc = rc


_lib = None


def load() -> C.CDLL:
    """Load libjzhip.so (built by ``python -m juzhen_amd.build``)."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise FileNotFoundError(
            f"{LIB_PATH} is missing: build it with `python -m juzhen_amd.build` "
            "(there is no fallback implementation)")
    lib = C.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the ABI and the table diverge
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(name: str, rc: int) -> None:
    if rc != 0:
        text = load().jzhip_error_string(rc)
        raise JzhipError(name, rc, text.decode() if text else "?")


class _Checked:
    """``jz.fill(ptr, n, v)`` calls ``jzhip_fill`` and raises on a non-zero rc."""

    def __getattr__(self, short: str):
        name = "jzhip_" + short
        fn = getattr(load(), name)
        res = SIGNATURES[name][0]
        if res is not I or short in ("runtime_available", "version", "num_compute_units", "attention_flash_supported",
                                    "attention_flash_order"):
            return fn

        def call(*args):
            check(name, fn(*args))

        call.__name__ = name
        setattr(self, short, call)
        return call


jz = _Checked()
