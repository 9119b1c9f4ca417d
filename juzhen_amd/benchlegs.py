"""The legs of the headline metric beside the transformer step: fp32 GEMM at
4096^3 against the MFMA roofline, streaming kernels at 1 GiB and more against
the HBM roofline, the per-op latencies of the 1024 x 1024 expression chain, and
the step times of the other benchmark configurations (MLP, CNN, UNet) on this
backend (bench.py times the reference's CPU build of the same program beside them).

    from juzhen_amd import benchlegs
    benchlegs.run_all()   -> dict with the keys gemm_4096, streaming, c1_ops, configs

Timing follows tests/benchmarkCoreOps.cu:35-54,62-104 of the reference: 3
warm-up calls, 20 timed samples, HIP events on the library's stream; the
median is reported.  A sample of a short kernel is an event pair around enough
back-to-back launches to last about 100 us.  bench.py calls this after its
timed region; nothing here runs inside it.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
import tempfile
import time
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
HBM_GBS = 8000.0
MFMA_TFLOPS = 157.3
WARMUP, SAMPLES = 3, 20


class _Timer:
    def __init__(self, lib):
        h = self.hip = C.CDLL("libamdhip64.so")
        h.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        h.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        h.hipEventSynchronize.argtypes = [C.c_void_p]
        h.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.a, self.b = C.c_void_p(), C.c_void_p()
        assert h.hipEventCreate(C.byref(self.a)) == 0 and h.hipEventCreate(C.byref(self.b)) == 0
        self.stream = C.c_void_p(lib.jzhip_get_stream())

    def _ms(self, fn, reps):
        h = self.hip
        assert h.hipEventRecord(self.a, self.stream) == 0
        for _ in range(reps):
            fn()
        assert h.hipEventRecord(self.b, self.stream) == 0
        assert h.hipEventSynchronize(self.b) == 0
        ms = C.c_float()
        assert h.hipEventElapsedTime(C.byref(ms), self.a, self.b) == 0
        return ms.value / reps

    def median_us(self, fn):
        for _ in range(WARMUP):
            fn()
        first = self._ms(fn, 1)
        reps = max(1, min(64, int(0.1 / max(first, 1e-4))))
        ts = sorted(self._ms(fn, reps) for _ in range(SAMPLES))
        return ts[len(ts) // 2] * 1e3


def _P(t):
    return C.c_void_p(t.data_ptr())


def _hbm(us, nbytes):
    gbs = nbytes / (us * 1e-6) / 1e9
    return {"us": round(us, 1), "MB": round(nbytes / 1e6, 1), "GB/s": round(gbs), "frac": round(gbs / HBM_GBS, 3)}


def gemm_4096(jz, tm, torch):
    """C = op(A) op(B) at 4096^3 in the four transpose variants (2*m*n*k flops)."""
    n = 4096
    A, B, Cm = (torch.randn(n * n, device="cuda") for _ in range(3))
    out = {}
    # the GPU has idled through the CPU leg before this one: bring its clocks back up first
    for _ in range(40):
        jz.gemm(_P(A), _P(B), _P(Cm), n, n, n, 0, 0, n, n, n, 1.0, 0.0)
    for name, ta, tb in (("NN", 0, 0), ("NT", 0, 1), ("TN", 1, 0), ("TT", 1, 1)):
        us = tm.median_us(lambda: jz.gemm(_P(A), _P(B), _P(Cm), n, n, n, ta, tb, n, n, n, 1.0, 0.0))
        tf = 2.0 * n ** 3 / (us * 1e-6) / 1e12
        out[name] = {"us": round(us, 1), "TFLOP/s": round(tf, 1), "frac": round(tf / MFMA_TFLOPS, 3)}
    return out


def streaming(jz, tm, torch):
    """Bandwidth-bound entry points on operands of 1 GiB (algorithmic bytes per call
    over the median time, against 8 TB/s)."""
    out = {}
    n = 1 << 28
    a, b, o = torch.randn(n, device="cuda"), torch.randn(n, device="cuda"), torch.empty(n, device="cuda")
    out["copy 2^28"] = _hbm(tm.median_us(lambda: jz.copy(_P(o), _P(a), n)), 8 * n)
    out["exp 2^28"] = _hbm(tm.median_us(lambda: jz.exp(_P(o), _P(a), n)), 8 * n)
    out["axpby 2^28"] = _hbm(tm.median_us(lambda: jz.axpby(_P(o), _P(a), _P(b), n, 1.0, 2.0)), 12 * n)
    r = c = 16384
    v = torch.empty(r, device="cuda")
    out["sum_rows 16384x16384"] = _hbm(tm.median_us(lambda: jz.sum_rows(_P(v), _P(a), r, c, r)), 4 * (r * c + r))
    out["sum_cols 16384x16384"] = _hbm(tm.median_us(lambda: jz.sum_cols(_P(v), _P(a), r, c, r)), 4 * (r * c + c))
    out["softmax_cols 16384x16384"] = _hbm(tm.median_us(lambda: jz.softmax_cols(_P(o), _P(a), r, c, r)), 8 * r * c)
    out["softmax_rows 16384x16384"] = _hbm(tm.median_us(lambda: jz.softmax_rows(_P(o), _P(a), r, c, r)), 8 * r * c)
    # single-read row softmax forms (rows of at most 2048 columns) at 0.5 GiB and 128 MiB
    out["softmax_rows 65536x2048"] = _hbm(tm.median_us(lambda: jz.softmax_rows(_P(o), _P(a), 65536, 2048, 65536)), 8 * 65536 * 2048)
    out["softmax_rows 16384x2048"] = _hbm(tm.median_us(lambda: jz.softmax_rows(_P(o), _P(a), 16384, 2048, 16384)), 8 * 16384 * 2048)
    out["softmax_rows 131072x256"] = _hbm(tm.median_us(lambda: jz.softmax_rows(_P(o), _P(a), 131072, 256, 131072)), 8 * 131072 * 256)
    dim, N = 512, 1 << 19
    inv, g, be = torch.empty(N, device="cuda"), torch.ones(dim, device="cuda"), torch.zeros(dim, device="cuda")
    out["layernorm_fwd 512x524288"] = _hbm(
        tm.median_us(lambda: jz.layernorm_fwd(_P(o), _P(b), _P(inv), _P(a), _P(g), _P(be), dim, N)),
        4 * (3 * dim * N + N + 2 * dim))
    del b, o
    m, vv = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    w = torch.randn(n, device="cuda")
    out["adamw_step 2^28"] = _hbm(
        tm.median_us(lambda: jz.adamw_step(_P(w), _P(a), _P(m), _P(vv), n, 1e-3, 0.9, 0.999, 1e-8, 0.01, 3)), 28 * n)
    return out


def c1_ops(jz, tm, torch):
    """Median latency of each operation of the expression-chain configuration
    (log(exp(A*B)+1)/5, row softmax, row and column sums) on 1024 x 1024 operands."""
    n = 1024
    A, B = torch.randn(n * n, device="cuda") / 32, torch.randn(n * n, device="cuda") / 32
    Cm, S, v = torch.empty(n * n, device="cuda"), torch.empty(n * n, device="cuda"), torch.empty(n, device="cuda")
    ops = {
        "gemm": lambda: jz.gemm(_P(A), _P(B), _P(Cm), n, n, n, 0, 0, n, n, n, 1.0, 0.0),
        "exp": lambda: jz.exp(_P(S), _P(Cm), n * n),
        "affine": lambda: jz.affine(_P(S), _P(Cm), n * n, 1.0, 1.0),
        "log": lambda: jz.log(_P(S), _P(A), n * n),
        "softmax_rows": lambda: jz.softmax_rows(_P(S), _P(Cm), n, n, n),
        "softmax_cols": lambda: jz.softmax_cols(_P(S), _P(Cm), n, n, n),
        "sum_rows": lambda: jz.sum_rows(_P(v), _P(Cm), n, n, n),
        "sum_cols": lambda: jz.sum_cols(_P(v), _P(Cm), n, n, n),
    }
    A.abs_().add_(0.5)
    return {k: round(tm.median_us(f), 2) for k, f in ops.items()}


CONFIG_RUNS = {  # config -> (steps on the GPU, steps of a CPU run of the same program, key of the RESULT line)
    "c1": (0, 0, "c1_chain_ms"), "c2": (203, 23, "c2_ms_per_step"), "c3": (102, 12, "c3_ms_per_step"),
    "c5": (41, 3, "c5_ms_per_step"),
}


def run_config_program(exe, cfg, steps, key, tmp):
    """One run of a build of juzhen_amd/harness/configs.cu; returns (value of its RESULT line, wall seconds)."""
    env = dict(os.environ, JZ_CONFIG=cfg, JZ_SCALE="full", JZ_STEPS=str(steps), JZ_OUT=tmp)
    t0 = time.perf_counter()
    try:
        r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=240, env=env)
        val = next((float(l.split()[2]) for l in r.stdout.splitlines() if l.startswith(f"RESULT {key} ")), None)
    except Exception:   # a leg that fails must not take the headline number down with it
        val = None
    return val, round(time.perf_counter() - t0, 1)


def configs():
    """ms per training step of the MLP (c2), CNN (c3) and UNet (c5) configurations and ms per
    evaluation of the expression chain (c1) on this backend: juzhen_amd/harness/configs.cu built
    against Matrix<ROCMfloat> (juzhen_amd/bin/configs_rocm)."""
    exe = PKG / "bin" / "configs_rocm"
    out = {}
    with tempfile.TemporaryDirectory() as tmp:
        for cfg, (steps, _, key) in CONFIG_RUNS.items():
            if not exe.exists():
                out[cfg] = {"gpu_ms": None}
                continue
            val, wall = run_config_program(exe, cfg, steps, key, tmp)
            out[cfg] = {"gpu_ms": val, "gpu_steps": steps, "gpu_wall_s": wall}
    out["unit"] = "ms per step (c1: ms per evaluation of the chain)"
    return out


def run_all():
    import torch

    from juzhen_amd import capi
    lib = capi.load()
    tm = _Timer(lib)
    res = {"convention": f"{WARMUP} warm-ups, median of {SAMPLES} samples, HIP events on the library's stream"}
    res["gemm_4096"] = gemm_4096(capi.jz, tm, torch)
    torch.cuda.empty_cache()
    res["streaming"] = streaming(capi.jz, tm, torch)
    torch.cuda.empty_cache()
    res["c1_ops"] = c1_ops(capi.jz, tm, torch)
    torch.cuda.empty_cache()
    res["configs"] = configs()
    return res


if __name__ == "__main__":
    import json
    print(json.dumps(run_all()))
