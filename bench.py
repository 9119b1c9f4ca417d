#!/usr/bin/env python3
"""Headline benchmark: transformer train-step tokens/s on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--two-stream] [--no-cpu-baseline] [--no-dropin] [--no-legs]

Workload (the character-level transformer configuration): language model over
vocab 256 byte tokens drawn from Zipf(s=1.1), context 256, batch 64 (16 384 tokens per step), 6
pre-LayerNorm decoder blocks, d_model 512, 8 heads, causal softmax attention,
FFN 2048 with GELU, tied embeddings, learned positional table, cross-entropy,
AdamW (lr 3e-4, wd 0.01), fp32 everywhere.  One step = forward + loss +
backward + optimiser on a synthetic batch that is already resident in HBM.

The whole step runs on one stream in program order, so a per-kernel trace of
the timed steps measures every kernel alone.  `--two-stream` issues the weight,
bias and LayerNorm-parameter gradients (leaves of the backward graph) on a
second stream beside the gradient chain; with the present GEMM kernels that is
2 % slower per step (concurrent tiled products share the CUs and each other's
L2), and the individual durations stop measuring the kernel.

Prints ONE JSON line.  `roofline` describes the dominant kernel (the fp32 MFMA
GEMM): algorithmic flops (2*m*n*k summed over its launches) divided by its
launch time, measured with HIP events around every launch in separate
instrumented steps after the timed region; those steps always run on one
stream.  `cpu_baseline` times the
reference's own CPU path (oracle/_ref, OpenBLAS build when available) on a
bounded sample of the same workload.  `dropin_api` is the same model written on
the reference's layer classes and run through the drop-in Matrix<ROCMfloat> API
(a prebuilt program started after the timed region; `--no-dropin` skips it, as
the profiler commands do).  `gemm_4096`, `streaming`, `c1_ops` and `configs` are
the other legs of the metric and the other benchmark configurations
(juzhen_amd/benchlegs.py), measured after the timed region; `--no-legs` skips them.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_FP32_MFMA_TFLOPS = 157.3

CFG = dict(vocab=256, d_model=512, heads=8, d_ff=2048, layers=6, seq=256, batch=64)


def zipf_tokens(rng, vocab, batch, seq, s=1.1):
    import numpy as np
    p = 1.0 / np.arange(1, vocab + 1) ** s
    p /= p.sum()
    return rng.choice(vocab, size=(batch, seq + 1), p=p).astype(np.int32)


class HipEvents:
    """hipEvent timing on the stream the library launches on (plain HIP runtime)."""

    def __init__(self):
        self.hip = C.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.hip.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [C.c_void_p]
        self.hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.hip.hipDeviceSynchronize.argtypes = []

    def event(self):
        e = C.c_void_p()
        assert self.hip.hipEventCreate(C.byref(e)) == 0
        return e

    def record(self, e, stream):
        assert self.hip.hipEventRecord(e, stream) == 0

    def elapsed_ms(self, a, b):
        assert self.hip.hipEventSynchronize(b) == 0
        ms = C.c_float()
        assert self.hip.hipEventElapsedTime(C.byref(ms), a, b) == 0
        return float(ms.value)

    def sync(self):
        assert self.hip.hipDeviceSynchronize() == 0


TRAFFIC_PROFILE = ROOT / "profiles" / "train_step_c4_hbm_traffic.txt"


def measured_traffic_bytes(kernel, path=TRAFFIC_PROFILE):
    """HBM bytes per launch of `kernel`, averaged over its dispatches in the counter runs of
    this script: the row of that kernel in the committed summary (rocprofv3 FETCH_SIZE and
    WRITE_SIZE, each scaled by what the same counter reads for a plain 256 MiB copy; columns
    `kernel  dispatches  fetch KiB  write KiB  total MiB`).  A kernel the summary does not
    hold raises: a renamed or re-tuned kernel must not report another kernel's bytes."""
    import re
    row = re.compile(r"^(?P<name>\S.*?)\s+(?P<n>\d+)\s+(?P<f>[\d.]+)\s+(?P<w>[\d.]+)\s+(?P<t>[\d.]+)\s*$")
    names = []
    for line in Path(path).read_text().splitlines():
        m = row.match(line)
        if not m:
            continue
        names.append(m["name"])
        # the summary truncates long names; the names compared are those of this library's kernels
        if m["name"] == kernel or (len(m["name"]) >= 60 and kernel.startswith(m["name"])):
            return (float(m["f"]) + float(m["w"])) * 1024.0
    raise KeyError(f"{path.name} holds no row for kernel {kernel!r} (rows: {names}); regenerate the counter summary")


def cpu_baseline(seconds_budget=40.0):
    """Reference CPU path (nearest reference architecture: ReLU FFN, Adam, untied
    head; examples/demo_transformer.cu wiring) at the benchmark's model size on a
    bounded sample of sequences."""
    import numpy as np
    import oracle
    ob = oracle.REF_DIR / "libjzref_openblas.so"
    kind_note = "OpenBLAS"
    lib = None
    cores = 1
    if ob.exists():
        try:
            lib = C.CDLL(str(ob))
            for dep in sorted(Path("/usr/local/lib").glob("python3*/dist-packages/scipy.libs/libscipy_openblas*.so")):
                blas = C.CDLL(str(dep))
                want = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
                blas.scipy_openblas_set_num_threads(C.c_int(want))
                blas.scipy_openblas_get_num_threads.restype = C.c_int
                cores = int(blas.scipy_openblas_get_num_threads())
                break
        except OSError:
            lib = None
    if lib is None:
        if not oracle.REF_LIB.exists():
            return None
        lib = C.CDLL(str(oracle.REF_LIB))
        kind_note = "BLAS-free (cpp/cpulinalg.hpp)"
        cores = 1
    lib.jzref_init()
    lib.jzref_lm_create.restype = C.c_void_p
    lib.jzref_lm_create.argtypes = [C.c_int] * 7
    lib.jzref_lm_step.restype = C.c_float
    lib.jzref_lm_step.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
    lib.jzref_lm_destroy.argtypes = [C.c_void_p]
    V, d, heads, ff, L, S = CFG["vocab"], CFG["d_model"], CFG["heads"], CFG["d_ff"], CFG["layers"], CFG["seq"]
    # the OpenBLAS build runs the benchmark's own batch (all 64 sequences: one warm-up step, then
    # two timed ones); the BLAS-free fallback is two orders of magnitude slower and gets one sequence
    B = CFG["batch"] if kind_note == "OpenBLAS" else 1
    N = S * B
    rng = np.random.default_rng(1234)
    tok = zipf_tokens(rng, V, B, S)          # the same ids the GPU leg trains on
    X = np.zeros((N, V + S), np.float32)     # column-major ((V+S) x N)
    Y = np.zeros((N, V), np.float32)
    n = np.arange(N)
    b, s_ = n // S, n % S
    X[n, tok[b, s_]] = 1
    X[n, V + s_] = 1
    Y[n, tok[b, s_ + 1]] = 1
    h = lib.jzref_lm_create(V, d, heads, ff, L, S, B)
    warm = 1 if kind_note == "OpenBLAS" else 0
    for _ in range(warm):
        lib.jzref_lm_step(h, X.ctypes.data, Y.ctypes.data)
    t0 = time.perf_counter()
    steps = 0
    while True:
        lib.jzref_lm_step(h, X.ctypes.data, Y.ctypes.data)
        steps += 1
        el = time.perf_counter() - t0
        if steps >= 2 or el > seconds_budget:
            break
    el = time.perf_counter() - t0
    lib.jzref_lm_destroy(h)
    return {
        "value": round(N * steps / el, 2), "unit": "tokens/s", "cores": cores, "kind": "reference",
        "sample": f"{steps} timed train step(s) after {warm} warm-up of the reference's own CPU classes (LinearLayer + "
                  f"6 TransformerLayer<float> + LogisticLayer, ReLU FFN, Adam, untied head: the nearest model the "
                  f"reference contains; {kind_note} build) at d_model 512 / 8 heads / d_ff 2048 / context 256 on "
                  f"{B} of the 64 sequences of the GPU leg's batch ({N} tokens per step); {cores} core(s) for BLAS, "
                  f"1 core elsewhere; {el:.1f} s timed",
    }


def cpu_configs(rows):
    """CPU baseline of the other configurations: oracle/_ref/bin/configs_cpu, the reference's
    Matrix<float> build (OpenBLAS for products, one core elsewhere) of the program whose
    Matrix<ROCMfloat> build produced `rows`, run after it on the same box for a few steps."""
    import tempfile
    from juzhen_amd import benchlegs
    exe = ROOT / "oracle" / "_ref" / "bin" / "configs_cpu"
    if not exe.exists():
        return
    with tempfile.TemporaryDirectory() as tmp:
        for cfg, (_, steps, key) in benchlegs.CONFIG_RUNS.items():
            val, wall = benchlegs.run_config_program(exe, cfg, steps, key, tmp)
            rows[cfg].update({"cpu_ms": val, "cpu_steps": steps, "cpu_wall_s": wall})
            if val and rows[cfg].get("gpu_ms"):
                rows[cfg]["speedup"] = round(val / rows[cfg]["gpu_ms"], 1)
    rows["cpu"] = ("reference Matrix<float> build of the same program (oracle/_ref/bin/configs_cpu), OpenBLAS with "
                   f"{os.environ.get('OMP_NUM_THREADS', os.cpu_count())} threads for products, one core elsewhere")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-legs", action="store_true",
                    help="skip the other legs of the metric (4096^3 GEMM, streaming kernels at 1 GiB, the "
                         "expression-chain ops and the MLP / CNN / UNet configurations), which run after the timed region")
    ap.add_argument("--no-dropin", action="store_true",
                    help="skip the run of the same model on the reference's layer classes (dropin_api key)")
    ap.add_argument("--two-stream", action="store_true",
                    help="issue the weight-gradient work of the backward pass on a second stream in the timed steps")
    ap.add_argument("--serial", action="store_true",
                    help="one stream, program order: the default (accepted so that older command lines still run)")
    ap.add_argument("--fresh-batches", action="store_true",
                    help="hand a new batch of host token ids to the model before every step (PCIe-inclusive rate); "
                         "by default one batch is uploaded before the timed region and reused")
    ap.add_argument("--cpu-baseline-only", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch a plain copy of 2^26 floats three times, so that a counter run of this "
                         "command holds a kernel of known traffic (256 MiB read, 256 MiB written per launch)")
    args = ap.parse_args()
    if args.cpu_baseline_only:
        # child process: the reference library prints its cumulative timers on
        # exit (cpp/helper.hpp:162-169), which must not reach the parent's stdout
        print("CPU_BASELINE " + json.dumps(cpu_baseline()), flush=True)
        return
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU only; --gpus N with N > 1 is not supported "
              "(the path has no collectives).", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch  # device presence check only; all compute goes through libjzhip.so

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from juzhen_amd import capi
    from juzhen_amd.lm import CharLM

    lib = capi.load()
    ev = HipEvents()
    stream = lib.jzhip_get_stream()

    model = CharLM(**CFG, gelu=True, tied=True, adamw=True, lr=3e-4, weight_decay=0.01, overlap=args.two_stream and not args.serial)
    model.init_random(0)
    rng = np.random.default_rng(1234)
    model.set_batch(zipf_tokens(rng, CFG["vocab"], CFG["batch"], CFG["seq"]))
    tokens_per_step = model.tokens_per_step

    if args.copy_calibration:
        n = 1 << 26
        src, dst = torch.zeros(n, device="cuda"), torch.empty(n, device="cuda")
        for _ in range(3):
            assert lib.jzhip_copy(C.c_void_p(dst.data_ptr()), C.c_void_p(src.data_ptr()), n) == 0
        ev.sync()
        del src, dst

    fresh = ([zipf_tokens(rng, CFG["vocab"], CFG["batch"], CFG["seq"]) for _ in range(8)]
             if args.fresh_batches else None)
    for i in range(args.warmup):
        if fresh:
            model.set_batch(fresh[i % len(fresh)])
        model.step()
    ev.sync()
    first_loss = model.loss()

    e0, e1 = ev.event(), ev.event()
    ev.sync()
    t0 = time.perf_counter()
    ev.record(e0, stream)
    for i in range(args.steps):
        if fresh:
            model.set_batch(fresh[i % len(fresh)])
        model.step()
    ev.record(e1, stream)
    gpu_ms = ev.elapsed_ms(e0, e1)
    ev.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    last_loss = model.loss()
    ms_per_step = max(gpu_ms, wall_ms) / args.steps
    value = tokens_per_step / (ms_per_step * 1e-3)

    # instrumented steps: HIP events around every tiled-GEMM launch, one stream
    model.set_overlap(False)
    lib.jzhip_profile_gemm(1)
    prof_steps = 2
    for _ in range(prof_steps):
        model.step()
    buf = C.create_string_buffer(1 << 16)
    assert lib.jzhip_profile_gemm_report(buf, len(buf)) == 0
    lib.jzhip_profile_gemm(0)
    kernels = json.loads(buf.value.decode())
    kernels.sort(key=lambda k: -k["total_ms"])
    gemm_ms_per_step = sum(k["total_ms"] for k in kernels) / prof_steps
    gemm_flops_per_step = sum(k["flops"] for k in kernels) / prof_steps
    dom = kernels[0]
    achieved = dom["flops"] / (dom["total_ms"] * 1e-3) / 1e12
    roofline = {
        "bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
        "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4),
        "traffic": round(measured_traffic_bytes(dom["kernel"])),
        "traffic_source": "profiles/train_step_c4_hbm_traffic.txt (rocprofv3 FETCH_SIZE + WRITE_SIZE runs of this script)",
        "kernel": dom["kernel"], "launches_per_step": dom["launches"] // prof_steps,
        "avg_launch_us": round(dom["total_ms"] * 1e3 / dom["launches"], 2),
        "flops_per_launch": round(dom["flops"] / dom["launches"], 1),
        "measured_in": "instrumented steps on one stream, as the timed steps",
        "all_gemm_kernels": {"tflops": round(gemm_flops_per_step / (gemm_ms_per_step * 1e-3) / 1e12, 2),
                             "ms_per_step": round(gemm_ms_per_step, 3),
                             "share_of_step": round(gemm_ms_per_step / ms_per_step, 3)},
    }

    cpu = None
    if not args.no_cpu_baseline:
        try:
            import subprocess
            r = subprocess.run([sys.executable, str(Path(__file__).resolve()), "--cpu-baseline-only"],
                               capture_output=True, text=True, timeout=300)
            line = next(l for l in r.stdout.splitlines() if l.startswith("CPU_BASELINE "))
            cpu = json.loads(line[len("CPU_BASELINE "):])
        except Exception as exc:  # the baseline must never take the GPU number down with it
            cpu = {"value": None, "unit": "tokens/s", "cores": 0, "kind": "reference", "sample": f"failed: {exc}"}

    # The same model written on the reference's own layer classes (LinearLayer + 6 x
    # TransformerLayer<ROCMfloat> + LogisticLayer, ReLU FFN, Adam) through the drop-in API:
    # what a user of Matrix<ROCMfloat> gets without the harness.  A prebuilt program; run
    # after the timed region, reported beside the headline number, never part of it.
    dropin = None
    dropin_bin = ROOT / "juzhen_amd" / "bin" / "lm_dropin_rocm"
    if not args.no_dropin and dropin_bin.exists():
        try:
            import re
            import subprocess
            r = subprocess.run([str(dropin_bin)], capture_output=True, text=True, timeout=200)
            line = next(l for l in r.stdout.splitlines() if l.startswith("RESULT dropin"))
            kv = dict(re.findall(r"(\w+)=(\S+)", line))
            dropin = {"tokens_per_s": float(kv["tokens_per_second"]), "ms_per_step": float(kv["mean_ms"]),
                      "steps": int(kv["steps"]), "warmup": int(kv["warmup"]),
                      "model": "LinearLayer + 6 x TransformerLayer<ROCMfloat> + LinearLayer + LogisticLayer "
                               "(ml/layer.hpp), d_model 512, 8 heads, FFN 2048 ReLU, context 256, batch 64, Adam",
                      "program": "juzhen_amd/bin/lm_dropin_rocm (juzhen_amd/harness/lm_dropin.cu)"}
        except Exception as exc:
            dropin = {"tokens_per_s": None, "error": str(exc)}

    param_count = int(model.param_count)
    flash_attention = model.flash_attention
    model.close()
    # The other legs of the metric (GEMM TFLOP/s and elementwise GB/s against their rooflines) and the
    # other benchmark configurations, measured in this run after the timed region; with the CPU
    # baseline enabled, the reference's CPU build of the same configurations program is timed beside them.
    legs = None
    if not args.no_legs:
        try:
            from juzhen_amd import benchlegs
            legs = benchlegs.run_all()
            if not args.no_cpu_baseline:
                cpu_configs(legs["configs"])
        except Exception as exc:
            legs = {"error": f"{type(exc).__name__}: {exc}"}

    out = {
        "metric": "transformer train-step tokens/s", "value": round(value, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "char-LM train step: vocab 256 (Zipf 1.1), context 256, batch 64, 6 pre-LN blocks, "
                               "d_model 512, 8 heads, FFN 2048 GELU, tied embeddings, learned positions, AdamW "
                               "lr 3e-4 wd 0.01", "tokens_per_step": tokens_per_step,
                   "backward_streams": 2 if args.two_stream and not args.serial else 1,
                   "batch_upload": "every step (host ids -> device inside the timed region)" if fresh
                                   else "once, before the timed region",
                   "attention": "no S x S matrix kept (jzhip_attention_flash_fwd/_bwd)" if flash_attention
                                else "probabilities materialised (jzhip_attention_fwd_ld/_bwd_ld)",
                   "parameters": param_count, "loss_first": round(first_loss, 4),
                   "loss_last": round(last_loss, 4), "gpu_ms_per_step": round(gpu_ms / args.steps, 3)},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "dropin_api": dropin,
    }
    if cpu and cpu.get("value"):
        out["speedup_vs_cpu_baseline"] = round(value / cpu["value"], 1)
    if legs:
        out.update(legs)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
