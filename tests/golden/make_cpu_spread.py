"""Writes tests/golden/c3_full_cpu_build_spread.json: how far the reference's own two
CPU builds drift apart over 100 training steps of the CNN configuration at full size.

    python tests/golden/make_cpu_spread.py        (build container: needs /root/reference, ~2 min)

The program is juzhen_amd/harness/configs.cu compiled against the reference's CPU
Matrix<float> twice: with OpenBLAS products (oracle/_ref/bin/configs_cpu, built by
`python -m juzhen_amd.build --host`) and with the reference's own BLAS-free products
(-DJUZHEN_NO_BLAS, cpp/cpulinalg.hpp; compiled here into oracle/_ref/bin/).  Both train
on the same host-generated batch; only the summation order inside the products differs.
The configuration memorises one batch of random labels, the loss falls by three orders
of magnitude, and the two loss curves separate step by step; the fixture holds both
curves and their relative difference, which bounds what any third implementation can be
asked to reproduce after that many steps.
"""
import json
import os
import subprocess
import tempfile
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent.parent
REF = Path(os.environ.get("JUZHEN_REFERENCE", "/root/reference"))
BIN = ROOT / "oracle" / "_ref" / "bin"
STEPS = 100


def main():
    blas = BIN / "configs_cpu"
    assert blas.exists(), "run `python -m juzhen_amd.build --host` first"
    plain = BIN / "configs_cpu_noblas"
    subprocess.run(["g++", "-std=c++20", "-O2", "-x", "c++", "-DLOGGING_OFF", '-DPROJECT_DIR="/tmp/jz_project"', "-w",
                    f"-I{REF}", f"-I{REF / 'tests'}", "-DJUZHEN_NO_BLAS", "-ffp-contract=off",
                    str(REF / "cpp" / "launcher.cu"), str(ROOT / "juzhen_amd" / "harness" / "configs.cu"),
                    "-o", str(plain)], check=True)
    curves = {}
    for name, exe in (("openblas", blas), ("blas_free", plain)):
        with tempfile.TemporaryDirectory() as tmp:
            env = dict(os.environ, JZ_CONFIG="c3", JZ_SCALE="full", JZ_STEPS=str(STEPS), JZ_OUT=tmp)
            subprocess.run([str(exe)], check=True, env=env, capture_output=True)
            curves[name] = np.fromfile(Path(tmp) / "c3_losses.cpu.f32", dtype=np.float32)
    a, b = curves["openblas"].astype(np.float64), curves["blas_free"].astype(np.float64)
    rel = np.abs(a - b) / np.abs(a)
    out = {"config": "c3 full (CNN, batch 128), 100 Adam steps on one batch",
           "program": "juzhen_amd/harness/configs.cu against the reference's Matrix<float>",
           "losses_openblas": [float.hex(float(x)) for x in curves["openblas"]],
           "losses_blas_free": [float.hex(float(x)) for x in curves["blas_free"]],
           "relative_difference": [float(f"{x:.3e}") for x in rel]}
    (Path(__file__).resolve().parent / "c3_full_cpu_build_spread.json").write_text(json.dumps(out, indent=1))
    print("worst relative difference", rel.max(), "at step", int(rel.argmax()))


if __name__ == "__main__":
    main()
