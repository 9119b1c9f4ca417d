"""The reference's own ROCm test programs, compiled unchanged against this
backend (juzhen_amd/cpp/hipmatrix.cuh, hipmatrix.cpp, hipkernels.cpp swapped
into an overlay of the reference tree) and run on the GPU.  The binaries are
built in the container by `python -m juzhen_amd.build --host` into
oracle/_ref/bin/ and travel with the working tree; each must exit 0
(the reference's ctest convention, CMakeLists.txt:320-400; 77 = skip).
The programs of juzhen_amd/harness/ (this package's own sources on the
Matrix<ROCMfloat> API) are built by the same step into juzhen_amd/bin/."""
import json
import os
import struct
import subprocess
from pathlib import Path

import pytest

from util import need_ref_binary

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parent.parent
BIN = ROOT / "oracle" / "_ref" / "bin"
HARNESS_BIN = ROOT / "juzhen_amd" / "bin"
PROJECT_DIR = Path("/tmp/jz_project")   # the PROJECT_DIR the programs were compiled with

PROGRAMS = ["testRocmDeviceProof", "testRocmOpsSmoke", "testRocmCpuParity", "testbasic", "testStackOps",
            "testElementwiseReduceTorchDump", "testConvBackendParity", "testUNet", "testTransformerRef",
            "testTransformer", "testUNetLearning", "testTransformerTorchDump", "testRectifiedFlowTinyUNetParity",
            "testRectifiedPathParity"]


@pytest.fixture(scope="module")
def project_dir():
    (PROJECT_DIR / "res").mkdir(parents=True, exist_ok=True)
    (PROJECT_DIR / "tests").mkdir(parents=True, exist_ok=True)
    # tests/basic.testdata in the .matrix layout (cpp/core.hpp:518-525)
    gold = json.loads((ROOT / "tests" / "golden" / "basic_chain.json").read_text())
    data = [float.fromhex(h) for h in gold["data"]]
    raw = struct.pack("<3i", gold["numrow"], gold["numcol"], gold["transpose"]) + struct.pack(f"<{len(data)}f", *data)
    (PROJECT_DIR / "tests" / "basic.testdata").write_bytes(raw)
    return PROJECT_DIR


@pytest.mark.parametrize("name", PROGRAMS)
def test_reference_program(gpu, project_dir, name):
    exe = need_ref_binary(BIN / name)
    print(f"running {name}", flush=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300, cwd=str(project_dir))
    tail = "\n".join((r.stdout + r.stderr).splitlines()[-40:])
    if r.returncode == 77:
        pytest.skip(f"{name} skipped itself:\n{tail}")
    assert r.returncode == 0, f"{name} exited {r.returncode}\n{tail}"


def test_mirror_transpose_and_ownership_semantics(gpu, project_dir):
    """juzhen_amd/harness/semantics.cu: every add / hadmd / division / slice /
    stack / sum / reduce / softmax case with mismatched transpose flags, the
    rvalue buffer-reuse rules, the tests/basic.testdata chain and the
    shape-mismatch exceptions, Matrix<ROCMfloat> against Matrix<float> in one
    program, bit for bit (tests/testbasic.cu and tests/testStackOps.cu hold no
    ROCMfloat section, so a ROCm build of those two runs the CPU type only)."""
    exe = need_ref_binary(HARNESS_BIN / "semantics_rocm")
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300, cwd=str(project_dir))
    lines = [l for l in (r.stdout + r.stderr).splitlines() if not l.startswith("profiler:")]
    print("\n".join(lines[-30:]))
    assert r.returncode == 0, "\n".join(l for l in lines if "FAIL" in l or "exception" in l)[-4000:]
    assert any(l.startswith("PASSED") for l in lines)


def test_forward_mode_tangents(gpu, project_dir):
    """juzhen_amd/harness/jvp_check.cu: LayerNorm, dense-stack and TransformerLayer
    tangents on Matrix<ROCMfloat> against the CPU tangents of layers with the same
    weights (1e-3; 1e-4 for the dense stack and LayerNorm), adjoint consistency with
    backprop on the device (1e-4) and central differences (5e-2, the criteria of
    tests/testJVP.cu:60-95, which itself skips on ROCm)."""
    exe = need_ref_binary(HARNESS_BIN / "jvp_check_rocm")
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300, cwd=str(project_dir))
    lines = [l for l in (r.stdout + r.stderr).splitlines() if l.startswith(("ok", "FAIL", "PASSED"))]
    print("\n".join(lines))
    assert r.returncode == 0, (r.stdout + r.stderr)[-3000:]
    assert any(l.startswith("PASSED") for l in lines)


def test_transformer_dump_against_float64_autograd(gpu, project_dir):
    """tests/testTransformerTorchDump.cu run on Matrix<ROCMfloat> writes weights,
    input, upstream gradient, forward output and input gradient of one
    TransformerLayer (format :14-18).  The reference checks that file with a
    PyTorch script; here the same file is checked against a float64 autograd
    statement of the block written from its definition (pre-LN, causal softmax
    attention with 1/sqrt(d_h), ReLU FFN, two residuals; ml/layer.hpp:2865-3024)
    at the reference's tolerance 1e-4."""
    import numpy as np
    import torch
    exe = need_ref_binary(BIN / "testTransformerTorchDump")
    dump = PROJECT_DIR / "res" / "transformer_torch_dump.bin"
    if dump.exists():
        dump.unlink()
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300, cwd=str(project_dir))
    assert r.returncode == 0 and dump.exists(), (r.stdout + r.stderr)[-2000:]
    raw = dump.read_bytes()
    assert raw[:8] == b"JZTFDMP1"
    d_model, d_k, d_ff, S, B, heads = struct.unpack("<6i", raw[8:32])
    at = 32
    mats = []
    for _ in range(17):
        rows, cols = struct.unpack("<2i", raw[at:at + 8])
        at += 8
        a = np.frombuffer(raw, dtype="<f4", count=rows * cols, offset=at).reshape(cols, rows).T
        at += 4 * rows * cols
        mats.append(torch.tensor(a.astype(np.float64)))
    assert at == len(raw)
    Wq, Wk, Wv, Wo, bo, W1, b1, W2, b2, g1, be1, g2, be2, x, g, out, dx = mats
    x = x.clone().requires_grad_(True)
    dh = d_k // heads

    def ln(t, gamma, beta):
        mu = t.mean(0, keepdim=True)
        var = ((t - mu) ** 2).mean(0, keepdim=True)
        return (t - mu) / torch.sqrt(var + 1e-5) * gamma + beta

    x1 = ln(x, g1, be1)
    q, k, v = Wq @ x1, Wk @ x1, Wv @ x1
    mask = torch.triu(torch.ones(S, S, dtype=torch.bool), 1)
    H = torch.zeros_like(q)
    for hh in range(heads):
        for b in range(B):
            rs, cs = slice(hh * dh, (hh + 1) * dh), slice(b * S, (b + 1) * S)
            sc = (q[rs, cs].T @ k[rs, cs]) / np.sqrt(dh)
            a = torch.softmax(sc.masked_fill(mask, -1e9), dim=1)
            H[rs, cs] = v[rs, cs] @ a.T
    R = x + Wo @ H + bo
    want = R + W2 @ torch.relu(W1 @ ln(R, g2, be2) + b1) + b2
    want.backward(g)
    assert float((out - want.detach()).abs().max()) <= 1e-4
    assert float((dx - x.grad).abs().max()) <= 1e-4
