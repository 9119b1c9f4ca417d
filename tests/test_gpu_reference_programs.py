"""The reference's own ROCm test programs, compiled unchanged against this
backend (juzhen_amd/cpp/hipmatrix.cuh, hipmatrix.cpp, hipkernels.cpp swapped
into an overlay of the reference tree) and run on the GPU.  The binaries are
built in the container by `python -m juzhen_amd.build --host` into
oracle/_ref/bin/ and travel with the working tree; each must exit 0
(the reference's ctest convention, CMakeLists.txt:320-400; 77 = skip)."""
import json
import os
import struct
import subprocess
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parent.parent
BIN = ROOT / "oracle" / "_ref" / "bin"
PROJECT_DIR = Path("/tmp/jz_project")   # the PROJECT_DIR the programs were compiled with

PROGRAMS = ["testRocmDeviceProof", "testRocmOpsSmoke", "testRocmCpuParity", "testbasic", "testStackOps",
            "testElementwiseReduceTorchDump", "testConvBackendParity", "testUNet", "testTransformerRef",
            "testTransformer"]


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
    exe = BIN / name
    if not exe.exists():
        pytest.skip(f"{exe} not built (needs the reference tree at build time)")
    print(f"running {name}", flush=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300, cwd=str(project_dir))
    tail = "\n".join((r.stdout + r.stderr).splitlines()[-40:])
    if r.returncode == 77:
        pytest.skip(f"{name} skipped itself:\n{tail}")
    assert r.returncode == 0, f"{name} exited {r.returncode}\n{tail}"
