"""The C-ABI library loads and exports every symbol include/jzhip.h declares,
and the ctypes table mirrors the header.  No compute calls: runs without a GPU."""
import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "jzhip.h"


def declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(jzhip_\w+)\s*\(", text)))


def test_header_declares_the_reference_device_api():
    """One entry point per Juzhen::Rocm* function of cpp/hipbackend.hpp:10-136."""
    names = set(declared_symbols())
    rocm = ["runtime_available", "malloc", "free", "memcpy_h2d", "memcpy_d2h", "memcpy_d2d", "rand_uniform",
            "rand_normal", "fill", "exp_inplace", "log_inplace", "axpby", "affine_inplace", "hadamard",
            "hadamard_inplace", "eleminv_inplace", "copy", "square", "square_inplace", "tanh", "tanh_inplace",
            "dtanh", "dtanh_inplace", "stack_copy_cols", "stack_copy_rows", "slice_extract", "slice_assign",
            "gemm", "gemv", "gemm_nn", "im2col", "col2im", "conv_forward_reshape_bias", "conv_backward_reshape",
            "convtrans_scatter", "convtrans_gather", "convtrans_reshape"]
    assert len(rocm) == 37
    for r in rocm:
        assert "jzhip_" + r in names, r


def test_library_exports_every_declared_symbol():
    from juzhen_amd import capi
    if not capi.LIB_PATH.exists():
        pytest.fail(f"{capi.LIB_PATH} not built: run python -m juzhen_amd.build")
    lib = ctypes.CDLL(str(capi.LIB_PATH))
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, missing


def test_ctypes_table_matches_header():
    from juzhen_amd import capi
    assert sorted(capi.SIGNATURES) == declared_symbols()
    # argument counts agree with the prototypes
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    for name, (_, args) in capi.SIGNATURES.items():
        m = re.search(r"\b" + name + r"\s*\(([^;]*?)\)\s*;", text, flags=re.S)
        assert m, name
        params = m.group(1).strip()
        n = 0 if params in ("", "void") else params.count(",") + 1
        assert n == len(args), (name, n, len(args))


def test_argument_validation_without_gpu():
    """Null pointers and non-positive sizes are rejected with rc -1 before any launch
    (cpp/hipmatrix.cpp:611-612,672-674)."""
    from juzhen_amd import capi
    lib = capi.load()
    assert lib.jzhip_gemm(None, None, None, 2, 2, 2, 0, 0, 2, 2, 2, 1.0, 0.0) == -1
    assert lib.jzhip_gemm(None, None, None, 0, 2, 2, 0, 0, 2, 2, 2, 1.0, 0.0) == -1
    assert lib.jzhip_gemv(None, None, None, 2, 2, 0, 2, 1, 1, 1.0, 0.0) == -1
    assert lib.jzhip_sum_cols(None, None, 4, 4, 4) == -1
    assert lib.jzhip_im2col(None, None, 1, 4, 4, 3, 3, 1, 1, 1, 1, 4, 4, 1) == -1
    assert lib.jzhip_layernorm_fwd(None, None, None, None, None, None, 8, 8) == -1
    assert lib.jzhip_adam_update(None, None, None, 4, 1e-3, 0.9, 0.999, 1e-8, 1) == -1
    assert lib.jzhip_softmax_xent_dense(None, None, None, None, 4, 4, 4, 0.25) == -1
    assert lib.jzhip_mse_loss(None, None, None, 4, 1.0) == -1
    assert lib.jzhip_mse_grad(None, None, None, 4, 1.0) == -1
    assert lib.jzhip_mse_grad(None, None, None, 0, 1.0) == 0   # empty input is a no-op
    assert lib.jzhip_fill(None, 0, 1.0) == 0
    assert lib.jzhip_error_string(-1).decode().startswith("jzhip")
    assert lib.jzhip_version() >= 100


def test_product_code_never_reaches_into_the_oracle():
    """The oracle is test infrastructure: nothing that ships (the package's Python,
    the kernels, the C++ mirror, the train-step harness) may import, include or
    link it.  (juzhen_amd/build.py only names oracle/_ref as the output directory
    of the reference-program builds.)"""
    import re
    root = Path(__file__).resolve().parent.parent
    bad = []
    for p in (root / "juzhen_amd").rglob("*"):
        if p.is_dir() or "build" in p.relative_to(root).parts[1:2] or p.suffix not in (
                ".py", ".hip", ".hpp", ".cuh", ".cpp", ".cu", ".h"):
            continue
        text = p.read_text(errors="ignore")
        if p.suffix == ".py":
            if re.search(r"^\s*(import oracle|from oracle)", text, re.M):
                bad.append(str(p))
        elif re.search(r'#include\s*[<"][^>"]*(oracle|jz_oracle|ref_shim)', text) or "jzo_" in text or "jzref_" in text:
            bad.append(str(p))
    assert not bad, bad


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU: `--gpus N` with N above 1, or a launch under a
    multi-rank launcher, exits with status 2 and says why, before anything touches
    a GPU."""
    import os
    import subprocess
    import sys
    env = {k: v for k, v in os.environ.items() if k not in ("WORLD_SIZE", "RANK", "LOCAL_RANK")}
    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       env=env, timeout=300)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""
    r = subprocess.run([sys.executable, str(ROOT / "bench.py")], capture_output=True, text=True,
                       env={**env, "WORLD_SIZE": "2"}, timeout=300)
    assert r.returncode == 2
    assert "one GPU" in r.stderr


def test_roofline_traffic_comes_from_the_committed_counter_summary():
    """bench.py reads the HBM bytes per launch of its dominant kernel from the rocprofv3
    summary under profiles/ instead of carrying constants: every tiled-GEMM row parses,
    the bytes are fetch + write KiB of the row, and a kernel the summary does not hold
    raises instead of reporting nothing."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_module", ROOT / "bench.py")
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    text = bench.TRAFFIC_PROFILE.read_text()
    rows = [l for l in text.splitlines() if l.startswith("gemm_mfma_kernel<")]
    assert len(rows) >= 4
    for l in rows:
        name = l[:l.index(">") + 1]
        f, w = (float(x) for x in l.split()[-3:-1])
        assert bench.measured_traffic_bytes(name) == (f + w) * 1024.0
    with pytest.raises(KeyError):
        bench.measured_traffic_bytes("gemm_mfma_kernel<9, 9, 9, 9, false, false, false, false>")


@pytest.mark.parametrize("S", [32, 64, 96, 128, 160, 192, 224, 256])
@pytest.mark.parametrize("causal", [0, 1])
def test_flash_attention_visiting_order(S, causal):
    """Host logic of the attention backward that keeps no S x S matrix: every cell
    (query tile, key tile) the mask leaves is visited exactly once, the waves of a step
    are on distinct query tiles (each element of dQ therefore has one summation order),
    a wave owns key tiles o and S/16-1-o and finishes the first before the second, and
    under the causal mask every wave gets the same number of cells."""
    import numpy as np
    from juzhen_amd import capi
    lib = ctypes.CDLL(str(capi.LIB_PATH))
    tiles, owners = S // 16, S // 32
    cells = (ctypes.c_int * (2 * 2 * tiles * owners))()
    steps = lib.jzhip_attention_flash_order(S, causal, cells, len(cells))
    assert steps == (tiles + 1 if causal else 2 * tiles)
    c = np.array(cells[:2 * steps * owners]).reshape(steps, owners, 2)
    seen = np.zeros((tiles, tiles), int)
    for j in range(steps):
        assert len(set(c[j, :, 0])) == owners                      # distinct query tiles within a step
        for o in range(owners):
            t, k = c[j, o]
            assert k in (o, tiles - 1 - o) and (not causal or t >= k)
            seen[t, k] += 1
    want = np.tril(np.ones((tiles, tiles), int)) if causal else np.ones((tiles, tiles), int)
    assert np.array_equal(seen, want)
    for o in range(owners):
        ks = list(c[:, o, 1])
        assert ks == sorted(ks, key=lambda k: k != o)               # all of key tile o first
    assert lib.jzhip_attention_flash_order(S, causal, cells, 3) == -1
    assert lib.jzhip_attention_flash_order(S + 16, causal, cells, len(cells)) == -1
