"""Build the gfx950 device library (libjzhip.so) in-tree with hipcc.

Usage: python -m juzhen_amd.build [--force]

One shared object is produced from every ``csrc/*.hip`` file.  Objects are
rebuilt only when their source (or a header) is newer, unless --force.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
OBJ = PKG / "build"
LIB = PKG / "lib" / "libjzhip.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -ffp-contract=off: the CPU path this library is checked against rounds after
# every multiply and add; gfx950 fp32 arithmetic is IEEE, so with contraction
# off the elementwise/Adam kernels are bit-identical to it.  The MFMA GEMM is
# unaffected by the flag.  Packed-fp32 instructions are disabled on purpose.
COMMON_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    f"-I{ROOT / 'include'}",
    f"-I{CSRC}",
]


def _stale(target: Path, deps: list[Path]) -> bool:
    if not target.exists():
        return True
    t = target.stat().st_mtime
    return any(d.stat().st_mtime > t for d in deps)


def _compile(src: Path, force: bool) -> Path:
    obj = OBJ / (src.stem + ".o")
    headers = list(CSRC.glob("*.hpp")) + [ROOT / "include" / "jzhip.h"]
    if force or _stale(obj, [src, *headers]):
        cmd = [HIPCC, *COMMON_FLAGS, "-c", str(src), "-o", str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        # hipcc's host pass warns that it does not know -packed-fp32-ops: harmless
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src.name}:\n{err}")
        if err.strip():
            sys.stderr.write(err + "\n")
    return obj


def build(force: bool = False, jobs: int = 6) -> Path:
    OBJ.mkdir(parents=True, exist_ok=True)
    LIB.parent.mkdir(parents=True, exist_ok=True)
    srcs = sorted(CSRC.glob("*.hip"))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    if force or _stale(LIB, objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stderr}")
    return LIB


# ── host-side mirror: Matrix<ROCMfloat> + the reference's own programs ─────────
#
# juzhen_amd/cpp holds drop-in replacements for three files of the reference
# tree (cpp/hipmatrix.cuh, cpp/hipmatrix.cpp, cpp/hipkernels.cpp).  They only
# compile together with the reference's headers, so this step needs the
# reference tree.  It never copies reference sources: it builds a directory of
# symlinks ("overlay") in which those three names point at our files and every
# other name points into the reference tree, compiles the reference's own
# ROCm test programs in that overlay against libjzhip.so, and writes those
# binaries (the reference's own tests: checkers) to oracle/_ref/bin/.  The
# programs of juzhen_amd/harness/*.cu, this package's own sources written
# against the Matrix<ROCMfloat> API, go to juzhen_amd/bin/.
REFERENCE_ROOT = Path(os.environ.get("JUZHEN_REFERENCE", "/root/reference"))
OVERLAY = OBJ / "overlay"
REF_BIN = ROOT / "oracle" / "_ref" / "bin"
BIN = PKG / "bin"
HOST_SRC = PKG / "cpp"
OURS = {"hipmatrix.cuh", "hipmatrix.cpp", "hipkernels.cpp"}
# a writable PROJECT_DIR that exists on any box (tests that dump files use it)
PROJECT_DIR = "/tmp/jz_project"

REFERENCE_PROGRAMS = [
    "tests/testRocmDeviceProof.cu",
    "tests/testRocmOpsSmoke.cu",
    "tests/testRocmCpuParity.cu",
    "tests/testbasic.cu",
    "tests/testStackOps.cu",
    "tests/testElementwiseReduceTorchDump.cu",
    "tests/testConvBackendParity.cu",
    "tests/testUNet.cu",
    "tests/testTransformerRef.cu",
    "tests/testTransformer.cu",
    "tests/testUNetLearning.cu",
    "tests/testTransformerTorchDump.cu",
    "tests/testRectifiedFlowTinyUNetParity.cu",
    "tests/testRectifiedPathParity.cu",
]

HOST_FLAGS = [
    "-x", "hip", "--offload-arch=gfx950", "-std=c++20", "-O2", "-fPIC",
    "-DROCM_HIP", "-DLOGGING_OFF", "-DJUZHEN_NO_BLAS", f'-DPROJECT_DIR="{PROJECT_DIR}"',
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-w",
    f"-I{ROOT / 'include'}",
]


def _link_tree(src_dir: Path, dst_dir: Path, replace: dict[str, Path]):
    dst_dir.mkdir(parents=True, exist_ok=True)
    for f in src_dir.iterdir():
        target = replace.get(f.name, f)
        link = dst_dir / f.name
        if link.is_symlink() or link.exists():
            link.unlink()
        link.symlink_to(target)


def _relink(link: Path, target: Path):
    if link.is_symlink() or link.exists():
        link.unlink()
    link.symlink_to(target)


def make_overlay() -> Path:
    """Symlink farm: the reference tree with our three cpp/ files swapped in,
    and ml/util.cuh / ml/layer.hpp each followed by the one ROCm hook include a
    maintainer appends to those files."""
    _link_tree(REFERENCE_ROOT / "cpp", OVERLAY / "cpp", {n: HOST_SRC / n for n in OURS})
    for extra in HOST_SRC.glob("hipfused*.hpp"):
        _relink(OVERLAY / "cpp" / extra.name, extra)
    _link_tree(REFERENCE_ROOT / "ml", OVERLAY / "ml", {})
    # ml/util.cuh: upstream file followed by the one hook include.  ml/layer.hpp: the same, and
    # the ROCm ConvLayer and convtransLayer blocks of the upstream file (ml/layer.hpp:1562-1872) are replaced by
    # cpp/hipconv.hpp -- the maintainer swaps the block for an #include; here the upstream class
    # is compiled under another name so that the reference file itself stays untouched.
    wrappers = {
        "util.cuh": '#include "./upstream_util.cuh"\n#ifdef ROCM_HIP\n#include "../cpp/hipfused_util.hpp"\n#endif\n',
        "layer.hpp": '#ifdef ROCM_HIP\n#define ConvLayer ConvLayer_patch_matrix_route\n'
                     '#define convtransLayer convtransLayer_patch_matrix_route\n'
                     '#define ConvTransLayer ConvTransLayer_patch_matrix_route\n#endif\n'
                     '#include "./upstream_layer.hpp"\n'
                     '#ifdef ROCM_HIP\n#undef ConvLayer\n#undef convtransLayer\n#undef ConvTransLayer\n'
                     '#include "../cpp/hipfused.hpp"\n'
                     '#include "../cpp/hipconv.hpp"\n#endif\n',
    }
    for extra in HOST_SRC.glob("hipconv*.hpp"):
        _relink(OVERLAY / "cpp" / extra.name, extra)
    for fname, text in wrappers.items():
        upstream = OVERLAY / "ml" / ("upstream_" + fname)
        _relink(upstream, REFERENCE_ROOT / "ml" / fname)
        wrapper = OVERLAY / "ml" / fname
        wrapper.unlink()
        wrapper.write_text(text)
    _link_tree(REFERENCE_ROOT / "tests", OVERLAY / "tests", {})
    _link_tree(REFERENCE_ROOT / "examples", OVERLAY / "examples", {})
    _relink(OVERLAY / "external", REFERENCE_ROOT / "external")
    return OVERLAY


def _hipcc(args: list[str], what: str):
    r = subprocess.run([HIPCC, *args], capture_output=True, text=True)
    if r.returncode != 0:
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
        raise RuntimeError(f"{what} failed:\n{err[-6000:]}")


def build_host(force: bool = False, jobs: int = 6):
    """Compile the Matrix<ROCMfloat> mirror and the reference's ROCm programs.
    Returns the list of binaries, or [] when the reference tree is absent."""
    if not REFERENCE_ROOT.exists():
        return [*(sorted(REF_BIN.glob("*")) if REF_BIN.exists() else []), *(sorted(BIN.glob("*")) if BIN.exists() else [])]
    build()
    ov = make_overlay()
    REF_BIN.mkdir(parents=True, exist_ok=True)
    BIN.mkdir(parents=True, exist_ok=True)
    hostobj = OBJ / "host"
    hostobj.mkdir(parents=True, exist_ok=True)
    ours = [HOST_SRC / n for n in sorted(OURS)] + list(HOST_SRC.glob("*.hpp"))

    def compile_one(rel: str) -> Path:
        src = ov / rel
        obj = hostobj / (Path(rel).stem + ".o")
        if force or _stale(obj, [src.resolve(), *ours, ROOT / "include" / "jzhip.h"]):
            _hipcc([*HOST_FLAGS, "-c", str(src), "-o", str(obj)], f"compile {rel}")
        return obj

    lib_srcs = ["cpp/launcher.cu", "cpp/hipmatrix.cpp", "cpp/hipkernels.cpp"]
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        lib_objs = list(ex.map(compile_one, lib_srcs))
        prog_objs = list(ex.map(compile_one, REFERENCE_PROGRAMS))
    # the benchmark-configuration harness, once per backend
    cfg_src = PKG / "harness" / "configs.cu"
    cfg_obj = hostobj / "configs_rocm.o"
    if force or _stale(cfg_obj, [cfg_src, *ours, ROOT / "include" / "jzhip.h"]):
        _hipcc([*HOST_FLAGS, f"-I{ov / 'tests'}", "-c", str(cfg_src), "-o", str(cfg_obj)], "compile configs.cu (rocm)")
    # transpose-flag / ownership semantics of the mirror against Matrix<float>, one binary
    sem_src = PKG / "harness" / "semantics.cu"
    sem_obj = hostobj / "semantics_rocm.o"
    if force or _stale(sem_obj, [sem_src, *ours, ROOT / "include" / "jzhip.h"]):
        _hipcc([*HOST_FLAGS, f"-I{ov / 'tests'}", "-c", str(sem_src), "-o", str(sem_obj)], "compile semantics.cu")
    # the character LM written with the reference's own layer classes (drop-in API measurement)
    dro_src = PKG / "harness" / "lm_dropin.cu"
    dro_obj = hostobj / "lm_dropin_rocm.o"
    if force or _stale(dro_obj, [dro_src, *ours, ROOT / "include" / "jzhip.h"]):
        _hipcc([*HOST_FLAGS, f"-I{ov / 'tests'}", "-c", str(dro_src), "-o", str(dro_obj)], "compile lm_dropin.cu")
    # forward-mode tangents on the device against the CPU (the reference's testJVP skips on ROCm)
    jvp_src = PKG / "harness" / "jvp_check.cu"
    jvp_obj = hostobj / "jvp_check_rocm.o"
    if force or _stale(jvp_obj, [jvp_src, *ours, ROOT / "include" / "jzhip.h"]):
        _hipcc([*HOST_FLAGS, f"-I{ov / 'tests'}", "-c", str(jvp_src), "-o", str(jvp_obj)], "compile jvp_check.cu")
    # timing of the header templates elemwise<F> / reduce<F>
    tpl_src = PKG / "harness" / "templates_bench.cu"
    tpl_obj = hostobj / "templates_bench_rocm.o"
    if force or _stale(tpl_obj, [tpl_src, *ours, ROOT / "include" / "jzhip.h"]):
        _hipcc([*HOST_FLAGS, f"-I{ov / 'tests'}", "-c", str(tpl_src), "-o", str(tpl_obj)], "compile templates_bench.cu")
    harness_programs = [("configs_rocm", cfg_obj), ("templates_bench_rocm", tpl_obj), ("jvp_check_rocm", jvp_obj),
                        ("semantics_rocm", sem_obj), ("lm_dropin_rocm", dro_obj)]
    cpu_bin = REF_BIN / "configs_cpu"
    if force or _stale(cpu_bin, [cfg_src]):
        blas = sorted(Path("/usr/local/lib").glob("python3*/dist-packages/scipy.libs/libscipy_openblas*.so"))
        cmd = ["g++", "-std=c++20", "-O2", "-x", "c++", "-DLOGGING_OFF", f'-DPROJECT_DIR="{PROJECT_DIR}"', "-w",
               f"-I{REFERENCE_ROOT}", f"-I{REFERENCE_ROOT / 'tests'}"]
        if blas:   # the reference's default CBLAS configuration (cpp/helper.hpp:190-250)
            cmd += [f"-I{REFERENCE_ROOT / 'external' / 'OpenBLAS' / 'include'}"] + \
                   [f"-Dcblas_{f}=scipy_cblas_{f}" for f in ("sgemm", "dgemm", "sgemv", "dgemv")]
        else:      # BLAS-free configuration (cpp/cpulinalg.hpp)
            cmd += ["-DJUZHEN_NO_BLAS", "-ffp-contract=off"]
        cmd += [str(REFERENCE_ROOT / "cpp" / "launcher.cu"), str(cfg_src), "-o", str(cpu_bin)]
        if blas:
            cmd += ["-x", "none", str(blas[0]), f"-Wl,-rpath,{blas[0].parent}"]
        r = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
        if r.returncode != 0:
            raise RuntimeError(f"configs.cu (cpu) failed:\n{r.stderr[-4000:]}")
    bins = [cpu_bin]
    links = [(REF_BIN / Path(rel).stem, obj, "$ORIGIN/../../../juzhen_amd/lib") for rel, obj in zip(REFERENCE_PROGRAMS, prog_objs)]
    links += [(BIN / name, obj, "$ORIGIN/../lib") for name, obj in harness_programs]
    for out, obj, rpath in links:
        if force or _stale(out, [obj, *lib_objs, LIB]):
            _hipcc(["--offload-arch=gfx950", "-o", str(out), str(obj), *map(str, lib_objs),
                    f"-L{LIB.parent}", "-ljzhip", f"-Wl,-rpath,{rpath}"],
                   f"link {out.name}")
        bins.append(out)
    # earlier builds wrote the harness programs beside the reference's tests
    for name, _ in harness_programs:
        stale = REF_BIN / name
        if stale.exists():
            stale.unlink()
    return bins


# ── model harness (host C++ on the C ABI) ──────────────────────────────────────
HARNESS_LIB = PKG / "lib" / "libjzlm.so"


def build_harness(force: bool = False) -> Path:
    """Compile the train-step harness library (plain host C++, links libjzhip)."""
    build()
    srcs = sorted((PKG / "harness").glob("*.cpp"))
    if force or _stale(HARNESS_LIB, [*srcs, LIB, ROOT / "include" / "jzhip.h"]):
        cmd = ["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-fvisibility=hidden",
               f"-I{ROOT / 'include'}", "-o", str(HARNESS_LIB), *map(str, srcs),
               f"-L{LIB.parent}", "-ljzhip", "-Wl,-rpath,$ORIGIN"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"harness build failed:\n{r.stderr}")
    return HARNESS_LIB


if __name__ == "__main__":
    path = build(force="--force" in sys.argv)
    print(path)
    print(build_harness(force="--force" in sys.argv))
    if "--host" in sys.argv:
        for b in build_host(force="--force" in sys.argv):
            print(b)
