"""Builds the HIP library in-tree: csrc/*.hip -> lib/libgemmzoo.so (gfx950 only).

Run as a script (``python gemm-zoo_amd/build.py``) or through ``build_all()``.
The comparator that wraps hipBLASLt is a separate shared object so that the
product library depends on the HIP runtime alone.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
LIB = HERE / "lib"
OBJ = HERE / "build"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# packed fp32 VALU instructions are switched off for every translation unit
COMMON = [
    "-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    "-Wno-option-ignored", "-Wno-unused-function",
]

PRODUCT_SOURCES = [
    "gz_api.hip", "gz_fill_compare.hip", "rung0_naive.hip", "rung1_coalesced.hip",
    "rung23_lds.hip", "rung4_mfma_s8s8s32.hip", "rung4_mfma_bf16bf16f32.hip", "rung4_mfma_bf16bf16bf16.hip",
    "rung4_mfma_f16f16f16.hip", "rung4_mfma_f32f32f32.hip", "rung4_mfma_e4m3e4m3f16.hip",
    "rung4_mfma_e5m2e5m2f16.hip", "rung4_mfma_acc16.hip", "rung5_skinny.hip",
]
COMPARATOR_SOURCES = ["gz_hipblaslt.cpp"]


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    out = (proc.stdout + proc.stderr)
    # the host pass does not know the device-only target feature; that note is harmless
    out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(map(str, cmd)), out))
    return out


def _compile(src: Path, extra=()):
    OBJ.mkdir(exist_ok=True)
    obj = OBJ / (src.stem + ".o")
    cmd = [HIPCC, *COMMON, *extra, "-c", str(src), "-o", str(obj)]
    if src.suffix == ".cpp":
        cmd.insert(1, "-x")
        cmd.insert(2, "hip")
    out = _run(cmd)
    return obj, out


def build_product(verbose=True, jobs=8):
    LIB.mkdir(exist_ok=True)
    srcs = [CSRC / s for s in PRODUCT_SOURCES]
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(_compile, srcs))
    objs = [str(o) for o, _ in results]
    if verbose:
        for _, out in results:
            if out.strip():
                print(out)
    target = LIB / "libgemmzoo.so"
    _run([HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", str(target), *objs])
    return target


def build_comparator(verbose=True):
    LIB.mkdir(exist_ok=True)
    srcs = [CSRC / s for s in COMPARATOR_SOURCES if (CSRC / s).exists()]
    if not srcs:
        return None
    objs = []
    for s in srcs:
        o, out = _compile(s)
        objs.append(str(o))
        if verbose and out.strip():
            print(out)
    target = LIB / "libgemmzoo_hipblaslt.so"
    _run([HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", str(target), *objs,
          "-L/opt/rocm/lib", "-lhipblaslt", "-Wl,-rpath,/opt/rocm/lib"])
    return target


def build_benches(verbose=True, jobs=8):
    """The C++ drivers under bench/ (gemm-zoo's bench mains on the functor surface) -> bench/bin/."""
    bench_dir = HERE / "bench"
    out_dir = bench_dir / "bin"
    out_dir.mkdir(exist_ok=True)
    include = HERE.parent / "include"

    def one(src: Path):
        exe = out_dir / src.stem
        _run([HIPCC, "-O2", "-std=c++17", "-x", "hip", f"--offload-arch={ARCH}", "-Wno-unused-command-line-argument",
              "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
              f"-I{include}", str(src), "-o", str(exe), f"-L{LIB}", "-lgemmzoo", "-lgemmzoo_hipblaslt",
              "-Wl,-rpath,$ORIGIN/../../lib", "-Wl,-rpath,/opt/rocm/lib"])
        return exe

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        return list(ex.map(one, sorted(bench_dir.glob("*.cpp"))))


def build_all(verbose=True):
    out = [build_product(verbose)]
    cmp_lib = build_comparator(verbose)
    if cmp_lib:
        out.append(cmp_lib)
        out.extend(build_benches(verbose))
    return out


if __name__ == "__main__":
    for t in build_all():
        print("built", t)
    sys.exit(0)
