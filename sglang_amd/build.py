"""Build recipe for libsglq.so and libsglq_bench.so (hipcc, gfx950 only).

``python -m sglang_amd.build`` compiles the operator sources under ``csrc/`` into
``sglang_amd/libsglq.so`` (plain C ABI, ``include/sglq.h``; does not link against torch) and
the measurement kernels (``csrc/bench_kernels.hip``: MFMA ceiling loop, clock probe, streaming
passes) into ``sglang_amd/libsglq_bench.so``, which only ``bench.py`` loads.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libsglq.so"
BENCH_LIB_PATH = PKG_DIR / "libsglq_bench.so"
SOURCES = ["common.hip", "quant.hip", "moe.hip", "gemm.hip"]
BENCH_SOURCES = ["bench_kernels.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # packed-FP32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def build(verbose: bool = False, jobs: int = 4) -> Path:
    hipcc = find_hipcc()
    obj_dir = PKG_DIR / "build"
    obj_dir.mkdir(exist_ok=True)
    procs = []
    objs = []
    bench_objs = []
    for src in SOURCES + BENCH_SOURCES:
        obj = obj_dir / (src + ".o")
        (bench_objs if src in BENCH_SOURCES else objs).append(str(obj))
        cmd = [hipcc, *HIPCC_FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs, verbose)
    _drain(procs, verbose)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", str(LIB_PATH), *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if out.returncode != 0:
        raise RuntimeError("link failed:\n" + out.stdout)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", str(BENCH_LIB_PATH), *bench_objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if out.returncode != 0:
        raise RuntimeError("link of the measurement kernels failed:\n" + out.stdout)
    return LIB_PATH


def _drain(procs, verbose):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        noise = "is not a recognized feature for this target"
        text = "\n".join(l for l in out.splitlines() if noise not in l)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{text}")
        if verbose and text.strip():
            print(text)


if __name__ == "__main__":
    path = build(verbose=True)
    print(f"built {path}")
    sys.exit(0)
