"""Build libslora_hip.so (HIP kernels + C ABI) for gfx950 with hipcc.

Usage: ``python s-lora_amd/build.py``.  The library lands in
``s-lora_amd/lib/`` next to the sources, so it travels with the tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libslora_hip.so")

SOURCES = ["cabi.hip", "bgmv_decode.hip", "sgmm_prefill.hip", "pool_ops.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 VALU forms are kept off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; libslora_hip.so cannot be built")


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{out}")
    if verbose and out.strip():
        print(out, flush=True)


def build_library(verbose: bool = True) -> str:
    """Compile every source to an object (in parallel, one hipcc each), then link."""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    hipcc = hipcc_path()
    inc = ["-I", os.path.join(ROOT, "include"), "-I", CSRC]
    jobs = []
    for s in SOURCES:
        obj = os.path.join(obj_dir, os.path.splitext(s)[0] + ".o")
        jobs.append((obj, [hipcc, *HIPCC_FLAGS, *inc, "-c", os.path.join(CSRC, s), "-o", obj]))
    with ThreadPoolExecutor(max_workers=min(len(jobs), 8)) as pool:
        list(pool.map(lambda j: _run(j[1], verbose), jobs))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *[j[0] for j in jobs], "-o", LIB_PATH], verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
    sys.exit(0)
