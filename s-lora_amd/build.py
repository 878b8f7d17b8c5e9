"""Build libslora_hip.so (HIP kernels + C ABI) for gfx950 with hipcc, and the
PyTorch extension ``slora_hip/_kernels*.so`` that calls it.

Usage: ``python s-lora_amd/build.py``.  Both land in the tree next to the
sources (``s-lora_amd/lib/`` and ``s-lora_amd/slora_hip/``), so they travel with it.
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

SOURCES = ["cabi.hip", "bgmv_decode.hip", "bgmv_lora.hip", "sgmm_prefill.hip", "pool_ops.hip"]

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


def extension_path() -> str:
    import sysconfig
    return os.path.join(HERE, "slora_hip", "_kernels" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_extension(verbose: bool = True) -> str:
    """Compile csrc/torch_ext.cpp (host code only: pybind11 + tensor checks + calls into
    the C ABI) against this interpreter's torch and link it to libslora_hip.so."""
    import sysconfig
    import torch
    from torch.utils import cpp_extension
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: build_library() first")
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    out = extension_path()
    cmd = [hipcc_path(), "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall",
           "-Wno-unused-function", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_kernels",
           "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           "-I", os.path.join(ROOT, "include"), "-I", sysconfig.get_paths()["include"]]
    for inc in cpp_extension.include_paths():
        cmd += ["-isystem", inc]
    cmd += [os.path.join(CSRC, "torch_ext.cpp"), "-o", out,
            "-L", torch_lib, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
            "-L", LIB_DIR, "-lslora_hip", "-Wl,-rpath,$ORIGIN/../lib", "-Wl,--no-as-needed"]
    _run(cmd, verbose)
    return out


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_extension(verbose=True))
    sys.exit(0)
