"""ctypes binding of libslora_hip.so (the declarations of include/slora_hip.h), for the tests
that call the C ABI directly.  The product binds the same functions from C++
(s-lora_amd/csrc/torch_ext.cpp)."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(os.path.dirname(_HERE), "s-lora_amd", "lib", "libslora_hip.so")

DTYPE_F16, DTYPE_BF16, DTYPE_F32 = 0, 1, 2
MAX_RANK = 512  # SLORA_MAX_RANK of include/slora_hip.h

OK = 0
ERR_NULL_POINTER, ERR_BAD_DTYPE, ERR_BAD_SHAPE, ERR_UNSUPPORTED, ERR_ALIGNMENT, ERR_LAUNCH, ERR_TOO_LARGE = \
    -1, -2, -3, -4, -5, -6, -7


class SloraTables(C.Structure):
    _fields_ = [
        ("a_start", C.c_void_p),
        ("a_len", C.c_void_p),
        ("a_loc", C.c_void_p),
        ("n_adapters", C.c_int64),
        ("n_loc", C.c_int64),
    ]


_P, _I64, _I = C.c_void_p, C.c_int64, C.c_int
_TP = C.POINTER(SloraTables)

# name -> (restype, argtypes); mirrors include/slora_hip.h one to one
SIGNATURES = {
    "slora_version": (_I, []),
    "slora_strerror": (C.c_char_p, [_I]),
    "slora_bgmv_shrink": (_I, [_P, _P, _P, _TP, _P, _I64, _I64, _I64, _I64, _I64, _I, _I, _P]),
    "slora_bgmv_expand": (_I, [_P, _P, _P, _TP, _P, _P, _I, _I64, _I64, _I64, _I64, _I64, _I, _I, _P]),
    "slora_bgmv_shrink_qkv": (_I, [_P, _P, _P, _P, _P, _TP, _P, _I64, _I64, _I64, _I64, _I64, _I, _P]),
    "slora_bgmv_expand_qkv": (_I, [_P, _P, _P, _P, _P, _P, _P, _TP, _P, _P, _I, _I64, _I64, _I64, _I64, _I64,
                                   _I64, _I64, _I, _P]),
    "slora_bgmv_plan_bytes": (_I64, [_I64, _I64]),
    "slora_plan_status": (_I, [_P, C.POINTER(C.c_int), _P]),
    "slora_bgmv_plan_build": (_I, [_P, _I64, _TP, _P, _I64, _I64, _I64, _P]),
    "slora_bgmv_shrink_planned": (_I, [_P, _I64, _I64, _I, _P, _P, _P, _P, _P, _TP, _P, _I64, _I64, _I64, _I64, _I64,
                                       _I, _I, _P]),
    "slora_bgmv_expand_planned": (_I, [_P, _I64, _I64, _I, _P, _P, _P, _P, _P, _P, _P, _TP, _P, _P, _I, _I64, _I64,
                                       _I64, _I64, _I64, _I64, _I64, _I, _I, _P]),
    "slora_bgmv_lora_planned": (_I, [_P, _I64, _I64, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _TP, _P, _P, _I, _I64, _I64,
                                     _I64, _I64, _I64, _I64, _I64, _I64, _I, _I, _P]),
    "slora_sgmm_shrink": (_I, [_P, _P, _P, _TP, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64,
                               _I, _I, _P]),
    "slora_sgmm_plan_bytes": (_I64, []),
    "slora_sgmm_plan_build": (_I, [_P, _I64, _TP, _P, _P, _P, _I64, _I64, _I64, _I64, C.POINTER(C.c_int), _P]),
    "slora_sgmm_shrink_planned": (_I, [_P, _P, _P, _P, _TP, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64,
                                       _I64, _I, _I, _P]),
    "slora_sgmm_shrink_qkv": (_I, [_P, _P, _P, _P, _P, _P, _TP, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64,
                                   _I64, _I64, _I, _P]),
    "slora_sgmm_expand": (_I, [_P, _P, _P, _TP, _P, _I, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64,
                               _I64, _I64, _I, _I, _P]),
    "slora_sgmm_expand_qkv": (_I, [_P, _P, _P, _P, _P, _P, _P, _TP, _P, _I, _P, _P, _P, _I64, _I64, _I64, _I64, _I64,
                                   _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I, _P]),
    "slora_pool_scatter_rows": (_I, [_P, _P, _I, _P, _I64, _I64, _I64, _I64, _I64, _P]),
    "slora_pool_pack_transposed": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _P, _I64, _I64, _I64, _P]),
    "slora_var_len_copy": (_I, [_P, _P, _P, _P, _P, _I64, _I64, _I64, _P]),
    "slora_tables_compact": (_I, [_TP, _P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P]),
    "slora_pool_gather_a": (_I, [_P, _I64, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _P]),
    "slora_pool_alloc_workspace_bytes": (_I64, [_I64]),
    "slora_pool_alloc": (_I, [_P, _I64, _I64, _P, _P, _P, _P]),
    "slora_pool_alloc_contiguous": (_I, [_P, _I64, _I64, _P, _P, _P, _P]),
    "slora_pool_alloc_contiguous_static": (_I, [_P, _I64, _I64, _P, _P, _P]),
    "slora_pool_free": (_I, [_P, _I64, _P, _I64, _P]),
    "slora_pool_page_checksums": (_I, [_P, _P, _P, _I64, _I64, _I64, _P]),
    "slora_pool_page_xor": (_I, [_P, _P, _I64, _I64, _I64, C.c_uint32, _P]),
}

_lib = None


def lib_path() -> str:
    return _LIB_PATH


def load_library():
    """Load libslora_hip.so and set every prototype.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError(
            f"{_LIB_PATH} is missing: build it with `python s-lora_amd/build.py` "
            "(there is no non-HIP fallback for the LoRA kernels)")
    lib = C.CDLL(_LIB_PATH)
    missing = [name for name in SIGNATURES if not hasattr(lib, name)]
    if missing:
        raise RuntimeError(f"{_LIB_PATH} does not export {missing}: rebuild it with `python s-lora_amd/build.py`")
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def version() -> int:
    return int(load_library().slora_version())


def strerror(code: int) -> str:
    return load_library().slora_strerror(int(code)).decode()


def check(code: int, what: str, detail: str = "") -> None:
    """Turn a non-zero return code into the RuntimeError the reference's
    TORCH_CHECK would have raised."""
    if code != OK:
        raise RuntimeError(f"{what}: {strerror(code)}{(' ' + detail) if detail else ''}")
