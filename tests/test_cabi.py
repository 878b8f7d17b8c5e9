"""The C ABI without a GPU: the library loads, exports every symbol that
include/slora_hip.h declares, and rejects bad arguments on the host before any
launch.  No compute call is made here."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    import cabi_ctypes as _cabi
    if not os.path.exists(_cabi.lib_path()):
        import importlib.util
        spec = importlib.util.spec_from_file_location("slora_build", os.path.join(ROOT, "s-lora_amd", "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build_library(verbose=False)
        mod.build_extension(verbose=False)
    return _cabi.load_library()


def declared_functions():
    text = open(os.path.join(ROOT, "include", "slora_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(slora_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree(lib):
    import cabi_ctypes as _cabi
    names = declared_functions()
    assert names == sorted(_cabi.SIGNATURES)
    for n in names:
        assert hasattr(lib, n), n


def test_version_and_strerror(lib):
    import cabi_ctypes as _cabi
    assert lib.slora_version() == 200
    assert _cabi.strerror(0) == "ok"
    assert "No suitable kernel" in _cabi.strerror(_cabi.ERR_UNSUPPORTED)
    for code in range(-7, 0):
        assert _cabi.strerror(code) != "unknown error"
    assert _cabi.strerror(-99) == "unknown error"


def _tables(ptr=0x1000):
    import cabi_ctypes as _cabi
    return _cabi.SloraTables(ptr, ptr, ptr, 4, 64)


def test_shrink_argument_checks(lib):
    import cabi_ctypes as A
    t = _tables()
    P = 0x10000  # never dereferenced: every call below fails validation or has nothing to do
    f = lib.slora_bgmv_shrink
    assert f(P, P, P, C.byref(t), P, 0, 4096, 64, 4096, 100, 0, A.DTYPE_F16, None) == A.OK          # empty batch
    assert f(P, P, P, C.byref(t), P, 8, 4096, 64, 4096, 100, 0, 7, None) == A.ERR_BAD_DTYPE
    assert f(P, P, P, C.byref(t), P, -1, 4096, 64, 4096, 100, 0, A.DTYPE_F16, None) == A.ERR_BAD_SHAPE
    assert f(P, P, P, C.byref(t), P, 8, 4096, 64, 4096, 100, 4, A.DTYPE_F16, None) == A.ERR_BAD_SHAPE
    assert f(None, P, P, C.byref(t), P, 8, 4096, 64, 4096, 100, 0, A.DTYPE_F16, None) == A.ERR_NULL_POINTER
    assert f(P, P, P, None, P, 8, 4096, 64, 4096, 100, 0, A.DTYPE_F16, None) == A.ERR_NULL_POINTER
    assert f(P, P, P, C.byref(t), None, 8, 4096, 64, 4096, 100, 0, A.DTYPE_F16, None) == A.ERR_NULL_POINTER
    assert f(P, P, P, C.byref(t), P, 8, 4100, 64, 4104, 100, 0, A.DTYPE_F16, None) == A.ERR_UNSUPPORTED  # h_in % 8
    assert f(P, P, P, C.byref(t), P, 8, 4096, 64, 2048, 100, 0, A.DTYPE_F16, None) == A.ERR_UNSUPPORTED  # row > page
    assert f(P, P, P, C.byref(t), P, 8, 4096, 1024, 4096, 100, 0, A.DTYPE_F16, None) == A.ERR_UNSUPPORTED  # rank cap
    assert f(P, P + 2, P, C.byref(t), P, 8, 4096, 64, 4096, 100, 0, A.DTYPE_F16, None) == A.ERR_ALIGNMENT
    assert f(P, P, P, C.byref(t), P, 8, 4096, 64, 4096, 0, 0, A.DTYPE_F16, None) == A.ERR_BAD_SHAPE      # empty pool


def test_expand_argument_checks(lib):
    import cabi_ctypes as A
    t = _tables()
    P = 0x10000
    f = lib.slora_bgmv_expand
    assert f(P, P, P, C.byref(t), P, P, A.DTYPE_F16, 0, 64, 4096, 4096, 100, 0, A.DTYPE_F16, None) == A.OK
    assert f(P, P, P, C.byref(t), P, P, 9, 8, 64, 4096, 4096, 100, 0, A.DTYPE_F16, None) == A.ERR_BAD_DTYPE
    assert f(P, P, P, C.byref(t), P, None, A.DTYPE_F16, 8, 64, 4096, 4096, 100, 0, A.DTYPE_F16, None) == A.ERR_NULL_POINTER
    assert f(P, P, P, C.byref(t), P, P, A.DTYPE_F16, 8, 64, 4096, 4100, 100, 0, A.DTYPE_F16, None) == A.ERR_UNSUPPORTED
    assert f(P, P, P, C.byref(t), P, P, A.DTYPE_F16, 8, 64, 4096, 4096, 100, -1, A.DTYPE_F16, None) == A.ERR_BAD_SHAPE
    assert f(P, P + 8, P, C.byref(t), P, P, A.DTYPE_F16, 8, 64, 4096, 4096, 100, 0, A.DTYPE_F16, None) == A.ERR_ALIGNMENT


def test_sgmm_argument_checks(lib):
    import cabi_ctypes as A
    t = _tables()
    P = 0x10000
    s = lib.slora_sgmm_shrink
    assert s(P, P, P, C.byref(t), P, P, P, 0, 0, 0, 4096, 64, 4096, 4096, 64, 100, 0, A.DTYPE_BF16, None) == A.OK
    assert s(P, P, P, C.byref(t), P, P, P, 4, 16, 64, 4096, 64, 4000, 4096, 64, 100, 0, A.DTYPE_BF16, None) == A.ERR_BAD_SHAPE
    assert s(P, P, P, C.byref(t), None, P, P, 4, 16, 64, 4096, 64, 4096, 4096, 64, 100, 0, A.DTYPE_BF16, None) == A.ERR_NULL_POINTER
    assert s(P, P, P, C.byref(t), P, P, P, 4, 16, 64, 4096, 64, 4096, 4096, 64, 100, 0, 3, None) == A.ERR_BAD_DTYPE
    assert s(P, P, P, C.byref(t), P, P, P, 4, 16, 64, 4096, 64, 4096, 4096, 64, 0, 0, A.DTYPE_BF16, None) == A.ERR_BAD_SHAPE
    e = lib.slora_sgmm_expand
    assert e(P, P, P, C.byref(t), P, A.DTYPE_F16, P, P, P, 0, 0, 0, 4096, 4096, 64, 64, 4096, 4096, 100, 0, A.DTYPE_F16, None) == A.OK
    assert e(P, P, P, C.byref(t), None, A.DTYPE_F16, P, P, P, 4, 16, 64, 4096, 4096, 64, 64, 4096, 4096, 100, 0, A.DTYPE_F16, None) == A.ERR_NULL_POINTER
    assert e(P, P, P, C.byref(t), P, A.DTYPE_F16, P, P, P, 4, 16, 64, 4096, 4096, 64, 32, 4096, 4096, 100, 0, A.DTYPE_F16, None) == A.ERR_BAD_SHAPE
    # q, k and v in one launch: o_q o_k o_v x_q x_k x_v w tables scales scales_dtype b_start_loc b_seq_len b_indicies
    # n_requests max_input_len n_tokens feat_out_q feat_out_kv page_elems max_rank x_stride w_stride o_stride_q o_stride_kv n_pages dtype stream
    f = lib.slora_sgmm_expand_qkv
    head = (P, P, P, P, P, P, P, C.byref(t), P, A.DTYPE_F16, P, P, P)
    assert f(*head, 0, 0, 0, 4096, 1024, 4096, 64, 64, 4096, 4096, 1024, 100, A.DTYPE_F16, None) == A.OK
    assert f(*head, 4, 16, 64, 4096, 1024, 4096, 64, 64, 4096, 4096, 512, 100, A.DTYPE_F16, None) == A.ERR_BAD_SHAPE   # o_k rows narrower than feat_out_kv
    assert f(*head, 4, 16, 64, 4096, 1024, 4096, 64, 32, 4096, 4096, 1024, 100, A.DTYPE_F16, None) == A.ERR_BAD_SHAPE  # x rows narrower than max_rank
    assert f(*head, 4, 16, 64, 4096, 1024, 4096, 64, 64, 4096, 4096, 1024, 100, 9, None) == A.ERR_BAD_DTYPE
    assert f(P, None, P, P, P, P, P, C.byref(t), P, A.DTYPE_F16, P, P, P, 4, 16, 64, 4096, 1024, 4096, 64, 64, 4096, 4096,
             1024, 100, A.DTYPE_F16, None) == A.ERR_NULL_POINTER


def test_python_mirror_rejects_cpu_tensors():
    """Reference behaviour: CHECK_CUDA -> RuntimeError (lora_ops.cc:29, 79-85)."""
    import torch
    from slora_hip import dispatch_bgmv, lora_get_qkvo_fwd_shrink
    y = torch.zeros(2, 8, dtype=torch.float16)
    x = torch.zeros(2, 64, dtype=torch.float16)
    w = torch.zeros(32, 4, 16, dtype=torch.float16)
    i64 = torch.zeros(2, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        dispatch_bgmv(y, x, w, i64, i64, i64, i64, 0, torch.ones(2, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        lora_get_qkvo_fwd_shrink(x, w.view(32, 64), y, i64, i64, i64, i64.int(), i64.int(), i64, 64, 0, 8, 4)
