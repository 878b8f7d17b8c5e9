"""The four operators through the raw C ABI on the GPU, with no PyTorch in the call path: device
memory comes from the HIP runtime (libamdhip64 through ctypes), the entry points of
include/slora_hip.h are called with plain device pointers through tests/cabi_ctypes.py, and the
results are compared with the oracle at rtol 1e-2 / atol 1e-3.  This is the surface a non-Python
caller binds (the reference's own: slora/csrc/lora_ops.cc:76-126)."""
import ctypes as C

import numpy as np
import pytest

from lora_cases import make_case, make_segments
from oracle import lora_oracle as O

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-2, 1e-3
H2D, D2H = 1, 2  # hipMemcpyHostToDevice, hipMemcpyDeviceToHost


class Hip:
    """The handful of HIP runtime calls the test needs."""

    def __init__(self):
        self.rt = C.CDLL("libamdhip64.so")
        self.rt.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        self.rt.hipFree.argtypes = [C.c_void_p]
        self.rt.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        self.rt.hipMemset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        n = C.c_int(0)
        if self.rt.hipGetDeviceCount(C.byref(n)) != 0 or n.value < 1:
            pytest.skip("no GPU")
        assert self.rt.hipSetDevice(0) == 0
        self.owned = []

    def upload(self, a: np.ndarray) -> int:
        a = np.ascontiguousarray(a)
        p = C.c_void_p()
        assert self.rt.hipMalloc(C.byref(p), max(a.nbytes, 16)) == 0
        self.owned.append(p)
        assert self.rt.hipMemcpy(p, a.ctypes.data_as(C.c_void_p), a.nbytes, H2D) == 0
        return p.value

    def download(self, ptr: int, shape, dtype) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert self.rt.hipDeviceSynchronize() == 0
        assert self.rt.hipMemcpy(out.ctypes.data_as(C.c_void_p), C.c_void_p(ptr), out.nbytes, D2H) == 0
        return out

    def close(self):
        self.rt.hipDeviceSynchronize()
        for p in self.owned:
            self.rt.hipFree(p)
        self.owned = []


@pytest.fixture(scope="module")
def hip():
    h = Hip()
    yield h
    h.close()


def to_bits(a, dtype):
    """float32 values representable in `dtype` -> the 16-bit patterns the kernels read"""
    a = np.ascontiguousarray(a, dtype=np.float32)
    if dtype == "f16":
        return a.astype(np.float16).view(np.uint16)
    return (a.view(np.uint32) >> 16).astype(np.uint16)


def from_bits(u, dtype):
    if dtype == "f16":
        return u.view(np.float16).astype(np.float32)
    return (u.astype(np.uint32) << 16).view(np.float32)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_decode_operators_through_the_c_abi(hip, dtype):
    import cabi_ctypes as A
    lib = A.load_library()
    ranks = [64, 32, 16, 8, 8]
    H, batch, R = 1024, 37, 64
    c = make_case(21, H, ranks, batch, dtype=dtype, zipf_alpha=1.0)
    dt = A.DTYPE_F16 if dtype == "f16" else A.DTYPE_BF16
    key, val = hip.upload(to_bits(c.key, dtype)), hip.upload(to_bits(c.value, dtype))
    tables = A.SloraTables(hip.upload(c.a_start.astype(np.int64)), hip.upload(c.a_len.astype(np.int64)),
                           hip.upload(c.a_loc.astype(np.int64)), len(ranks), int(c.a_loc.size))
    bins = hip.upload(c.bins.astype(np.int64))
    scales = hip.upload(c.scales.astype(np.float16))           # the table is fp16 whatever the data type
    x = hip.upload(to_bits(c.x, dtype))
    for p in range(4):
        delta = hip.upload(np.zeros((batch, R), np.uint16))
        print(f"c-abi decode {dtype} projection {p}", flush=True)
        rc = lib.slora_bgmv_shrink(delta, x, key, C.byref(tables), bins, batch, H, R, c.page_elems, c.n_pages, p, dt,
                                   None)
        assert rc == A.OK, A.strerror(rc)
        d_gpu = from_bits(hip.download(delta, (batch, R), np.uint16), dtype)
        d_ref = O.ref_bgmv_shrink(np.zeros((batch, R), np.float32), c.x, c.key, c.a_start, c.a_len, c.a_loc, c.bins, p,
                                  dtype)
        np.testing.assert_allclose(d_gpu, d_ref, rtol=RTOL, atol=ATOL)
        y0 = O.round_to(np.random.default_rng(p).standard_normal((batch, H)).astype(np.float32) * 0.25, dtype)
        y = hip.upload(to_bits(y0, dtype))
        rc = lib.slora_bgmv_expand(y, delta, val, C.byref(tables), bins, scales, A.DTYPE_F16, batch, R, H,
                                   c.page_elems, c.n_pages, p, dt, None)
        assert rc == A.OK, A.strerror(rc)
        y_gpu = from_bits(hip.download(y, (batch, H), np.uint16), dtype)
        y_ref = O.ref_bgmv_expand(y0, d_gpu, c.value, c.a_start, c.a_len, c.a_loc, c.bins, p, c.scales, dtype)
        # y0 + update rounds once at the magnitude of the operands, here as in the reference
        step = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(y0), np.abs(y_ref - y0)) + 1e-30)) - (10 if dtype == "f16" else 7))
        assert np.all(np.abs(y_gpu - y_ref) <= ATOL + RTOL * np.abs(y_ref) + step)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_prefill_operators_through_the_c_abi(hip, dtype):
    import cabi_ctypes as A
    lib = A.load_library()
    ranks = [64, 16, 8, 32]
    H, R = 512, 64
    start, lens, ids = make_segments(4, 9, 1, 90, len(ranks))
    T = int(lens.sum())
    c = make_case(22, H, ranks, T, dtype=dtype, bins=np.repeat(ids, lens))
    dt = A.DTYPE_F16 if dtype == "f16" else A.DTYPE_BF16
    key, val = hip.upload(to_bits(c.key, dtype)), hip.upload(to_bits(c.value, dtype))
    tables = A.SloraTables(hip.upload(c.a_start.astype(np.int64)), hip.upload(c.a_len.astype(np.int64)),
                           hip.upload(c.a_loc.astype(np.int64)), len(ranks), int(c.a_loc.size))
    st, ln, rq = hip.upload(start.astype(np.int32)), hip.upload(lens.astype(np.int32)), hip.upload(ids.astype(np.int64))
    scales = hip.upload(c.scales.astype(np.float16))
    x = hip.upload(to_bits(c.x, dtype))
    for p in range(4):
        o = hip.upload(np.full((T, R), 0x3c00, np.uint16))      # the operator writes every column up to max_rank
        print(f"c-abi prefill {dtype} projection {p}", flush=True)
        rc = lib.slora_sgmm_shrink(o, x, key, C.byref(tables), st, ln, rq, len(lens), int(lens.max()), T, H, R, H, H,
                                   R, c.n_pages, p, dt, None)
        assert rc == A.OK, A.strerror(rc)
        o_gpu = from_bits(hip.download(o, (T, R), np.uint16), dtype)
        o_ref = O.ref_prefill_shrink(np.ones((T, R), np.float32), c.x, c.key, c.a_loc, c.a_start, c.a_len, start, lens,
                                     ids, p, R, dtype)
        np.testing.assert_allclose(o_gpu, o_ref, rtol=RTOL, atol=ATOL)
        y = hip.upload(np.zeros((T, H), np.uint16))
        rc = lib.slora_sgmm_expand(y, o, val, C.byref(tables), scales, A.DTYPE_F16, st, ln, rq, len(lens),
                                   int(lens.max()), T, H, 0, R, R, H, H, c.n_pages, p, dt, None)
        assert rc == A.OK, A.strerror(rc)
        y_gpu = from_bits(hip.download(y, (T, H), np.uint16), dtype)
        y_ref = O.ref_prefill_expand(np.zeros((T, H), np.float32), o_gpu, c.value, c.scales, c.a_loc, c.a_start,
                                     c.a_len, start, lens, ids, p, R, dtype)
        np.testing.assert_allclose(y_gpu, y_ref, rtol=RTOL, atol=ATOL)


def test_a_plan_of_another_rank_cap_does_nothing_and_says_so(hip):
    """A planned launch that names another rank cap or batch than the plan was built for leaves its
    output alone and sets bit 0 of the plan's status word; the launch the plan was built for works
    and the word is 0 after a build.  The buffer is sized for the largest launch made with it: a
    launch reads its item records before it has seen the header."""
    import cabi_ctypes as A
    lib = A.load_library()
    ranks = [16, 8, 32]
    H, batch, R = 512, 9, 64
    c = make_case(23, H, ranks, batch, dtype="f16")
    key = hip.upload(to_bits(c.key, "f16"))
    tables = A.SloraTables(hip.upload(c.a_start.astype(np.int64)), hip.upload(c.a_len.astype(np.int64)),
                           hip.upload(c.a_loc.astype(np.int64)), len(ranks), int(c.a_loc.size))
    bins = hip.upload(c.bins.astype(np.int64))
    x = hip.upload(to_bits(c.x, "f16"))
    nbytes = lib.slora_bgmv_plan_bytes(batch, R)
    assert nbytes >= lib.slora_bgmv_plan_bytes(batch, 32) and nbytes >= lib.slora_bgmv_plan_bytes(batch - 1, R)
    plan = hip.upload(np.zeros(nbytes // 4, np.int32))
    status = C.c_int(-1)

    def shrink(n_tokens, rank_cap, delta):
        rc = lib.slora_bgmv_shrink_planned(plan, rank_cap, 0, 1, delta, None, None, x, key, C.byref(tables), bins,
                                           n_tokens, H, R, c.page_elems, c.n_pages, 0, A.DTYPE_F16, None)
        assert rc == A.OK, A.strerror(rc)

    for what, n_tokens, rank_cap in (("rank cap", batch, 32), ("batch", batch - 1, R)):
        assert lib.slora_bgmv_plan_build(plan, nbytes, C.byref(tables), bins, batch, R, c.n_pages, None) == A.OK
        assert lib.slora_plan_status(plan, C.byref(status), None) == A.OK and status.value == 0
        delta = hip.upload(np.full((batch, R), 0x3c00, np.uint16))
        print(f"c-abi planned shrink that names another {what}", flush=True)
        shrink(n_tokens, rank_cap, delta)
        assert np.all(hip.download(delta, (batch, R), np.uint16) == 0x3c00)
        assert lib.slora_plan_status(plan, C.byref(status), None) == A.OK and status.value == 1
    # the launch the plan was built for
    assert lib.slora_bgmv_plan_build(plan, nbytes, C.byref(tables), bins, batch, R, c.n_pages, None) == A.OK
    delta = hip.upload(np.zeros((batch, R), np.uint16))
    print("c-abi planned shrink with its own plan", flush=True)
    shrink(batch, R, delta)
    d_gpu = from_bits(hip.download(delta, (batch, R), np.uint16), "f16")
    d_ref = O.ref_bgmv_shrink(np.zeros((batch, R), np.float32), c.x, c.key, c.a_start, c.a_len, c.a_loc, c.bins, 0, "f16")
    np.testing.assert_allclose(d_gpu, d_ref, rtol=RTOL, atol=ATOL)
    assert lib.slora_plan_status(plan, C.byref(status), None) == A.OK and status.value == 0


def test_a_prefill_plan_of_another_batch_does_nothing_and_says_so(hip):
    """slora_sgmm_shrink_planned with the plan of another batch shape leaves its output alone and sets
    the plan's status word; with its own plan it gives the oracle's result and the word is 0."""
    import cabi_ctypes as A
    lib = A.load_library()
    ranks = [64, 16, 8, 32]
    H, R, dtype = 512, 64, "f16"
    start, lens, ids = make_segments(5, 6, 20, 90, len(ranks))
    T = int(lens.sum())
    c = make_case(24, H, ranks, T, dtype=dtype, bins=np.repeat(ids, lens))
    key = hip.upload(to_bits(c.key, dtype))
    tables = A.SloraTables(hip.upload(c.a_start.astype(np.int64)), hip.upload(c.a_len.astype(np.int64)),
                           hip.upload(c.a_loc.astype(np.int64)), len(ranks), int(c.a_loc.size))
    st, ln, rq = hip.upload(start.astype(np.int32)), hip.upload(lens.astype(np.int32)), hip.upload(ids.astype(np.int64))
    x = hip.upload(to_bits(c.x, dtype))
    nbytes = lib.slora_sgmm_plan_bytes()
    plan = hip.upload(np.zeros(nbytes // 4, np.int32))
    usable, status = C.c_int(0), C.c_int(-1)

    def build(n_req, max_len, n_tokens):
        rc = lib.slora_sgmm_plan_build(plan, nbytes, C.byref(tables), st, ln, rq, n_req, max_len, n_tokens, R,
                                       C.byref(usable), None)
        assert rc == A.OK and usable.value == 1

    def shrink(o):
        return lib.slora_sgmm_shrink_planned(plan, o, x, key, C.byref(tables), st, ln, rq, len(lens), int(lens.max()), T, H,
                                             R, H, H, R, c.n_pages, 0, A.DTYPE_F16, None)

    # a plan for the first request alone: another number of row parts than the launch below has
    build(1, int(lens[0]), int(lens[0]))
    assert lib.slora_plan_status(plan, C.byref(status), None) == A.OK and status.value == 0
    o = hip.upload(np.full((T, R), 0x3c00, np.uint16))
    print("c-abi planned prefill shrink with the plan of another batch", flush=True)
    assert shrink(o) == A.OK
    assert np.all(hip.download(o, (T, R), np.uint16) == 0x3c00)
    assert lib.slora_plan_status(plan, C.byref(status), None) == A.OK and status.value == 1
    build(len(lens), int(lens.max()), T)
    assert lib.slora_plan_status(plan, C.byref(status), None) == A.OK and status.value == 0
    print("c-abi planned prefill shrink with its own plan", flush=True)
    assert shrink(o) == A.OK
    o_gpu = from_bits(hip.download(o, (T, R), np.uint16), dtype)
    o_ref = O.ref_prefill_shrink(np.ones((T, R), np.float32), c.x, c.key, c.a_loc, c.a_start, c.a_len, start, lens, ids,
                                 0, R, dtype)
    np.testing.assert_allclose(o_gpu, o_ref, rtol=RTOL, atol=ATOL)
    assert lib.slora_plan_status(plan, C.byref(status), None) == A.OK and status.value == 0
