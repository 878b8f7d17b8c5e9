"""The entry point that allocates nothing, slora_pool_alloc_contiguous_static, against
slora_pool_alloc_contiguous (the same search with a caller-owned workspace), through the
C ABI.  Index work: start, page list and the map afterwards are compared bit for bit, on
two calls in a row that share the library's static workspace, the second on a smaller map.
"""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _random_map(rng, tot, run):
    """A map with free stretches of mixed lengths and at least one of `run` pages."""
    state = (rng.random(tot) < 0.55).astype(np.uint8)
    if tot >= run:
        at = int(rng.integers(tot // 2, tot - run + 1))
        state[at:at + run] = 1
        if at:
            state[at - 1] = 0
    return state


def _call(lib, fn_static, state_np, need, dev):
    import cabi_ctypes as _cabi
    state = torch.from_numpy(state_np.copy()).to(dev)
    out = torch.full((max(need, 1),), -7, dtype=torch.int64, device=dev)
    result = torch.full((2,), -9, dtype=torch.int64, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    tot = state.numel()
    if fn_static:
        rc = lib.slora_pool_alloc_contiguous_static(state.data_ptr(), tot, need, out.data_ptr(), result.data_ptr(), stream)
    else:
        nbytes = int(lib.slora_pool_alloc_workspace_bytes(tot))
        work = torch.empty((nbytes + 7) // 8, dtype=torch.int64, device=dev)
        rc = lib.slora_pool_alloc_contiguous(state.data_ptr(), tot, need, out.data_ptr(), result.data_ptr(),
                                             work.data_ptr(), stream)
    _cabi.check(rc, "alloc_contiguous")
    torch.cuda.synchronize()
    return state.cpu().numpy(), out.cpu().numpy(), result.cpu().numpy()


def test_static_workspace_allocator_equals_the_workspace_one(gpu):
    import cabi_ctypes as _cabi
    lib = _cabi.load_library()
    rng = np.random.default_rng(77)
    # a large map first (many workgroup entries of the workspace in use), then a smaller
    # one whose search must not see what the first call left behind, then no run at all
    cases = [(300000, 96), (9000, 40), (5000, 4000)]
    for tot, need in cases:
        state_np = _random_map(rng, tot, need if need < 1000 else 8)
        got = _call(lib, True, state_np, need, gpu)
        exp = _call(lib, False, state_np, need, gpu)
        for g, e, what in zip(got, exp, ("map", "pages", "result")):
            assert np.array_equal(g, e), (tot, need, what)
        if need < 1000:
            assert exp[2][0] >= 0 and exp[2][1] == need
        else:
            assert exp[2][0] == -1 and np.array_equal(got[0], state_np)


def test_static_workspace_allocator_rejects_maps_beyond_its_capacity(gpu):
    import cabi_ctypes as _cabi
    lib = _cabi.load_library()
    one = torch.ones(16, dtype=torch.uint8, device=gpu)
    out = torch.zeros(2, dtype=torch.int64, device=gpu)
    rc = lib.slora_pool_alloc_contiguous_static(one.data_ptr(), (1 << 24) + 1, 1, out.data_ptr(), out.data_ptr(), None)
    assert rc == _cabi.ERR_TOO_LARGE
    with pytest.raises(RuntimeError, match="capacity"):
        _cabi.check(rc, "slora_pool_alloc_contiguous_static")
