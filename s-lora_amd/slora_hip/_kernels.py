"""Decode-time operator surface: ``dispatch_bgmv`` with the reference's exact
positional signature (slora/csrc/lora_ops.cc:76-78, 135), bound to the HIP
kernels of libslora_hip.so.

Call-compatible with ``from slora._kernels import dispatch_bgmv`` as used by
slora/models/peft/lora_unordered_batch_infer.py:267-273 and
test/kernel/test_kernel_correctness*.py.  Checks and messages follow the
reference's TORCH_CHECKs (lora_ops.cc:13-42, 79-96, 124); every failure is a
``RuntimeError``.  Checks the reference does not make (index dtypes, the
scaling table, the pool's page width) are added because a wrong one would be a
device fault here.
"""
from __future__ import annotations

import ctypes as C
import os
import weakref

import torch

from . import _cabi

_DTYPE_CODE = {torch.float16: _cabi.DTYPE_F16, torch.bfloat16: _cabi.DTYPE_BF16, torch.float32: _cabi.DTYPE_F32}


def _check_input(t, name: str) -> None:
    if not isinstance(t, torch.Tensor):
        raise RuntimeError(f"{name} must be a tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _check_dim(d: int, t, name: str) -> None:
    if t.dim() != d:
        raise RuntimeError(f"{name} must be a {d}D tensor")


def _check_index(t, name: str) -> None:
    if t.dtype != torch.int64:
        raise RuntimeError(f"{name} must be an int64 tensor, got {t.dtype}")


def _tables(start_indicies, lora_ranks, loc_indicies) -> _cabi.SloraTables:
    return _cabi.SloraTables(start_indicies.data_ptr(), lora_ranks.data_ptr(), loc_indicies.data_ptr(),
                             start_indicies.numel(), loc_indicies.numel())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t) -> int:
    """The current stream of ``t``'s device as a raw handle (the fast private
    accessor when this torch has it: the public one builds a Stream object)."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index if t.device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


def _validate_common(w, start_indicies, lora_ranks, loc_indicies, indicies, lora_scales=None):
    _check_input(w, "w")
    _check_input(start_indicies, "start_indicies")
    _check_input(lora_ranks, "lora_ranks")
    _check_input(loc_indicies, "loc_indicies")
    _check_input(indicies, "indicies")
    _check_dim(3, w, "w")
    _check_dim(1, indicies, "indicies")
    for t, n in ((start_indicies, "start_indicies"), (lora_ranks, "lora_ranks"), (loc_indicies, "loc_indicies"),
                 (indicies, "indicies")):
        _check_index(t, n)
    if start_indicies.numel() != lora_ranks.numel():
        raise RuntimeError(f"CHECK_EQ(start_indicies.size(0), lora_ranks.size(0)) failed. "
                           f"{start_indicies.numel()} vs {lora_ranks.numel()}")
    if lora_scales is not None:
        _check_input(lora_scales, "lora_scales")
        if lora_scales.dtype not in _DTYPE_CODE:
            raise RuntimeError(f"lora_scales must be float16, bfloat16 or float32, got {lora_scales.dtype}")
        if lora_scales.numel() < start_indicies.numel():
            raise RuntimeError(f"CHECK_EQ(lora_scales.size(0), start_indicies.size(0)) failed. "
                               f"{lora_scales.numel()} vs {start_indicies.numel()}")


class BgmvPlan:
    """Device-side list of the batch's runs (tokens that share an adapter) and
    their page ids, built once per decode step and passed as ``plan=`` to the
    ``dispatch_bgmv*`` calls of that step.  Valid while ``indicies`` and the
    adapter tables keep their contents."""

    def __init__(self, buf, rank_cap, batch, n_items=0, max_rank=0, n_runs=0):
        self.buf = buf
        self.rank_cap = int(rank_cap)
        self.batch = int(batch)
        self.n_items = int(n_items)    # 0 = not read back: launches are sized for the plan's capacity
        self.max_rank = int(max_rank)
        self.n_runs = int(n_runs)


def rebuild_plan(plan, start_indicies, lora_ranks, loc_indicies, indicies, n_pages) -> None:
    """Enqueue a rebuild of ``plan`` in place for a batch of the same size (no
    allocation, no synchronisation; the item count on the host is left as it
    is, so use it only when the caller knows the count or left it at 0)."""
    lib = _cabi.load_library()
    if indicies.numel() != plan.batch:
        raise RuntimeError(f"plan was built for {plan.batch} tokens, this batch has {indicies.numel()}")
    tables = _tables(start_indicies, lora_ranks, loc_indicies)
    rc = lib.slora_bgmv_plan_build(plan.buf.data_ptr(), plan.buf.numel() * 4, C.byref(tables), indicies.data_ptr(),
                                   plan.batch, plan.rank_cap, int(n_pages), _stream(indicies))
    _cabi.check(rc, "rebuild_plan")


def make_plan(start_indicies, lora_ranks, loc_indicies, indicies, rank_cap, n_pages, readback=True) -> BgmvPlan:
    """Build the plan for one batch.  ``rank_cap`` is the width of the shrink
    outputs (``max_lora_dim`` of lora_unordered_batch_infer.py:21-22),
    ``n_pages`` the number of pages of the pool buffers.  ``readback=True``
    copies the item count to the host (one synchronisation per step) so later
    launches have exactly one workgroup per item."""
    for t, n in ((start_indicies, "start_indicies"), (lora_ranks, "lora_ranks"), (loc_indicies, "loc_indicies"),
                 (indicies, "indicies")):
        _check_input(t, n)
        _check_index(t, n)
    lib = _cabi.load_library()
    batch = indicies.numel()
    nbytes = lib.slora_bgmv_plan_bytes(batch, int(rank_cap))
    if nbytes < 0:
        _cabi.check(int(nbytes), "make_plan", f"(batch={batch} rank_cap={rank_cap})")
    buf = torch.empty((max(int(nbytes), 64) + 3) // 4, dtype=torch.int32, device=indicies.device)
    tables = _tables(start_indicies, lora_ranks, loc_indicies)
    rc = lib.slora_bgmv_plan_build(buf.data_ptr(), buf.numel() * 4, C.byref(tables), indicies.data_ptr(), batch,
                                   int(rank_cap), int(n_pages), _stream(indicies))
    _cabi.check(rc, "make_plan")
    plan = BgmvPlan(buf, rank_cap, batch)
    if readback and batch > 0:
        head = buf[:8].cpu()
        plan.n_items, plan.max_rank, plan.n_runs = int(head[1]), int(head[2]), int(head[6])
    return plan


class _PlanCache:
    """Plans built on behalf of callers that pass none.  The reference's engine
    issues all 8 x n_layers ``dispatch_bgmv`` calls of a decode step with the same
    four index tensors (lora_unordered_batch_infer.py:254-318, 428-448), so the
    first call of a step builds the plan and the others reuse it.

    An entry is reused only if the four tensors are the very same Python objects
    (held through weak references) at the same ``_version`` (every in-place torch
    operation raises it), on the same stream, for the same output width and pool
    size.  Code that rewrites an index tensor behind torch's back (a raw pointer
    handed to a custom kernel) must call ``clear_plan_cache()`` or set
    ``SLORA_PLAN_CACHE=0``.  Nothing is cached while the stream is being captured
    into a graph: a plan built there would not exist until the graph is replayed.
    """

    def __init__(self, capacity: int = 4):
        self.capacity = capacity
        self.entries = []
        self.hits = 0
        self.builds = 0

    def clear(self) -> None:
        self.entries.clear()

    def get(self, tensors, rank_cap: int, n_pages: int, stream: int):
        versions = tuple(t._version for t in tensors)
        for i, (refs, vers, cap, pages, strm, plan) in enumerate(self.entries):
            if cap == rank_cap and pages == n_pages and strm == stream and vers == versions and \
                    all(r() is t for r, t in zip(refs, tensors)):
                if i:
                    self.entries.insert(0, self.entries.pop(i))
                self.hits += 1
                return plan
        plan = make_plan(*tensors, rank_cap, n_pages, readback=True)
        self.builds += 1
        self.entries.insert(0, (tuple(weakref.ref(t) for t in tensors), versions, rank_cap, n_pages, stream, plan))
        del self.entries[self.capacity:]
        return plan


_plan_cache = _PlanCache()


def clear_plan_cache() -> None:
    """Forget every plan built for calls that passed none."""
    _plan_cache.clear()


def _auto_plan(start_indicies, lora_ranks, loc_indicies, indicies, rank_cap: int, n_pages: int, stream: int):
    if os.environ.get("SLORA_PLAN_CACHE", "1") == "0" or indicies.numel() == 0:
        return None
    if rank_cap <= 0 or rank_cap > _cabi.MAX_RANK or torch.cuda.is_current_stream_capturing():
        return None
    return _plan_cache.get((start_indicies, lora_ranks, loc_indicies, indicies), int(rank_cap), int(n_pages), stream)


def dispatch_bgmv(y, x, w, start_indicies, lora_ranks, loc_indicies, indicies, qkvo, lora_scales, plan=None) -> None:
    """``y`` (in place) from ``x`` and the paged adapter pool ``w``.

    ``x.size(1) >= y.size(1)``: shrink, ``y[b, :r] = x[b] @ A`` (overwrite,
    unscaled, columns >= r untouched).  ``x.size(1) < y.size(1)``: expand,
    ``y[b] += (x[b, :r] @ B) * lora_scales[a]``.  ``a = indicies[b]``,
    ``r = lora_ranks[a] // 4``; A rows / B pages are
    ``w[loc_indicies[start_indicies[a] + r*qkvo + i]]`` (direction rule:
    slora/csrc/bgmv/bgmv_impl.cuh:221).

    ``plan`` (keyword, optional, not in the reference): a ``BgmvPlan`` from
    ``make_plan`` for this batch; same results, fewer dependent table reads.
    Without it the plan of the last call with the same index tensors is reused
    (see ``_PlanCache``); ``plan=False`` forces the kernels that need no plan.
    """
    _check_input(y, "y")
    _check_input(x, "x")
    _validate_common(w, start_indicies, lora_ranks, loc_indicies, indicies, lora_scales)
    _check_dim(2, y, "y")
    _check_dim(2, x, "x")
    batch, h_in = x.size(0), x.size(1)
    h_out = y.size(1)
    if indicies.size(0) != x.size(0):
        raise RuntimeError(f"CHECK_EQ(indicies.size(0), x.size(0)) failed. {indicies.size(0)} vs {x.size(0)}")
    if y.size(0) != x.size(0):
        raise RuntimeError(f"CHECK_EQ(y.size(0), x.size(0)) failed. {y.size(0)} vs {x.size(0)}")
    qkvo = int(qkvo)
    no_kernel = f"No suitable kernel. h_in={h_in} h_out={h_out} dtype={x.dtype}"
    if x.dtype not in (torch.float16, torch.bfloat16) or y.dtype != x.dtype or w.dtype != x.dtype:
        raise RuntimeError(no_kernel)
    if not (h_in < 65536 and h_out < 65536):
        raise RuntimeError(no_kernel)
    lib = _cabi.load_library()
    page_elems = w.size(1) * w.size(2)
    tables = _tables(start_indicies, lora_ranks, loc_indicies)
    code = _DTYPE_CODE[x.dtype]
    stream = _stream(x)
    if plan is None:
        plan = _auto_plan(start_indicies, lora_ranks, loc_indicies, indicies, min(h_in, h_out), w.size(0), stream)
    elif plan is False:
        plan = None
    if plan is not None and plan.batch != batch:
        raise RuntimeError(f"plan was built for {plan.batch} tokens, this call has {batch}")
    if h_in < h_out:
        if plan is not None:
            rc = lib.slora_bgmv_expand_planned(plan.buf.data_ptr(), plan.rank_cap, plan.n_items, 1, y.data_ptr(), None,
                                               None, x.data_ptr(), None, None, w.data_ptr(), C.byref(tables),
                                               indicies.data_ptr(), lora_scales.data_ptr(),
                                               _DTYPE_CODE[lora_scales.dtype], batch, h_in, h_out, 0, 0, page_elems,
                                               w.size(0), qkvo, code, stream)
        else:
            rc = lib.slora_bgmv_expand(y.data_ptr(), x.data_ptr(), w.data_ptr(), C.byref(tables),
                                       indicies.data_ptr(), lora_scales.data_ptr(), _DTYPE_CODE[lora_scales.dtype],
                                       batch, h_in, h_out, page_elems, w.size(0), qkvo, code, stream)
    else:
        if plan is not None:
            rc = lib.slora_bgmv_shrink_planned(plan.buf.data_ptr(), plan.rank_cap, plan.n_items, 1, y.data_ptr(), None,
                                               None, x.data_ptr(), w.data_ptr(), C.byref(tables), indicies.data_ptr(),
                                               batch, h_in, h_out, page_elems, w.size(0), qkvo, code, stream)
        else:
            rc = lib.slora_bgmv_shrink(y.data_ptr(), x.data_ptr(), w.data_ptr(), C.byref(tables),
                                       indicies.data_ptr(), batch, h_in, h_out, page_elems, w.size(0), qkvo, code,
                                       stream)
    if rc == _cabi.ERR_UNSUPPORTED:
        raise RuntimeError(no_kernel)
    _cabi.check(rc, "dispatch_bgmv", f"(h_in={h_in} h_out={h_out} qkvo={qkvo})")


def dispatch_bgmv_qkv_shrink(y_q, y_k, y_v, x, w, start_indicies, lora_ranks, loc_indicies, indicies,
                             plan=None) -> None:
    """The three shrink calls of one layer (qkvo = 0, 1, 2 on the same ``x``,
    lora_unordered_batch_infer.py:267-270, 287-290, 307-310) as one launch."""
    for t, n in ((y_q, "y_q"), (y_k, "y_k"), (y_v, "y_v"), (x, "x")):
        _check_input(t, n)
        _check_dim(2, t, n)
    _validate_common(w, start_indicies, lora_ranks, loc_indicies, indicies)
    batch, h_in, y_cols = x.size(0), x.size(1), y_q.size(1)
    for t, n in ((y_q, "y_q"), (y_k, "y_k"), (y_v, "y_v")):
        if t.size(0) != batch or t.size(1) != y_cols or t.dtype != x.dtype:
            raise RuntimeError(f"{n} must be [{batch}, {y_cols}] {x.dtype}")
    if indicies.size(0) != batch:
        raise RuntimeError(f"CHECK_EQ(indicies.size(0), x.size(0)) failed. {indicies.size(0)} vs {batch}")
    no_kernel = f"No suitable kernel. h_in={h_in} h_out={y_cols} dtype={x.dtype}"
    if x.dtype not in (torch.float16, torch.bfloat16) or w.dtype != x.dtype:
        raise RuntimeError(no_kernel)
    lib = _cabi.load_library()
    tables = _tables(start_indicies, lora_ranks, loc_indicies)
    if plan is None:
        plan = _auto_plan(start_indicies, lora_ranks, loc_indicies, indicies, y_cols, w.size(0), _stream(x))
    elif plan is False:
        plan = None
    if plan is not None:
        rc = lib.slora_bgmv_shrink_planned(plan.buf.data_ptr(), plan.rank_cap, plan.n_items, 3, y_q.data_ptr(),
                                           y_k.data_ptr(), y_v.data_ptr(), x.data_ptr(), w.data_ptr(),
                                           C.byref(tables), indicies.data_ptr(), batch, h_in, y_cols,
                                           w.size(1) * w.size(2), w.size(0), 0, _DTYPE_CODE[x.dtype], _stream(x))
    else:
        rc = lib.slora_bgmv_shrink_qkv(y_q.data_ptr(), y_k.data_ptr(), y_v.data_ptr(), x.data_ptr(), w.data_ptr(),
                                       C.byref(tables), indicies.data_ptr(), batch, h_in, y_cols,
                                       w.size(1) * w.size(2), w.size(0), _DTYPE_CODE[x.dtype], _stream(x))
    if rc == _cabi.ERR_UNSUPPORTED:
        raise RuntimeError(no_kernel)
    _cabi.check(rc, "dispatch_bgmv_qkv_shrink")


def dispatch_bgmv_qkv_expand(y_q, y_k, y_v, x_q, x_k, x_v, w, start_indicies, lora_ranks, loc_indicies, indicies,
                             lora_scales, plan=None) -> None:
    """The three expand calls of one layer (lora_unordered_batch_infer.py:271-273,
    291-295, 311-315) as one launch.  ``y_k``/``y_v`` may be narrower than
    ``y_q`` (grouped-query attention)."""
    for t, n in ((y_q, "y_q"), (y_k, "y_k"), (y_v, "y_v"), (x_q, "x_q"), (x_k, "x_k"), (x_v, "x_v")):
        _check_input(t, n)
        _check_dim(2, t, n)
    _validate_common(w, start_indicies, lora_ranks, loc_indicies, indicies, lora_scales)
    batch, x_cols = x_q.size(0), x_q.size(1)
    for t, n in ((x_k, "x_k"), (x_v, "x_v")):
        if t.size(0) != batch or t.size(1) != x_cols or t.dtype != x_q.dtype:
            raise RuntimeError(f"{n} must be [{batch}, {x_cols}] {x_q.dtype}")
    for t, n in ((y_q, "y_q"), (y_k, "y_k"), (y_v, "y_v")):
        if t.size(0) != batch or t.dtype != x_q.dtype:
            raise RuntimeError(f"{n} must have {batch} rows of {x_q.dtype}")
    if indicies.size(0) != batch:
        raise RuntimeError(f"CHECK_EQ(indicies.size(0), x.size(0)) failed. {indicies.size(0)} vs {batch}")
    no_kernel = f"No suitable kernel. h_in={x_cols} h_out={y_q.size(1)} dtype={x_q.dtype}"
    if x_q.dtype not in (torch.float16, torch.bfloat16) or w.dtype != x_q.dtype:
        raise RuntimeError(no_kernel)
    lib = _cabi.load_library()
    tables = _tables(start_indicies, lora_ranks, loc_indicies)
    if plan is None:
        plan = _auto_plan(start_indicies, lora_ranks, loc_indicies, indicies, x_cols, w.size(0), _stream(x_q))
    elif plan is False:
        plan = None
    if plan is not None:
        rc = lib.slora_bgmv_expand_planned(plan.buf.data_ptr(), plan.rank_cap, plan.n_items, 3, y_q.data_ptr(),
                                           y_k.data_ptr(), y_v.data_ptr(), x_q.data_ptr(), x_k.data_ptr(),
                                           x_v.data_ptr(), w.data_ptr(), C.byref(tables), indicies.data_ptr(),
                                           lora_scales.data_ptr(), _DTYPE_CODE[lora_scales.dtype], batch, x_cols,
                                           y_q.size(1), y_k.size(1), y_v.size(1), w.size(1) * w.size(2), w.size(0), 0,
                                           _DTYPE_CODE[x_q.dtype], _stream(x_q))
    else:
        rc = lib.slora_bgmv_expand_qkv(y_q.data_ptr(), y_k.data_ptr(), y_v.data_ptr(), x_q.data_ptr(), x_k.data_ptr(),
                                       x_v.data_ptr(), w.data_ptr(), C.byref(tables), indicies.data_ptr(),
                                       lora_scales.data_ptr(), _DTYPE_CODE[lora_scales.dtype], batch, x_cols,
                                       y_q.size(1), y_k.size(1), y_v.size(1), w.size(1) * w.size(2), w.size(0),
                                       _DTYPE_CODE[x_q.dtype], _stream(x_q))
    if rc == _cabi.ERR_UNSUPPORTED:
        raise RuntimeError(no_kernel)
    _cabi.check(rc, "dispatch_bgmv_qkv_expand")
