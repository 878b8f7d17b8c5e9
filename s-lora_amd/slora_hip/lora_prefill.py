"""Prefill-time operator surface: ``lora_get_qkvo_fwd_shrink`` and
``lora_get_qkvo_fwd_expand`` with the reference's exact positional signatures
(slora/models/peft/triton_kernel/lora/lora_prefill.py:139 and :105), bound to
the segmented gather-GEMM HIP kernels of libslora_hip.so.

Note the argument order: these take ``(b_loc, b_lora_start, b_lora_ranks)``
while ``dispatch_bgmv`` takes ``(start, ranks, loc)``.  ``x``, ``w`` and ``o``
are 2-D and may be row-strided views (the reference passes ``stride(0)`` and
``stride(1)``; a column stride other than 1 is rejected here).
"""
from __future__ import annotations

import ctypes as C
import os
import weakref

import torch

from . import _cabi
from ._kernels import _DTYPE_CODE, _stream

_F16_BF16 = (torch.float16, torch.bfloat16)


def _check_2d(t, name):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if t.dim() != 2:
        raise RuntimeError(f"{name} must be a 2D tensor")
    if t.size(1) > 1 and t.stride(1) != 1:
        raise RuntimeError(f"{name} must have unit column stride, got {t.stride(1)}")


def _check_1d(t, name, dtype):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if t.dim() != 1 or not t.is_contiguous():
        raise RuntimeError(f"{name} must be a contiguous 1D tensor")
    if t.dtype != dtype:
        raise RuntimeError(f"{name} must be {dtype}, got {t.dtype}")


def _common(x, w, o, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies):
    _check_2d(x, "x")
    _check_2d(w, "w")
    _check_2d(o, "o")
    _check_1d(b_loc, "b_loc", torch.int64)
    _check_1d(b_lora_start, "b_lora_start", torch.int64)
    _check_1d(b_lora_ranks, "b_lora_ranks", torch.int64)
    _check_1d(b_indicies, "b_indicies", torch.int64)
    _check_1d(b_start_loc, "b_start_loc", torch.int32)
    _check_1d(b_seq_len, "b_seq_len", torch.int32)
    if x.dtype not in _F16_BF16 or w.dtype != x.dtype or o.dtype != x.dtype:
        raise RuntimeError(f"x, w and o must share a dtype of float16 or bfloat16, got {x.dtype}, {w.dtype}, {o.dtype}")
    if not (b_start_loc.numel() == b_seq_len.numel() == b_indicies.numel()):
        raise RuntimeError("b_start_loc, b_seq_len and b_indicies must have one entry per request")
    if b_lora_start.numel() != b_lora_ranks.numel():
        raise RuntimeError("b_lora_start and b_lora_ranks must have one entry per adapter")
    if x.size(0) != o.size(0):
        raise RuntimeError(f"x and o must have the same number of rows, got {x.size(0)} and {o.size(0)}")
    return _cabi.SloraTables(b_lora_start.data_ptr(), b_lora_ranks.data_ptr(), b_loc.data_ptr(),
                             b_lora_start.numel(), b_loc.numel())


class SgmmPlan:
    """How the shrink kernel shares a prefill batch out over its workgroups, computed
    once for the 4 x n_layers shrink calls of a prefill step (they all pass the same
    request tensors, lora_unordered_batch_infer.py:358-410).  ``usable`` is False for
    batch shapes that take no plan; the planned call then runs the plain kernel."""

    def __init__(self, buf, usable, n_requests, n_tokens, max_rank, max_input_len):
        self.buf = buf
        self.usable = usable
        self.n_requests = n_requests
        self.n_tokens = n_tokens
        self.max_rank = max_rank
        self.max_input_len = max_input_len


@torch.inference_mode()
def make_prefill_plan(b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies, n_tokens, max_rank,
                      max_input_len) -> SgmmPlan:
    """Build the shrink plan of one prefill batch on the current stream (one small launch)."""
    _check_1d(b_lora_start, "b_lora_start", torch.int64)
    _check_1d(b_lora_ranks, "b_lora_ranks", torch.int64)
    _check_1d(b_indicies, "b_indicies", torch.int64)
    _check_1d(b_start_loc, "b_start_loc", torch.int32)
    _check_1d(b_seq_len, "b_seq_len", torch.int32)
    if not (b_start_loc.numel() == b_seq_len.numel() == b_indicies.numel()):
        raise RuntimeError("b_start_loc, b_seq_len and b_indicies must have one entry per request")
    if b_lora_start.numel() != b_lora_ranks.numel():
        raise RuntimeError("b_lora_start and b_lora_ranks must have one entry per adapter")
    lib = _cabi.load_library()
    nbytes = int(lib.slora_sgmm_plan_bytes())
    buf = torch.empty(nbytes // 4, dtype=torch.int32, device=b_seq_len.device)
    # the plan reads no page ids: the loc table only has to be non-null
    tables = _cabi.SloraTables(b_lora_start.data_ptr(), b_lora_ranks.data_ptr(), b_lora_start.data_ptr(),
                               b_lora_start.numel(), 0)
    usable = C.c_int(0)
    rc = lib.slora_sgmm_plan_build(buf.data_ptr(), nbytes, C.byref(tables), b_start_loc.data_ptr(),
                                   b_seq_len.data_ptr(), b_indicies.data_ptr(), b_seq_len.numel(),
                                   int(max_input_len), int(n_tokens), int(max_rank), C.byref(usable),
                                   _stream(b_seq_len))
    _cabi.check(rc, "make_prefill_plan", f"(n_tokens={n_tokens} max_rank={max_rank})")
    return SgmmPlan(buf, bool(usable.value), b_seq_len.numel(), int(n_tokens), int(max_rank), int(max_input_len))


class _PrefillPlanCache:
    """Plans for callers that pass none: the reference's engine issues all shrink calls
    of a prefill step with the same five index tensors, so the first call builds the plan
    and the others reuse it.  Same rules as the decode plan cache: an entry is reused only
    for the very same tensor objects (weak references) at the same ``_version``, sizes and
    stream; nothing is cached during graph capture; ``SLORA_PLAN_CACHE=0`` turns it off."""

    MISS_STREAK = 8   # builds in a row that no later call reused ...
    COOL_DOWN = 256   # ... switch the cache off for this many calls: the caller makes new tensors every time

    def __init__(self, capacity: int = 2):
        self.capacity = capacity
        self.entries = []
        self.hits = 0
        self.builds = 0
        self.streak = 0
        self.paused = 0

    def clear(self) -> None:
        self.entries.clear()
        self.streak = self.paused = 0

    def get(self, tensors, sizes, stream):
        if self.paused:
            self.paused -= 1
            return None
        versions = tuple(t._version for t in tensors)
        for i, (refs, vers, sz, strm, plan) in enumerate(self.entries):
            if sz == sizes and strm == stream and vers == versions and all(r() is t for r, t in zip(refs, tensors)):
                if i:
                    self.entries.insert(0, self.entries.pop(i))
                self.hits += 1
                self.streak = 0
                return plan
        self.streak += 1
        if self.streak > self.MISS_STREAK:
            self.streak = 0
            self.paused = self.COOL_DOWN
            return None
        plan = make_prefill_plan(*tensors, *sizes)
        self.builds += 1
        self.entries.insert(0, (tuple(weakref.ref(t) for t in tensors), versions, sizes, stream, plan))
        del self.entries[self.capacity:]
        return plan


_prefill_plan_cache = _PrefillPlanCache()


def clear_prefill_plan_cache() -> None:
    """Forget every plan built for shrink calls that passed none."""
    _prefill_plan_cache.clear()


@torch.inference_mode()
def lora_get_qkvo_fwd_shrink(x, w, o, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies,
                             hidden_size, qkvo, max_rank, max_input_len, plan=None) -> None:
    """``o[rows_i, :r] = x[rows_i] @ A_i`` per request i (rows ``b_start_loc[i] +
    [0, b_seq_len[i])``), zeros in columns ``r..max_rank``.

    ``plan`` (keyword, optional, not in the reference): an ``SgmmPlan`` from
    ``make_prefill_plan`` for this batch; same results, the split of the batch over the
    workgroups is read instead of recomputed.  Without it the plan of the last call with
    the same index tensors is reused (``_PrefillPlanCache``); ``plan=False`` forces the
    kernel that needs no plan."""
    tables = _common(x, w, o, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies)
    if x.size(1) < hidden_size or w.size(1) < hidden_size or o.size(1) < max_rank:
        raise RuntimeError("x/w narrower than hidden_size or o narrower than max_rank")
    lib = _cabi.load_library()
    stream = _stream(x)
    sizes = (x.size(0), int(max_rank), int(max_input_len))
    if plan is None and os.environ.get("SLORA_PLAN_CACHE", "1") != "0" and b_seq_len.numel() > 0 and \
            x.size(0) > 0 and 0 < max_rank <= _cabi.MAX_RANK and max_input_len > 0 and \
            not torch.cuda.is_current_stream_capturing():
        plan = _prefill_plan_cache.get((b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies), sizes, stream)
    if isinstance(plan, SgmmPlan):
        if (plan.n_requests, plan.n_tokens, plan.max_rank, plan.max_input_len) != (b_seq_len.numel(),) + sizes:
            raise RuntimeError("lora_get_qkvo_fwd_shrink: the plan was built for another batch "
                               f"({plan.n_requests} requests, {plan.n_tokens} tokens, max_rank {plan.max_rank}, "
                               f"max_input_len {plan.max_input_len})")
        if plan.usable:
            rc = lib.slora_sgmm_shrink_planned(plan.buf.data_ptr(), o.data_ptr(), x.data_ptr(), w.data_ptr(),
                                               C.byref(tables), b_start_loc.data_ptr(), b_seq_len.data_ptr(),
                                               b_indicies.data_ptr(), b_seq_len.numel(), int(max_input_len),
                                               x.size(0), int(hidden_size), int(max_rank), x.stride(0), w.stride(0),
                                               o.stride(0), w.size(0), int(qkvo), _DTYPE_CODE[x.dtype], stream)
            _cabi.check(rc, "lora_get_qkvo_fwd_shrink",
                        f"(planned, hidden_size={hidden_size} max_rank={max_rank} qkvo={qkvo})")
            return
    rc = lib.slora_sgmm_shrink(o.data_ptr(), x.data_ptr(), w.data_ptr(), C.byref(tables), b_start_loc.data_ptr(),
                               b_seq_len.data_ptr(), b_indicies.data_ptr(), b_seq_len.numel(), int(max_input_len),
                               x.size(0), int(hidden_size), int(max_rank), x.stride(0), w.stride(0), o.stride(0),
                               w.size(0), int(qkvo), _DTYPE_CODE[x.dtype], stream)
    _cabi.check(rc, "lora_get_qkvo_fwd_shrink", f"(hidden_size={hidden_size} max_rank={max_rank} qkvo={qkvo})")


@torch.inference_mode()
def lora_get_qkvo_fwd_expand(x, w, o, scale, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies,
                             feat_out, qkvo, max_rank, max_input_len) -> None:
    """``o[rows_i] += (x[rows_i, :r] @ B_i) * scale[a_i]`` per request i."""
    tables = _common(x, w, o, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies)
    if not isinstance(scale, torch.Tensor) or not scale.is_cuda or not scale.is_contiguous():
        raise RuntimeError("scale must be a contiguous CUDA tensor")
    if scale.dtype not in _DTYPE_CODE:
        raise RuntimeError(f"scale must be float16, bfloat16 or float32, got {scale.dtype}")
    if scale.numel() < b_lora_start.numel():
        raise RuntimeError("scale must have one entry per adapter")
    if o.size(1) < feat_out or x.size(1) < max_rank:
        raise RuntimeError("o narrower than feat_out or x narrower than max_rank")
    lib = _cabi.load_library()
    rc = lib.slora_sgmm_expand(o.data_ptr(), x.data_ptr(), w.data_ptr(), C.byref(tables), scale.data_ptr(),
                               _DTYPE_CODE[scale.dtype], b_start_loc.data_ptr(), b_seq_len.data_ptr(),
                               b_indicies.data_ptr(), b_seq_len.numel(), int(max_input_len), x.size(0),
                               int(feat_out), w.size(1), int(max_rank), x.stride(0), w.stride(0), o.stride(0),
                               w.size(0), int(qkvo), _DTYPE_CODE[x.dtype], _stream(x))
    _cabi.check(rc, "lora_get_qkvo_fwd_expand", f"(feat_out={feat_out} max_rank={max_rank} qkvo={qkvo})")
