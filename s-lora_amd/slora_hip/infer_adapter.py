"""Loading adapters into the unified pool and dropping them again: the device
side of ``InferAdapter`` (slora/server/router/model_infer/infer_adapter.py).

* ``load_rows_into_pool``    -- ``buffer[loc] = rows`` for many buffers in one launch
                               (``load_lora_A`` / ``load_lora_B``, :43-88).
* ``launch_var_len_copy``    -- same arguments as ``launch_var_len_copy_triton`` (:274-280).
* ``compact_adapter_tables`` -- the table rebuild of ``offload_adapters`` (:186-258).

* ``PageAllocator``          -- ``MemoryAllocator.alloc / alloc_contiguous / free``
                               (slora/common/mem_allocator.py:30-59, 185-199) on the device.

* ``merge_adapter`` / ``unmerge_adapter`` -- ``W_p +-= scaling * A_p B_p`` for the four
                               projections of a layer, reading A and B from the pool
                               (slora/models/peft/lora_single_batch_infer.py:60-93).

All of them are ctypes calls into libslora_hip.so; there is no fallback.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _cabi
from ._kernels import _DTYPE_CODE, _check_index, _check_input, _stream, _tables


def load_rows_into_pool(buffers, rows, loc) -> None:
    """``buffers[b][loc] = rows[b]`` for every b, in one launch per 64 buffers.

    ``buffers``: pool tensors ``[n_pages, ...]`` of one shape and dtype (e.g.
    ``key_buffer[l]`` and ``value_buffer[l]`` of every layer); ``rows``: as many
    tensors ``[len(loc), ...]`` with the same trailing shape (``w_combined[0]``
    and ``w_combined[1]`` of every layer); ``loc``: int64 page ids on the device.
    """
    buffers, rows = list(buffers), list(rows)
    if len(buffers) != len(rows):
        raise RuntimeError(f"{len(buffers)} pool buffers but {len(rows)} row blocks")
    if not buffers:
        return
    _check_input(loc, "loc")
    _check_index(loc, "loc")
    n_rows = loc.numel()
    b0 = buffers[0]
    row_elems = b0[0].numel() if b0.size(0) else 0
    for i, (b, r) in enumerate(zip(buffers, rows)):
        _check_input(b, f"buffers[{i}]")
        _check_input(r, f"rows[{i}]")
        if b.dtype != b0.dtype or r.dtype != b0.dtype:
            raise RuntimeError("pool buffers and rows must share one dtype")
        if b.shape != b0.shape:
            raise RuntimeError("pool buffers must share one shape")
        if r.size(0) != n_rows or r.numel() != n_rows * row_elems:
            raise RuntimeError(f"rows[{i}] must be [{n_rows}, {tuple(b0.shape[1:])}], got {tuple(r.shape)}")
    row_bytes = row_elems * b0.element_size()
    lib = _cabi.load_library()
    n = len(buffers)
    dst = (C.c_void_p * n)(*[b.data_ptr() for b in buffers])
    src = (C.c_void_p * n)(*[r.data_ptr() for r in rows])
    rc = lib.slora_pool_scatter_rows(dst, src, n, loc.data_ptr(), n_rows, row_bytes, row_bytes, row_bytes, b0.size(0),
                                     _stream(loc))
    _cabi.check(rc, "load_rows_into_pool")


def launch_var_len_copy(old_a_start, old_a_len, old_location, new_a_start, new_a_location) -> None:
    """``new_a_location[new_a_start[i] + k] = old_location[old_a_start[i] + k]``
    for ``k < old_a_len[i]`` (infer_adapter.py:261-280)."""
    for t, n in ((old_a_start, "old_a_start"), (old_a_len, "old_a_len"), (old_location, "old_location"),
                 (new_a_start, "new_a_start"), (new_a_location, "new_a_location")):
        _check_input(t, n)
        _check_index(t, n)
    n = old_a_start.numel()
    if old_a_len.numel() != n or new_a_start.numel() != n:
        raise RuntimeError("old_a_start, old_a_len and new_a_start must have one entry per adapter")
    lib = _cabi.load_library()
    rc = lib.slora_var_len_copy(old_a_start.data_ptr(), old_a_len.data_ptr(), old_location.data_ptr(),
                                new_a_start.data_ptr(), new_a_location.data_ptr(), n, old_location.numel(),
                                new_a_location.numel(), _stream(old_location))
    _cabi.check(rc, "launch_var_len_copy")


launch_var_len_copy_triton = launch_var_len_copy  # the name the reference imports


def compact_adapter_tables(a_start, a_len, a_loc, a_scaling, keep):
    """Drop the adapters with ``keep[i] == False``.  Returns ``(new_a_start,
    new_a_len, new_a_loc, new_a_scaling, removed_pages)``: the tables of the
    kept adapters in their old order and the page ids to give back to the
    allocator.  One launch and one 32-byte read-back."""
    for t, n in ((a_start, "a_start"), (a_len, "a_len"), (a_loc, "a_loc")):
        _check_input(t, n)
        _check_index(t, n)
    _check_input(a_scaling, "a_scaling")
    _check_input(keep, "keep")
    n = a_start.numel()
    if a_len.numel() != n or a_scaling.numel() != n or keep.numel() != n:
        raise RuntimeError("a_start, a_len, a_scaling and keep must have one entry per adapter")
    if a_scaling.dtype not in _DTYPE_CODE:
        raise RuntimeError(f"a_scaling must be float16, bfloat16 or float32, got {a_scaling.dtype}")
    if keep.dtype not in (torch.bool, torch.uint8):
        raise RuntimeError(f"keep must be a bool or uint8 tensor, got {keep.dtype}")
    dev = a_start.device
    n_loc = a_loc.numel()
    new_start = torch.empty(n, dtype=torch.int64, device=dev)
    new_len = torch.empty(n, dtype=torch.int64, device=dev)
    new_loc = torch.empty(n_loc, dtype=torch.int64, device=dev)
    new_scaling = torch.empty(n, dtype=a_scaling.dtype, device=dev)
    removed = torch.empty(n_loc, dtype=torch.int64, device=dev)
    counts = torch.zeros(4, dtype=torch.int64, device=dev)
    work = torch.empty(max(n, 1), dtype=torch.int64, device=dev)
    lib = _cabi.load_library()
    tables = _tables(a_start, a_len, a_loc)
    rc = lib.slora_tables_compact(C.byref(tables), a_scaling.data_ptr(), _DTYPE_CODE[a_scaling.dtype],
                                  keep.view(torch.uint8).data_ptr() if keep.dtype == torch.bool else keep.data_ptr(),
                                  new_start.data_ptr(), new_len.data_ptr(), new_loc.data_ptr(),
                                  new_scaling.data_ptr(), removed.data_ptr(), counts.data_ptr(), work.data_ptr(),
                                  _stream(a_start))
    _cabi.check(rc, "compact_adapter_tables")
    n_keep, n_keep_loc, _, n_removed_loc = (int(v) for v in counts.cpu())
    return new_start[:n_keep], new_len[:n_keep], new_loc[:n_keep_loc], new_scaling[:n_keep], removed[:n_removed_loc]


class PageAllocator:
    """The free map of the unified pool and the three operations the serving loop
    uses on it (``MemoryAllocator`` of slora/common/mem_allocator.py without the
    buffers): ``mem_state`` is a bool tensor, True = free, exactly the reference's;
    ``can_use_mem_size`` is kept on the host as the reference keeps it."""

    def __init__(self, tot_size: int, device="cuda"):
        self.tot_size = int(tot_size)
        self.device = torch.device(device)
        self.mem_state = torch.ones((self.tot_size,), dtype=torch.bool, device=self.device)
        self.can_use_mem_size = self.tot_size
        lib = _cabi.load_library()
        nbytes = int(lib.slora_pool_alloc_workspace_bytes(self.tot_size))
        self._work = torch.empty((nbytes + 7) // 8, dtype=torch.int64, device=self.device)
        self._result = torch.zeros(2, dtype=torch.int64, device=self.device)

    def _state_ptr(self) -> int:
        return self.mem_state.data_ptr()

    def alloc(self, need_size: int) -> torch.Tensor:
        need_size = int(need_size)
        if need_size > self.can_use_mem_size:
            raise Exception(f'warn no enough pool space: need_size {need_size} left_size {self.can_use_mem_size}')
        out = torch.empty(need_size, dtype=torch.int64, device=self.device)
        lib = _cabi.load_library()
        rc = lib.slora_pool_alloc(self._state_ptr(), self.tot_size, need_size, out.data_ptr(),
                                  self._result.data_ptr(), self._work.data_ptr(), _stream(self.mem_state))
        _cabi.check(rc, "PageAllocator.alloc")
        self.can_use_mem_size -= need_size
        return out

    def alloc_contiguous(self, need_size: int):
        need_size = int(need_size)
        if need_size > self.can_use_mem_size:
            raise Exception(f'warn no enough pool space: need_size {need_size} left_size {self.can_use_mem_size}')
        if need_size <= 0:
            raise RuntimeError("need_size must be positive")
        out = torch.empty(need_size, dtype=torch.int64, device=self.device)
        lib = _cabi.load_library()
        rc = lib.slora_pool_alloc_contiguous(self._state_ptr(), self.tot_size, need_size, out.data_ptr(),
                                             self._result.data_ptr(), self._work.data_ptr(),
                                             _stream(self.mem_state))
        _cabi.check(rc, "PageAllocator.alloc_contiguous")
        start = int(self._result[0].item())  # the reference reads the start back as well (mem_allocator.py:57)
        if start < 0:
            return None
        self.can_use_mem_size -= need_size
        return out, start, start + need_size

    def free(self, free_index: torch.Tensor) -> None:
        _check_input(free_index, "free_index")
        _check_index(free_index, "free_index")
        lib = _cabi.load_library()
        rc = lib.slora_pool_free(self._state_ptr(), self.tot_size, free_index.data_ptr(), free_index.numel(),
                                 _stream(self.mem_state))
        _cabi.check(rc, "PageAllocator.free")
        self.can_use_mem_size += free_index.shape[0]

    def free_all(self) -> None:
        self.mem_state[:] = True
        self.can_use_mem_size = self.tot_size


def gather_lora_a(key_buffer, a_loc, first: int, rank: int, hidden: int, out_cols: int = 0) -> torch.Tensor:
    """``A_p`` as a dense ``[hidden, out_cols]`` tensor out of the pool pages
    ``a_loc[first : first + rank]`` (lora_single_batch_infer.py:38-46); columns
    ``rank..out_cols`` are zero."""
    _check_input(key_buffer, "key_buffer")
    _check_input(a_loc, "a_loc")
    _check_index(a_loc, "a_loc")
    if key_buffer.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("key_buffer must be float16 or bfloat16")
    out_cols = int(out_cols) or int(rank)
    page_elems = key_buffer[0].numel() if key_buffer.size(0) else 0
    out = torch.empty((hidden, out_cols), dtype=key_buffer.dtype, device=key_buffer.device)
    lib = _cabi.load_library()
    rc = lib.slora_pool_gather_a(out.data_ptr(), out_cols, key_buffer.data_ptr(), a_loc.data_ptr(), a_loc.numel(),
                                 int(first), int(rank), int(hidden), page_elems, key_buffer.size(0),
                                 _stream(key_buffer))
    _cabi.check(rc, "gather_lora_a")
    return out


def merge_adapter(weights, key_buffer, value_buffer, a_start, a_len, a_loc, a_scaling, adapter_idx: int,
                  sign: float = 1.0) -> None:
    """One layer of ``LoraPEFTBatchInfer.merge_adapter`` (lora_single_batch_infer.py:60-76):
    ``weights[p] += sign * scaling * A_p @ B_p`` in place for p in q, k, v, o, with
    ``weights[p]`` the ``[hidden, h_out_p]`` matrix the base model multiplies
    activations with, and A, B read from the adapter's pool pages.

    A_p is unpacked by ``gather_lora_a``; the product and the update are the
    prefill expand kernel with the ``hidden`` rows of A_p standing for tokens of
    one request (float accumulate, scale applied to the sum, one rounding when
    the sum is added to W -- the reference rounds ``B * scaling`` and ``A @ B`` to
    the storage type on the way)."""
    from .lora_prefill import lora_get_qkvo_fwd_expand
    if len(weights) != 4:
        raise RuntimeError("weights must be the q, k, v, o matrices of one layer")
    start = int(a_start[adapter_idx].item())   # the reference reads these back too (:30-32)
    rank = int(a_len[adapter_idx].item()) // 4
    if rank == 0:
        return
    dev = key_buffer.device
    hidden = weights[0].size(0)
    cols = (rank + 7) // 8 * 8
    scale = a_scaling if sign == 1.0 else a_scaling * sign
    seg_start = torch.zeros(1, dtype=torch.int32, device=dev)
    seg_len = torch.full((1,), hidden, dtype=torch.int32, device=dev)
    seg_idx = torch.full((1,), int(adapter_idx), dtype=torch.int64, device=dev)
    page = value_buffer[0].numel()
    for p in range(4):
        w_p = weights[p]
        if w_p.size(0) != hidden or w_p.dtype != key_buffer.dtype:
            raise RuntimeError(f"weights[{p}] must be [{hidden}, h_out] {key_buffer.dtype}")
        a_p = gather_lora_a(key_buffer, a_loc, start + p * rank, rank, hidden, cols)
        lora_get_qkvo_fwd_expand(a_p, value_buffer.view(-1, page), w_p, scale, a_loc, a_start, a_len, seg_start,
                                 seg_len, seg_idx, w_p.size(1), p, cols, hidden)


def unmerge_adapter(weights, key_buffer, value_buffer, a_start, a_len, a_loc, a_scaling, adapter_idx: int) -> None:
    """``weights[p] -= scaling * A_p @ B_p`` (lora_single_batch_infer.py:78-93)."""
    merge_adapter(weights, key_buffer, value_buffer, a_start, a_len, a_loc, a_scaling, adapter_idx, sign=-1.0)
