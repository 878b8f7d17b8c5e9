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

All of them call libslora_hip.so through the compiled extension; there is no fallback.
"""
from __future__ import annotations

import torch

from . import _kernels
from ._kernels import launch_var_len_copy, load_rows_into_pool  # noqa: F401

launch_var_len_copy_triton = launch_var_len_copy  # the name the reference imports (infer_adapter.py:274)


def compact_adapter_tables(a_start, a_len, a_loc, a_scaling, keep):
    """Drop the adapters with ``keep[i] == False``.  Returns ``(new_a_start,
    new_a_len, new_a_loc, new_a_scaling, removed_pages)``: the tables of the
    kept adapters in their old order and the page ids to give back to the
    allocator.  One launch and one 32-byte read-back."""
    new_start, new_len, new_loc, new_scaling, removed, counts = _kernels.compact_adapter_tables_raw(
        a_start, a_len, a_loc, a_scaling, keep)
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
        nbytes = int(_kernels.pool_alloc_workspace_bytes(self.tot_size))
        self._work = torch.empty((nbytes + 7) // 8, dtype=torch.int64, device=self.device)
        self._result = torch.zeros(2, dtype=torch.int64, device=self.device)

    def alloc(self, need_size: int) -> torch.Tensor:
        need_size = int(need_size)
        if need_size > self.can_use_mem_size:
            raise Exception(f'warn no enough pool space: need_size {need_size} left_size {self.can_use_mem_size}')
        out = torch.empty(need_size, dtype=torch.int64, device=self.device)
        _kernels.pool_alloc(self.mem_state, need_size, out, self._result, self._work)
        self.can_use_mem_size -= need_size
        return out

    def alloc_contiguous(self, need_size: int):
        need_size = int(need_size)
        if need_size > self.can_use_mem_size:
            raise Exception(f'warn no enough pool space: need_size {need_size} left_size {self.can_use_mem_size}')
        if need_size <= 0:
            raise RuntimeError("need_size must be positive")
        out = torch.empty(need_size, dtype=torch.int64, device=self.device)
        _kernels.pool_alloc_contiguous(self.mem_state, need_size, out, self._result, self._work)
        start = int(self._result[0].item())  # the reference reads the start back as well (mem_allocator.py:57)
        if start < 0:
            return None
        self.can_use_mem_size -= need_size
        return out, start, start + need_size

    def free(self, free_index: torch.Tensor) -> None:
        _kernels.pool_free(self.mem_state, free_index)
        self.can_use_mem_size += free_index.shape[0]

    def free_all(self) -> None:
        self.mem_state[:] = True
        self.can_use_mem_size = self.tot_size


def gather_lora_a(key_buffer, a_loc, first: int, rank: int, hidden: int, out_cols: int = 0) -> torch.Tensor:
    """``A_p`` as a dense ``[hidden, out_cols]`` tensor out of the pool pages
    ``a_loc[first : first + rank]`` (lora_single_batch_infer.py:38-46); columns
    ``rank..out_cols`` are zero."""
    return _kernels.gather_lora_a(key_buffer, a_loc, int(first), int(rank), int(hidden), int(out_cols))


def merge_adapter(weights, key_buffer, value_buffer, a_start, a_len, a_loc, a_scaling, adapter_idx: int,
                  sign: float = 1.0, start: int = None, rank: int = None) -> None:
    """One layer of ``LoraPEFTBatchInfer.merge_adapter`` (lora_single_batch_infer.py:60-76):
    ``weights[p] += sign * scaling * A_p @ B_p`` in place for p in q, k, v, o, with
    ``weights[p]`` the ``[hidden, h_out_p]`` matrix the base model multiplies
    activations with, and A, B read from the adapter's pool pages.

    ``start`` / ``rank``: ``a_start[adapter_idx]`` and ``a_len[adapter_idx] // 4`` when the
    caller holds them on the host (``InferAdapter`` does); left out, they are read back from
    the device as the reference does (:30-32), which waits for the stream.

    A_p is unpacked by ``gather_lora_a``; the product and the update are the
    prefill expand kernel with the ``hidden`` rows of A_p standing for tokens of
    one request (float accumulate, scale applied to the sum, one rounding when
    the sum is added to W -- the reference rounds ``B * scaling`` and ``A @ B`` to
    the storage type on the way)."""
    from .lora_prefill import lora_get_qkvo_fwd_expand
    if len(weights) != 4:
        raise RuntimeError("weights must be the q, k, v, o matrices of one layer")
    if start is None or rank is None:
        start = int(a_start[adapter_idx].item())
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


def unmerge_adapter(weights, key_buffer, value_buffer, a_start, a_len, a_loc, a_scaling, adapter_idx: int,
                    start: int = None, rank: int = None) -> None:
    """``weights[p] -= scaling * A_p @ B_p`` (lora_single_batch_infer.py:78-93)."""
    merge_adapter(weights, key_buffer, value_buffer, a_start, a_len, a_loc, a_scaling, adapter_idx, sign=-1.0,
                  start=start, rank=rank)
