"""Loading adapters into the unified pool and dropping them again: the device
side of ``InferAdapter`` (slora/server/router/model_infer/infer_adapter.py).

* ``load_rows_into_pool``    -- ``buffer[loc] = rows`` for many buffers in one launch
                               (``load_lora_A`` / ``load_lora_B``, :43-88).
* ``pack_lora_into_pool``    -- A_p / B_p as the reference keeps them at home, transposed and
                               written straight into the adapter's pages: ``w_combined``
                               (slora/models/peft/layer_weights/lora_layer_weight.py:84-93)
                               and its index_put in one pass.
* ``launch_var_len_copy``    -- same arguments as ``launch_var_len_copy_triton`` (:274-280).
* ``compact_adapter_tables`` -- the table rebuild of ``offload_adapters`` (:186-258).
* ``InferAdapter``           -- the class itself: ``load_adapters`` / ``offload_adapters`` over
                               the four index tables (:11-39, 92-258).
* ``MemoryAllocator``        -- the reference's pool object (buffers + free map) on
                               ``PageAllocator``, with a placement call for adapters.

* ``PageAllocator``          -- ``MemoryAllocator.alloc / alloc_contiguous / free``
                               (slora/common/mem_allocator.py:30-59, 185-199) on the device.

* ``merge_adapter`` / ``unmerge_adapter`` -- ``W_p +-= scaling * A_p B_p`` for the four
                               projections of a layer, reading A and B from the pool
                               (slora/models/peft/lora_single_batch_infer.py:60-93).

All of them call libslora_hip.so through the compiled extension; there is no fallback.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List

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


def page_checksums(buffer: torch.Tensor, loc: torch.Tensor) -> torch.Tensor:
    """xor of the 32-bit words of each pool page ``buffer[loc[i]]`` (int32 tensor): a cheap way to
    tell whether the pages an adapter was loaded into still hold what was written there.  A page id
    outside the buffer gives 0."""
    return _kernels.page_checksums(buffer, loc)


def page_xor(buffer: torch.Tensor, loc: torch.Tensor, key: int = 0) -> None:
    """``buffer[loc[i]] ^= key`` on every 32-bit word, in place.  With ``key = 0`` nothing changes
    but every listed page is read and written once: the plain read-modify-write of scattered
    rows that the benchmark times as the floor of the kernels that update an output in place."""
    _kernels.page_xor(buffer, loc, int(key))


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


def pack_lora_into_pool(key_buffers, value_buffers, lora_A, lora_B, loc, rank: int) -> None:
    """Write one adapter into its pool pages ``loc`` (``4 * rank`` page ids, the same in every
    layer): ``lora_A[l][p]`` is A_p of layer l as the reference keeps it at home,
    ``[hidden, rank]`` (``q_lora_A_home`` ... of lora_layer_weight.py:57-76, 170-213), and
    ``lora_B[l][p]`` is B_p, ``[rank, h_out_p]``, p in q, k, v, o.  Page ``loc[p*rank + j]`` of
    ``key_buffers[l]`` receives column j of A_p; the pages ``loc[p*rank ..]`` of
    ``value_buffers[l]`` receive the ``(h_out_p, rank)`` row-major matrix B_p^T end to end
    (lora_layer_weight.py:84-93): what ``w_combined`` holds, without building it.  One launch
    per 8 layers."""
    n_layers = len(key_buffers)
    if not (len(value_buffers) == len(lora_A) == len(lora_B) == n_layers):
        raise RuntimeError("key_buffers, value_buffers, lora_A and lora_B must have one entry per layer")
    rank = int(rank)
    if rank <= 0 or n_layers == 0:
        return
    page_elems = key_buffers[0][0].numel() if key_buffers[0].size(0) else 0
    bufs, mats, first, pitch, slot = [], [], [], [], []
    for l in range(n_layers):
        if len(lora_A[l]) != 4 or len(lora_B[l]) != 4:
            raise RuntimeError("every layer needs the q, k, v, o matrices")
        for p in range(4):
            a, b = lora_A[l][p], lora_B[l][p]
            if a.dim() != 2 or a.size(1) != rank or b.dim() != 2 or b.size(0) != rank:
                raise RuntimeError(f"layer {l} projection {p}: A must be [hidden, {rank}] and B [{rank}, h_out], got "
                                   f"{tuple(a.shape)} and {tuple(b.shape)}")
            bufs += [key_buffers[l], value_buffers[l]]
            mats += [a, b]
            first += [p * rank, p * rank]
            pitch += [page_elems, rank]
            slot += [rank, rank]
    _kernels.pack_transposed_into_pool(bufs, mats, first, pitch, slot, loc)


class MemoryAllocator(PageAllocator):
    """``MemoryAllocator`` of slora/common/mem_allocator.py:10-234 with the same constructor,
    attributes and calls: per-layer ``key_buffer`` / ``value_buffer`` of ``[tot_size, head_num,
    head_dim]`` shared by the KV cache and the adapters, and the free map of ``PageAllocator``.

    ``alloc_adapter`` is the placement call for adapter pages (not in the reference, whose
    ``alloc`` hands out the first free pages wherever they lie, mem_allocator.py:30-39): one
    contiguous run when the map has one, so that an adapter's ``4 r`` pages are one stretch of
    the pool; the first free pages otherwise."""

    def __init__(self, tot_size, cache_size, dtype, head_num, head_dim, layer_num, device="cuda"):
        assert tot_size >= cache_size
        self.dtype = dtype
        self.head_num = head_num
        self.head_dim = head_dim
        self.layer_num = layer_num
        self.cell_size = head_num * head_dim
        self.cache_size = cache_size
        super().__init__(tot_size, device)
        self.key_buffer = [torch.empty((self.tot_size, head_num, head_dim), dtype=dtype, device=self.device)
                           for _ in range(layer_num)]
        self.value_buffer = [torch.empty((self.tot_size, head_num, head_dim), dtype=dtype, device=self.device)
                             for _ in range(layer_num)]

    def get_memory_size(self):
        return 2 * self.layer_num * self.tot_size * self.cell_size * torch.empty((), dtype=self.dtype).element_size()

    def alloc_adapter(self, need_size: int) -> torch.Tensor:
        need_size = int(need_size)
        if need_size <= 0:
            return torch.empty(0, dtype=torch.int64, device=self.device)
        got = self.alloc_contiguous(need_size)
        return got[0] if got is not None else self.alloc(need_size)


@dataclass
class InferAdapter:
    """The adapters that live in the pool and their index tables
    (slora/server/router/model_infer/infer_adapter.py:11-258): adapter i owns the page ids
    ``a_loc[a_start[i] : a_start[i] + a_len[i]]``, ``a_len[i] = 4 * rank``, ``a_scaling[i] =
    lora_alpha / rank``.  Same fields and calls as the reference's class.

    An adapter passed to ``load_adapters`` has ``lora_dir``, ``r``, ``scaling`` and either
    ``layers`` whose entries offer ``load_to_gpu()`` / ``w_combined`` / ``offload_from_gpu()``
    (the reference's ``LoraLayerWeight``: the rows are scattered into every layer's buffers in
    one launch) or ``lora_A`` / ``lora_B`` (per layer the q, k, v, o matrices ``[hidden, r]`` /
    ``[r, h_out]`` on the device: packed straight into the pages by ``pack_lora_into_pool``).
    ``placement=True`` asks the pool for one contiguous run per adapter
    (``MemoryAllocator.alloc_adapter``) instead of the reference's single ``alloc`` of the sum."""
    adapter_dirs: List[str]
    a_loc: torch.Tensor
    a_start: torch.Tensor
    a_len: torch.Tensor
    a_scaling: torch.Tensor
    mem_manager: Any
    idx_map: Dict[str, int] = field(default_factory=dict)
    prefetch_tag: Dict[str, int] = field(default_factory=dict)
    cur_tag: int = 0
    prefetch_stream: Any = None
    placement: bool = False
    len_host: List[int] = field(default_factory=list)   # a_len on the host, kept in step with the tables

    @classmethod
    def init(cls, mem_manager, prefetch_stream=None, placement=False, device="cuda"):
        dev = torch.device(device)
        return cls(adapter_dirs=[],
                   a_loc=torch.empty(0, dtype=torch.long, device=dev),
                   a_start=torch.empty(0, dtype=torch.long, device=dev),
                   a_len=torch.empty(0, dtype=torch.long, device=dev),
                   a_scaling=torch.empty(0, dtype=torch.float16, device=dev),
                   mem_manager=mem_manager, idx_map={}, prefetch_tag={}, cur_tag=0,
                   prefetch_stream=prefetch_stream, placement=placement)

    # ---- one adapter's weights into the pages `loc` of every layer (load_lora_A + load_lora_B, :43-88)
    def _load_weights(self, adapter, loc) -> None:
        mm = self.mem_manager
        if getattr(adapter, "lora_A", None) is not None:
            pack_lora_into_pool(mm.key_buffer, mm.value_buffer, adapter.lora_A, adapter.lora_B, loc, adapter.r)
            return
        for layer in adapter.layers:
            layer.load_to_gpu()
        load_rows_into_pool(list(mm.key_buffer) + list(mm.value_buffer),
                            [layer.w_combined[0] for layer in adapter.layers] +
                            [layer.w_combined[1] for layer in adapter.layers], loc)
        for layer in adapter.layers:
            layer.offload_from_gpu()

    def load_adapters(self, adapters, prefetch=False) -> None:
        if len(adapters) == 0:
            return
        new_adapters, tot_size = [], 0
        if prefetch:
            self.cur_tag ^= 1
            capacity = self.mem_manager.can_use_mem_size
            for adapter in adapters:
                if adapter is None:
                    continue
                self.prefetch_tag[adapter.lora_dir] = self.cur_tag
                if adapter.lora_dir not in self.idx_map and adapter not in new_adapters:
                    if tot_size + adapter.r * 4 > capacity:
                        break
                    new_adapters.append(adapter)
                    tot_size += adapter.r * 4
        else:
            for adapter in adapters:
                if adapter is not None and adapter.lora_dir not in self.idx_map and adapter not in new_adapters:
                    new_adapters.append(adapter)
                    tot_size += adapter.r * 4
        if not new_adapters:
            return
        dev = self.a_loc.device
        if self.placement and hasattr(self.mem_manager, "alloc_adapter"):
            new_loc = torch.cat([self.mem_manager.alloc_adapter(a.r * 4) for a in new_adapters])
        else:
            new_loc = self.mem_manager.alloc(tot_size)
        # the new adapters' tables, built on the host (sizes are host values) and appended in one go each
        lens = [a.r * 4 for a in new_adapters]
        starts, cum = [], 0
        loc_offset = self.a_loc.shape[0]
        for a, n in zip(new_adapters, lens):
            starts.append(loc_offset + cum)
            self.idx_map[a.lora_dir] = len(self.adapter_dirs)
            self.adapter_dirs.append(a.lora_dir)
            self.len_host.append(n)
            cum += n
        self.a_start = torch.cat((self.a_start, torch.tensor(starts, dtype=torch.long, device=dev)))
        self.a_len = torch.cat((self.a_len, torch.tensor(lens, dtype=torch.long, device=dev)))
        self.a_loc = torch.cat((self.a_loc, new_loc))
        self.a_scaling = torch.cat((self.a_scaling, torch.tensor([a.scaling for a in new_adapters],
                                                                 dtype=torch.float16, device=dev)))

        def copy_all(loc):
            cum = 0
            for a, n in zip(new_adapters, lens):
                self._load_weights(a, loc[cum: cum + n])
                cum += n

        if prefetch and self.prefetch_stream is not None:
            side = self.prefetch_stream
            side.wait_stream(torch.cuda.current_stream())  # new_loc is produced on this stream
            with torch.cuda.stream(side):
                # the page list the loaders read is the side stream's own copy (as the reference's clone,
                # :153-155): new_loc goes out of scope when this function returns, and a block that the main
                # stream's allocator hands out again must not be one the queued kernels still read
                loc_side = new_loc.clone()
                new_loc.record_stream(side)
                for a in new_adapters:
                    # weights produced on the main stream and read by kernels queued on the side stream
                    for name in ("lora_A", "lora_B"):
                        for per_layer in getattr(a, name, None) or ():
                            for m in (per_layer if isinstance(per_layer, (list, tuple)) else (per_layer,)):
                                if torch.is_tensor(m) and m.is_cuda:
                                    m.record_stream(side)
                copy_all(loc_side)
        else:
            copy_all(new_loc)

    def offload_adapters(self, reserve_adapter_dirs) -> None:
        if len(reserve_adapter_dirs) == len(self.adapter_dirs):
            return
        dev = self.a_loc.device
        if len(reserve_adapter_dirs) == 0:
            self.mem_manager.free(self.a_loc)
            self.adapter_dirs = []
            self.a_loc = torch.empty(0, dtype=torch.long, device=dev)
            self.a_start = torch.empty(0, dtype=torch.long, device=dev)
            self.a_len = torch.empty(0, dtype=torch.long, device=dev)
            self.a_scaling = torch.empty(0, dtype=torch.float16, device=dev)
            self.idx_map = {}
            self.len_host = []
            return
        keep, new_dirs, idx_map = [], [], {}
        for d in self.adapter_dirs:
            drop = d not in reserve_adapter_dirs and self.prefetch_tag.get(d) != self.cur_tag
            keep.append(not drop)
            if not drop:
                idx_map[d] = len(new_dirs)
                new_dirs.append(d)
        if all(keep):
            return
        self.idx_map = idx_map
        self.adapter_dirs = new_dirs
        self.len_host = [n for n, k in zip(self.len_host, keep) if k]
        # a_len[left_ind], cumsum, a_scaling[left_ind], var_len_copy and the cat of the removed lists, one launch
        self.a_start, self.a_len, self.a_loc, self.a_scaling, remove_ind = compact_adapter_tables(
            self.a_start, self.a_len, self.a_loc, self.a_scaling, torch.tensor(keep, dtype=torch.bool, device=dev))
        self.mem_manager.free(remove_ind)

    def start_and_rank(self, lora_dir: str):
        """``(a_start[i], a_len[i] // 4)`` of a loaded adapter from the host copy of the tables
        (no device read-back): what ``merge_adapter`` needs to find its pages."""
        i = self.idx_map[lora_dir]
        return sum(self.len_host[:i]), self.len_host[i] // 4

    def merge_adapter(self, weights, layer_id: int, lora_dir: str, sign: float = 1.0) -> None:
        """``weights[p] += sign * scaling * A_p B_p`` for the q, k, v, o matrices of one layer
        (slora/models/peft/lora_single_batch_infer.py:60-93) from the adapter's pool pages."""
        start, rank = self.start_and_rank(lora_dir)
        merge_adapter(weights, self.mem_manager.key_buffer[layer_id], self.mem_manager.value_buffer[layer_id],
                      self.a_start, self.a_len, self.a_loc, self.a_scaling, self.idx_map[lora_dir], sign=sign,
                      start=start, rank=rank)
