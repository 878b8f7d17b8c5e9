"""CPU restatement of S-LoRA's heterogeneous multi-LoRA batching math.

THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are
compared against; only tests, the smoke check and the benchmark's CPU-baseline
leg may import it.  Nothing in the product path calls it.

Every function restates one piece of the reference (citations are relative to
the reference checkout):

* ``pack_w_combined``      slora/models/peft/layer_weights/lora_layer_weight.py:84-93, 215-224
* ``unpack_from_pool``     slora/models/peft/lora_single_batch_infer.py:38-57   (independent inverse)
* ``build_tables``         slora/server/router/model_infer/infer_adapter.py:128-146
* ``load_into_pool``       slora/server/router/model_infer/infer_adapter.py:56-57, 81-82
* ``ref_bmm``              slora/models/bmm/lora_bmm_infer.py:33-50, 278-330  ("S-LoRA-bmm")
* ``ref_bgmv_shrink``      slora/csrc/bgmv/bgmv_impl.cuh:14-149
* ``ref_bgmv_expand``      slora/csrc/bgmv/bgmv_impl.cuh:152-208
* ``ref_prefill_shrink``   slora/models/peft/triton_kernel/lora/lora_prefill.py:57-102, 139-164
* ``ref_prefill_expand``   slora/models/peft/triton_kernel/lora/lora_prefill.py:10-54, 105-136
* ``ref_var_len_copy``     slora/server/router/model_infer/infer_adapter.py:261-280

Pinning (see tests/test_oracle.py): pack/unpack are inverse statements of the
pool layout taken from two different reference files; the paged restatements
(index arithmetic over ``a_loc``) must agree with the dense closed form
``y + scale * (x @ A) @ B`` evaluated in float64 by numpy, with the reference's
own executable specs (test/kernel/test_kernel_correctness.py:87-95 and
test_kernel_correctness_multi_rank.py:97-106) and with integer-exact one-hot
cases in which any wrong page, wrong ``r*qkvo`` offset or wrong ``n*r+d``
split changes bits.

Arrays are float32 ndarrays whose values are already representable in the
storage type ``dtype`` ("f16", "bf16" or "f32"); rounding to the storage type
happens exactly where the reference rounds.
"""
from __future__ import annotations

import numpy as np

DTYPES = ("f16", "bf16", "f32")


# ----------------------------------------------------------------------------
# storage-type rounding
# ----------------------------------------------------------------------------
def round_to(a, dtype: str) -> np.ndarray:
    """Round float32 values to the storage type (round-to-nearest-even) and
    return them as float32."""
    a = np.asarray(a, dtype=np.float32)
    if dtype == "f32":
        return a.copy()
    if dtype == "f16":
        with np.errstate(over="ignore"):
            return a.astype(np.float16).astype(np.float32)
    if dtype == "bf16":
        flat = np.ascontiguousarray(a).reshape(-1)
        u = flat.view(np.uint32).astype(np.uint64)
        lsb = (u >> 16) & 1
        u = (u + 0x7FFF + lsb) & 0xFFFF0000
        out = u.astype(np.uint32).view(np.float32).copy()
        out[np.isnan(flat)] = np.nan
        return out.reshape(a.shape)
    raise ValueError(f"unknown dtype {dtype!r}")


# ----------------------------------------------------------------------------
# pool layout: packing, tables, loading, unpacking
# ----------------------------------------------------------------------------
def pack_w_combined(A, B, page_elems: int) -> np.ndarray:
    """Build one layer's ``w_combined`` for one adapter.

    ``A[p]`` has shape (H_in, r) (so ``x @ A[p]`` is the shrink) and ``B[p]``
    has shape (r, H_out_p), p in q,k,v,o.  Returns ``[2, 4r, page_elems]``:

    * ``[0, p*r + j]`` = ``A[p][:, j]``  -- ``A.T.reshape(r, heads, -1)`` of
      lora_layer_weight.py:85-88;
    * ``[1, p*r : (p+1)*r]`` = the (H_out, r) row-major matrix ``B[p].T``
      flattened and cut into pages -- ``B.T.reshape(r, heads, -1)`` of
      lora_layer_weight.py:89-92 (``.T`` is a non-contiguous view, so
      ``reshape`` walks it in logical (H_out, r) order).

    The reference only has H_in == H_out == page_elems.  When H_out*r is
    smaller than r pages (grouped-query k/v), the flattened matrix fills the
    first H_out*r/page_elems pages of the projection's r-page slot and the
    rest stay zero.
    """
    r = A[0].shape[1]
    out = np.zeros((2, 4 * r, page_elems), dtype=np.float32)
    for p in range(4):
        a = np.asarray(A[p], dtype=np.float32)
        b = np.asarray(B[p], dtype=np.float32)
        assert a.shape[1] == r and b.shape[0] == r
        h_in = a.shape[0]
        assert h_in <= page_elems
        out[0, p * r:(p + 1) * r, :h_in] = a.T
        flat = np.ascontiguousarray(b.T).reshape(-1)  # (H_out, r) row-major
        assert flat.size <= r * page_elems
        slot = out[1, p * r:(p + 1) * r].reshape(-1)
        slot[:flat.size] = flat
    return out


def build_tables(ranks, new_loc):
    """Index tables of infer_adapter.py:128-146 for adapters loaded in one go.

    ``new_loc`` is what the pool allocator handed out (sum(4*r) page ids).
    Returns int64 ``a_start, a_len, a_loc``.
    """
    ranks = [int(r) for r in ranks]
    a_len = np.array([4 * r for r in ranks], dtype=np.int64)
    a_start = np.zeros(len(ranks), dtype=np.int64)
    cum = 0
    for i, r in enumerate(ranks):
        a_start[i] = cum
        cum += 4 * r
    new_loc = np.asarray(new_loc, dtype=np.int64)
    assert new_loc.size == cum
    return a_start, a_len, new_loc.copy()


def load_into_pool(key_buffer, value_buffer, w_combined, loc):
    """``key_buffer[loc] = w_combined[0]; value_buffer[loc] = w_combined[1]``
    (infer_adapter.py:56-57, 81-82).  Buffers are [pages, page_elems]."""
    key_buffer[loc] = w_combined[0]
    value_buffer[loc] = w_combined[1]


def unpack_from_pool(key_buffer, value_buffer, loc, h_in: int, h_out):
    """Inverse of pack+load, restating lora_single_batch_infer.py:38-57:
    ``A_p = key[loc[p r:(p+1) r]].reshape(r, H).T`` and
    ``B_p = value[loc[p r:(p+1) r]].reshape(H, r).T``.
    ``h_out`` is a 4-sequence of output widths."""
    loc = np.asarray(loc, dtype=np.int64)
    r = loc.size // 4
    A, B = [], []
    for p in range(4):
        pages = loc[p * r:(p + 1) * r]
        A.append(key_buffer[pages][:, :h_in].reshape(r, h_in).T.copy())
        flat = value_buffer[pages].reshape(-1)[: h_out[p] * r]
        B.append(flat.reshape(h_out[p], r).T.copy())
    return A, B


# ----------------------------------------------------------------------------
# dense semantics ("S-LoRA-bmm")
# ----------------------------------------------------------------------------
def ref_bmm(y, x, A, B, scaling, bins, dtype: str = "f32"):
    """Gather + zero-padded bmm + scatter-add (lora_bmm_infer.py:285-299).

    ``A[i]``: (H_in, r_i), ``B[i]``: (r_i, H_out) for adapter i; ``bins[t]`` is
    token t's adapter.  Tokens of one adapter need not be adjacent (the
    reference run-length-compresses ``adapter_dirs`` so they are; a gather by
    index is the same thing for any order).  Rounding chain of the reference
    in a 16-bit type: xA -> T, (xA)B -> T, *scale -> T, += -> T.
    """
    y = np.array(y, dtype=np.float32)
    x = np.asarray(x, dtype=np.float32)
    bins = np.asarray(bins, dtype=np.int64)
    n_adapters = len(A)
    max_r = max(a.shape[1] for a in A)
    h_in, h_out = x.shape[1], y.shape[1]
    counts = [int((bins == i).sum()) for i in range(n_adapters)]
    max_tok = max(counts + [1])
    pad_A = np.zeros((n_adapters, h_in, max_r), dtype=np.float32)
    pad_B = np.zeros((n_adapters, max_r, h_out), dtype=np.float32)
    emb = np.zeros((n_adapters, max_tok, h_in), dtype=np.float32)
    for i in range(n_adapters):
        r = A[i].shape[1]
        pad_A[i, :, :r] = A[i]
        pad_B[i, :r, :] = B[i]
        idx = np.nonzero(bins == i)[0]
        emb[i, : idx.size] = x[idx]
    xa = round_to(np.matmul(emb, pad_A), dtype)
    delta = round_to(np.matmul(xa, pad_B), dtype)
    for i in range(n_adapters):
        idx = np.nonzero(bins == i)[0]
        if idx.size == 0:
            continue
        s = round_to(np.float32(scaling[i]), dtype)
        upd = round_to(delta[i, : idx.size] * s, dtype)
        y[idx] = round_to(y[idx] + upd, dtype)
    return y


def dense_lora_f64(y, x, A, B, scaling, bins):
    """Closed form in float64, no intermediate rounding: the textbook value
    every other function here must approach."""
    out = np.array(y, dtype=np.float64)
    x = np.asarray(x, dtype=np.float64)
    for t in range(x.shape[0]):
        i = int(bins[t])
        out[t] += float(scaling[i]) * ((x[t] @ A[i].astype(np.float64)) @ B[i].astype(np.float64))
    return out


# ----------------------------------------------------------------------------
# paged decode semantics (BGMV)
# ----------------------------------------------------------------------------
def ref_bgmv_shrink(y, x, w, a_start, a_len, a_loc, bins, qkvo: int, dtype: str = "f16"):
    """bgmv_multi_lora_rank_shrink_kernel (bgmv_impl.cuh:14-149).

    ``w`` is the pool viewed as [pages, page_elems].  For token b with adapter
    a = bins[b], r = a_len[a] // 4 and j < r:
    ``y[b, j] = T( sum_k f32(w[a_loc[a_start[a] + r*qkvo + j], k]) * f32(x[b, k]) )``.
    Columns j >= r keep their previous value (the kernel returns early,
    bgmv_impl.cuh:36); no scaling is applied.
    """
    y = np.array(y, dtype=np.float32)
    x = np.asarray(x, dtype=np.float32)
    h_in = x.shape[1]
    for b in range(x.shape[0]):
        a = int(bins[b])
        r = int(a_len[a]) // 4
        r_eff = min(r, y.shape[1])
        if r_eff == 0:
            continue
        base = int(a_start[a]) + r * qkvo
        pages = np.asarray(a_loc[base: base + r_eff], dtype=np.int64)
        rows = w[pages][:, :h_in].astype(np.float32)
        acc = (rows.astype(np.float64) @ x[b].astype(np.float64)).astype(np.float32)
        y[b, :r_eff] = round_to(acc, dtype)
    return y


def ref_bgmv_expand(y, x, w, a_start, a_len, a_loc, bins, qkvo: int, scales, dtype: str = "f16"):
    """bgmv_multi_lora_rank_expand_kernel (bgmv_impl.cuh:152-208).

    For output n and rank index d the weight is element ``n*r + d`` of the
    projection's r pages laid end to end: page ``a_loc[a_start[a] + r*qkvo +
    (n*r+d) // page_elems]``, offset ``(n*r+d) % page_elems`` (:174-178,
    :191 with page stride == feat_out in the reference).  Each product is
    scaled inside the float32 sum (:194-198); the sum is rounded to T and added
    to y in T (:205-207).
    """
    y = np.array(y, dtype=np.float32)
    x = np.asarray(x, dtype=np.float32)
    page_elems = w.shape[1]
    h_out = y.shape[1]
    for b in range(x.shape[0]):
        a = int(bins[b])
        r = int(a_len[a]) // 4
        r_eff = min(r, x.shape[1])
        if r_eff == 0:
            continue
        base = int(a_start[a]) + r * qkvo
        n_pages = -(-(h_out * r) // page_elems)
        pages = np.asarray(a_loc[base: base + n_pages], dtype=np.int64)
        flat = w[pages].reshape(-1)[: h_out * r].astype(np.float32)
        wt = flat.reshape(h_out, r)[:, :r_eff]                 # (H_out, r) row-major
        s = np.float32(scales[a])
        xs = (x[b, :r_eff] * s).astype(np.float32)
        acc = (wt.astype(np.float64) @ xs.astype(np.float64)).astype(np.float32)
        y[b] = round_to(y[b] + round_to(acc, dtype), dtype)
    return y


# ----------------------------------------------------------------------------
# paged prefill semantics (segmented shrink / expand)
# ----------------------------------------------------------------------------
def ref_prefill_shrink(o, x, w, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len,
                       b_indicies, qkvo: int, max_rank: int, dtype: str = "f16"):
    """_shrink_fwd_kernel (lora_prefill.py:57-102).  Request i owns rows
    ``b_start_loc[i] + [0, b_seq_len[i])``; ``o[rows, j] = T(sum_k x[rows,k] *
    w[b_loc[start + r*qkvo + j], k])`` for j < r and **0 for r <= j < max_rank**
    (masked weight columns load as 0 and the store mask is row-only, :93,:100).
    Rows not owned by any request are left alone."""
    o = np.array(o, dtype=np.float32)
    x = np.asarray(x, dtype=np.float32)
    h_in = x.shape[1]
    for i in range(len(b_seq_len)):
        a = int(b_indicies[i])
        r = int(b_lora_ranks[a]) // 4
        n = int(b_seq_len[i])
        s = int(b_start_loc[i])
        if n == 0:
            continue
        r_eff = min(r, max_rank)
        base = int(b_lora_start[a]) + r * qkvo
        o[s:s + n, :max_rank] = 0.0
        if r_eff:
            pages = np.asarray(b_loc[base: base + r_eff], dtype=np.int64)
            rows = w[pages][:, :h_in].astype(np.float64)
            acc = (x[s:s + n].astype(np.float64) @ rows.T).astype(np.float32)
            o[s:s + n, :r_eff] = round_to(acc, dtype)
    return o


def ref_prefill_expand(o, x, w, scale, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len,
                       b_indicies, qkvo: int, max_rank: int, dtype: str = "f16"):
    """_expand_fwd_kernel (lora_prefill.py:10-54): ``o[rows, n] = T( f32(o[rows,n])
    + (sum_{d<r} x[rows,d] * Wflat[n*r+d]) * scale[a] )`` with the same flat
    (H_out, r) indexing as the decode expand (:42-43).  Columns d >= r of x are
    ignored (weight mask, :44)."""
    o = np.array(o, dtype=np.float32)
    x = np.asarray(x, dtype=np.float32)
    page_elems = w.shape[1]
    h_out = o.shape[1]
    for i in range(len(b_seq_len)):
        a = int(b_indicies[i])
        r = int(b_lora_ranks[a]) // 4
        n = int(b_seq_len[i])
        s = int(b_start_loc[i])
        r_eff = min(r, max_rank)
        if n == 0 or r_eff == 0:
            continue
        base = int(b_lora_start[a]) + r * qkvo
        n_pages = -(-(h_out * r) // page_elems)
        pages = np.asarray(b_loc[base: base + n_pages], dtype=np.int64)
        flat = w[pages].reshape(-1)[: h_out * r].astype(np.float64)
        wt = flat.reshape(h_out, r)[:, :r_eff]
        dot = (x[s:s + n, :r_eff].astype(np.float64) @ wt.T).astype(np.float32)
        sc = np.float32(scale[a])
        o[s:s + n] = round_to(o[s:s + n] + dot * sc, dtype)
    return o


# ----------------------------------------------------------------------------
# index-table compaction on offload
# ----------------------------------------------------------------------------
def ref_var_len_copy(old_a_start, old_a_len, old_a_loc, new_a_start, new_size: int):
    """What launch_var_len_copy_triton is for (infer_adapter.py:236-237,
    261-280): ``new_loc[new_start[i] + k] = old_loc[old_start[i] + k]`` for
    k < len[i].  (The reference's mask ``offset < length`` over-copies for
    lengths above its block of 256; the over-copied tail is overwritten by the
    next adapter or lies past the end, so the intended result is this one.)"""
    out = np.zeros(new_size, dtype=np.int64)
    for i in range(len(old_a_len)):
        n = int(old_a_len[i])
        out[int(new_a_start[i]): int(new_a_start[i]) + n] = old_a_loc[int(old_a_start[i]): int(old_a_start[i]) + n]
    return out


def ref_offload_tables(a_start, a_len, a_loc, a_scaling, keep):
    """The table rebuild of ``InferAdapter.offload_adapters``
    (infer_adapter.py:206-258) with ``keep[i]`` standing for "adapter i is in
    reserve_adapter_dirs or carries the current prefetch tag" (:207-215).

    Returns ``(new_a_start, new_a_len, new_a_loc, new_a_scaling, remove_ind)``:
    ``new_a_len = a_len[left_ind]`` (:238), ``new_a_start`` its exclusive running
    sum (:239-240), ``new_a_scaling = a_scaling[left_ind]`` (:241), ``new_a_loc``
    the kept lists copied by var_len_copy (:243-244), ``remove_ind`` the removed
    adapters' lists concatenated in order (:210, :224), which is what goes to
    ``mem_manager.free``."""
    a_start = np.asarray(a_start, dtype=np.int64)
    a_len = np.asarray(a_len, dtype=np.int64)
    a_loc = np.asarray(a_loc, dtype=np.int64)
    left = [i for i in range(len(a_len)) if keep[i]]
    gone = [i for i in range(len(a_len)) if not keep[i]]
    new_len = a_len[left] if left else np.zeros(0, np.int64)
    new_start = np.zeros(len(left), dtype=np.int64)
    if len(left) > 1:
        new_start[1:] = np.cumsum(new_len)[:-1]
    new_loc = ref_var_len_copy(a_start[left], new_len, a_loc, new_start, int(new_len.sum())) if left else \
        np.zeros(0, np.int64)
    removed = [a_loc[int(a_start[i]): int(a_start[i]) + int(a_len[i])] for i in gone]
    removed = np.concatenate(removed) if removed else np.zeros(0, np.int64)
    return new_start, new_len, new_loc, np.asarray(a_scaling)[left], removed


def ref_merge_adapter(W, A, B, scaling: float, sign: float = 1.0, dtype: str = "f16"):
    """``LoraPEFTBatchInfer.merge_adapter`` / ``unmerge_adapter`` for one projection
    (lora_single_batch_infer.py:60-93) with the reference's rounding points:
    ``b = T(B * scaling)`` (:68), ``ab = T(A @ b)`` (float accumulate inside bmm,
    :69), ``W = T(W +- ab)`` (:72-75).  ``W``: (H, H_out), ``A``: (H, r), ``B``:
    (r, H_out); returns the new W as float32 holding storage-type values."""
    b = round_to(np.asarray(B, np.float32) * np.float32(scaling), dtype)
    ab = round_to((np.asarray(A, np.float64) @ b.astype(np.float64)).astype(np.float32), dtype)
    return round_to(np.asarray(W, np.float32) + np.float32(sign) * ab, dtype)


# ----------------------------------------------------------------------------
# page allocator over the free map (slora/common/mem_allocator.py)
# ----------------------------------------------------------------------------
def ref_alloc(mem_state, need_size: int):
    """``MemoryAllocator.alloc`` (mem_allocator.py:30-39) on a 0/1 numpy map
    (1 = free), in place: ``select = (cumsum(mem_state) <= need_size) &
    (mem_state == 1)``; the selected pages are marked used and returned."""
    cum = np.cumsum(mem_state.astype(np.int64))
    select = np.nonzero((cum <= need_size) & (mem_state == 1))[0].astype(np.int64)
    mem_state[select] = 0
    return select


def ref_alloc_contiguous(mem_state, need_size: int):
    """``MemoryAllocator.alloc_contiguous`` (mem_allocator.py:42-59), in place:
    window sums from the running sum, the first start whose window of
    ``need_size`` pages is all free; ``None`` if there is none, else
    ``(select_index, start, end)``."""
    tot = mem_state.size
    if need_size > tot:
        return None
    cum = np.cumsum(mem_state.astype(np.int64))
    loc_sums = cum[need_size - 1:tot] - cum[0:tot - need_size + 1] + mem_state[0:tot - need_size + 1]
    can_use = np.nonzero(loc_sums == need_size)[0]
    if can_use.size == 0:
        return None
    start = int(can_use[0])
    select = np.arange(start, start + need_size, dtype=np.int64)
    mem_state[select] = 0
    return select, start, start + need_size


def ref_free(mem_state, free_index):
    """``MemoryAllocator.free`` (mem_allocator.py:185-199): ``mem_state[free_index] = 1``."""
    mem_state[np.asarray(free_index, dtype=np.int64)] = 1


# ----------------------------------------------------------------------------
# the reference's torch path on host cores (CPU baseline of the benchmark)
# ----------------------------------------------------------------------------
class BmmCpuLayer:
    """One layer of LoraBmmInfer on the CPU in torch float32: the padded
    ``batch_lora_A [4, n, H, max_r]`` / ``batch_lora_B [4, n, max_r, H_out]``
    are built once (lora_bmm_infer.py:33-50); ``decode`` is
    ``_batch_lora_get_qkv`` + ``_batch_lora_get_o`` without the base matmuls
    (:285-299, :393-415): copy each adapter's tokens into the padded batch,
    ``bmm(bmm(emb, A), B)``, then ``y[tokens] += delta * scaling``.

    ``A[i][p]``: (H, r_i), ``B[i][p]``: (r_i, H_out_p) as numpy arrays for the
    adapters that appear in the batch (the reference is handed exactly those).
    """

    def __init__(self, A, B, scaling, bins, threads=None):
        import torch
        if threads:
            torch.set_num_threads(int(threads))
        self.torch = torch
        n = len(A)
        max_r = max(a[0].shape[1] for a in A)
        h = A[0][0].shape[0]
        self.h_out = [B[0][p].shape[1] for p in range(4)]
        self.pad_A = [torch.zeros((n, h, max_r), dtype=torch.float32) for _ in range(4)]
        self.pad_B = [torch.zeros((n, max_r, self.h_out[p]), dtype=torch.float32) for p in range(4)]
        for i in range(n):
            r = A[i][0].shape[1]
            for p in range(4):
                self.pad_A[p][i, :, :r] = torch.from_numpy(np.ascontiguousarray(A[i][p]))
                self.pad_B[p][i, :r, :] = torch.from_numpy(np.ascontiguousarray(B[i][p]))
        bins = np.asarray(bins)
        self.idx = [torch.from_numpy(np.nonzero(bins == i)[0]) for i in range(n)]
        self.scaling = [float(s) for s in scaling]
        max_tok = max(int(ix.numel()) for ix in self.idx)
        self.emb = torch.zeros((n, max_tok, h), dtype=torch.float32)

    def _proj(self, p, x, y):
        torch = self.torch
        for i, ix in enumerate(self.idx):
            self.emb[i, : ix.numel()] = x[ix]
        delta = torch.bmm(torch.bmm(self.emb, self.pad_A[p]), self.pad_B[p])
        for i, ix in enumerate(self.idx):
            y[ix] += delta[i, : ix.numel()] * self.scaling[i]

    def decode(self, x_in, x_att, ys):
        """q, k, v from ``x_in``; o from ``x_att``; ``ys`` are updated in place."""
        for p in range(3):
            self._proj(p, x_in, ys[p])
        self._proj(3, x_att, ys[3])
