"""The LoRA half of the reference's batch engine
(slora/models/peft/lora_unordered_batch_infer.py:16-483): per inference step the
``delta`` buffers, the choice between the segmented (prefill) kernels and the
per-token BGMV kernels, and per layer the shrink + expand of the q, k, v and o
projections on top of the base model's matmul outputs.

The base model (matmuls, rotary embedding, attention, FFN) is the caller's: it
computes ``q``, ``cache_k``, ``cache_v`` / ``o`` with its own weights and hands
them to ``lora_get_qkv`` / ``lora_get_o``, which add the adapters' deltas in
place -- exactly what the reference does between its ``torch.mm`` calls and the
rotary embedding (:254-318 decode, :321-408 prefill, :411-483 o projection).

Two ways to issue the work, same results bit for bit:

* ``fused=False``: the reference's call sequence, one ``dispatch_bgmv`` or
  ``lora_get_qkvo_fwd_*`` call per projection and direction (8 per layer),
  ``delta[0]`` shared by q and o as in the reference;
* ``fused=True`` (default): q, k and v of a layer in one shrink launch (which reads
  the activations once) and one expand launch, in decode and in prefill steps.

Either way the first call of a step builds the batch's plan inside the library and
the other calls of the step reuse it (the index tensors are the same objects in
every call of a step); nothing here waits for the device.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ._kernels import (dispatch_bgmv, dispatch_bgmv_qkv_expand, dispatch_bgmv_qkv_shrink, lora_get_qkvo_fwd_expand,
                       lora_get_qkvo_fwd_expand_qkv, lora_get_qkvo_fwd_shrink, lora_get_qkvo_fwd_shrink_qkv)

# lora_unordered_batch_infer.py:334: the segmented kernels serve batches with a long
# request, adapters of rank >= 64 and at least two requests; everything else is BGMV
PREFILL_MIN_SEQ_LEN = 200
PREFILL_MIN_LORA_DIM = 64
PREFILL_MIN_REQUESTS = 2


class LoraUnorderedBatchInfer:
    """One object per batch, as in the reference (model_rpc.py:234 builds it per step).

    ``infer_adapter``: the tables ``a_loc / a_start / a_len / a_scaling``, ``adapter_dirs`` /
    ``idx_map`` and the pool as ``mem_manager.key_buffer / value_buffer`` or, like the reference's
    ``NaiveInferAdapter``, as ``key_buffer / value_buffer`` of its own (``slora_hip.InferAdapter`` or
    anything with those attributes).  ``adapters``: per request an object with ``lora_dir``
    and ``r`` (the reference's ``LoraTpPartAdapter``); ``None`` entries (requests on the bare
    base model, which the reference does not support either, :35-36) are rejected."""

    def __init__(self, infer_adapter, adapters: Sequence, kv_embed_dim: Optional[int] = None, fused: bool = True,
                 delta_dtype: Optional[torch.dtype] = None):
        if any(a is None for a in adapters):
            raise ValueError("requests without an adapter are not supported (as in the reference)")
        self.infer_adapter = infer_adapter
        # the pool's buffers: on the adapter table itself (the reference's NaiveInferAdapter, :28-30)
        # or on its memory manager (:31-33)
        owner = infer_adapter if hasattr(infer_adapter, "key_buffer") else infer_adapter.mem_manager
        self.key_buffer: List[torch.Tensor] = owner.key_buffer
        self.value_buffer: List[torch.Tensor] = owner.value_buffer
        dev = self.key_buffer[0].device
        self.max_lora_dim = max((int(a.r) for a in adapters), default=0)
        idx_map = getattr(infer_adapter, "idx_map", None)
        if idx_map:  # one dictionary lookup per request; the reference searches the list (:37)
            ids = [idx_map[a.lora_dir] for a in adapters]
        else:
            ids = [infer_adapter.adapter_dirs.index(a.lora_dir) for a in adapters]
        self.req_bins = torch.tensor(ids, dtype=torch.long, device=dev)
        kb = self.key_buffer[0]
        self.page_elems = int(kb.shape[1] * kb.shape[2])
        self.kv_embed_dim = int(kv_embed_dim) if kv_embed_dim is not None else self.page_elems
        self.fused = bool(fused)
        self.delta_dtype = delta_dtype or kb.dtype
        self.delta: List[torch.Tensor] = []
        self.is_prefill = False
        self.use_segmented = False
        self.batch_req_bins: Optional[torch.Tensor] = None
        self.max_b_seq_len = 0
        self._bins: Optional[torch.Tensor] = None

    # ---- per step (forward(), :44-80) -----------------------------------------------------
    def begin_step(self, b_start_loc: torch.Tensor, b_seq_len: torch.Tensor, is_prefill: bool,
                   max_b_seq_len: Optional[int] = None, total_token_num: Optional[int] = None) -> None:
        """The per-step part of ``forward``: ``delta`` (three zeroed ``[tokens, max_lora_dim]``
        buffers, :69 / :76), per-token adapter ids for a prefill batch (:66) and the kernel choice
        (:334).  ``max_b_seq_len`` spares the read-back of ``torch.max(b_seq_len).item()`` (:61)
        and ``total_token_num`` (the sum of ``b_seq_len``, an argument of the reference's ``forward``)
        the one inside ``repeat_interleave``, when the caller knows them: the step then starts
        without waiting for the device."""
        assert b_start_loc.shape[0] == b_seq_len.shape[0] == self.req_bins.shape[0]
        self.is_prefill = bool(is_prefill)
        self.b_start_loc, self.b_seq_len = b_start_loc, b_seq_len
        self.max_b_seq_len = int(max_b_seq_len) if max_b_seq_len is not None else int(torch.max(b_seq_len).item())
        n_req = int(b_seq_len.shape[0])
        if self.is_prefill:
            self.batch_req_bins = torch.repeat_interleave(self.req_bins, b_seq_len.to(torch.long),
                                                          output_size=total_token_num)
            n_tok = int(self.batch_req_bins.shape[0])
            self.use_segmented = (self.max_b_seq_len >= PREFILL_MIN_SEQ_LEN and
                                  self.max_lora_dim >= PREFILL_MIN_LORA_DIM and n_req >= PREFILL_MIN_REQUESTS)
            self._bins = self.batch_req_bins
        else:
            self.batch_req_bins = None
            n_tok = n_req
            self.use_segmented = False
            self._bins = self.req_bins
        dev = self.req_bins.device
        self.delta = [torch.zeros((n_tok, self.max_lora_dim), dtype=self.delta_dtype, device=dev) for _ in range(3)]

    # ---- q, k, v of one layer (:254-318 decode, :321-408 prefill) --------------------------
    def lora_get_qkv(self, layer_id: int, input_embs: torch.Tensor, q: torch.Tensor, cache_k: torch.Tensor,
                     cache_v: torch.Tensor) -> None:
        """``q / cache_k / cache_v += scaling * (input_embs A_p) B_p`` for p = q, k, v with every
        token's own adapter.  ``input_embs``: ``[tokens, hidden]``; the three outputs 2-D views
        ``[tokens, h_out]`` that already hold the base model's projections (``cache_k`` /
        ``cache_v`` may be row slices of the pool itself, transformer_layer_infer_template.py:39-41)."""
        ia = self.infer_adapter
        key, val = self.key_buffer[layer_id], self.value_buffer[layer_id]
        d = self.delta
        outs = (q, cache_k, cache_v)
        if self.max_lora_dim == 0 or input_embs.shape[0] == 0:
            return
        if self.use_segmented:
            key2, val2 = key.view(-1, self.page_elems), val.view(-1, self.page_elems)
            seg = (ia.a_loc, ia.a_start, ia.a_len, self.b_start_loc, self.b_seq_len, self.req_bins)
            hidden = int(input_embs.shape[1])
            if self.fused:
                lora_get_qkvo_fwd_shrink_qkv(input_embs, key2, d[0], d[1], d[2], *seg, hidden, self.max_lora_dim,
                                             self.max_b_seq_len)
            else:
                for p in range(3):
                    lora_get_qkvo_fwd_shrink(input_embs, key2, d[p], *seg, hidden, p, self.max_lora_dim,
                                             self.max_b_seq_len)
            if self.fused and cache_k.shape == cache_v.shape and cache_k.stride(0) == cache_v.stride(0):
                lora_get_qkvo_fwd_expand_qkv(d[0], d[1], d[2], val2, q, cache_k, cache_v, ia.a_scaling, *seg,
                                             int(q.shape[1]), int(cache_k.shape[1]), self.max_lora_dim,
                                             self.max_b_seq_len)
                return
            for p in range(3):
                lora_get_qkvo_fwd_expand(d[p], val2, outs[p], ia.a_scaling, *seg, int(outs[p].shape[1]), p,
                                         self.max_lora_dim, self.max_b_seq_len)
            return
        tabs = (ia.a_start, ia.a_len, ia.a_loc, self._bins)
        if self.fused:
            dispatch_bgmv_qkv_shrink(d[0], d[1], d[2], input_embs, key, *tabs)
            dispatch_bgmv_qkv_expand(q, cache_k, cache_v, d[0], d[1], d[2], val, *tabs, ia.a_scaling)
        else:
            for p in range(3):
                dispatch_bgmv(d[p], input_embs, key, *tabs, p, ia.a_scaling)
                dispatch_bgmv(outs[p], d[p], val, *tabs, p, ia.a_scaling)

    # ---- o of one layer (:411-483) ---------------------------------------------------------
    def lora_get_o(self, layer_id: int, input: torch.Tensor, o: torch.Tensor) -> None:
        """``o += scaling * (input A_o) B_o``; ``delta[0]`` is reused, as in the reference (:421, :447)."""
        ia = self.infer_adapter
        key, val = self.key_buffer[layer_id], self.value_buffer[layer_id]
        d = self.delta[0]
        if self.max_lora_dim == 0 or input.shape[0] == 0:
            return
        if self.use_segmented:
            key2, val2 = key.view(-1, self.page_elems), val.view(-1, self.page_elems)
            seg = (ia.a_loc, ia.a_start, ia.a_len, self.b_start_loc, self.b_seq_len, self.req_bins)
            lora_get_qkvo_fwd_shrink(input, key2, d, *seg, int(input.shape[1]), 3, self.max_lora_dim,
                                     self.max_b_seq_len)
            lora_get_qkvo_fwd_expand(d, val2, o, ia.a_scaling, *seg, int(o.shape[1]), 3, self.max_lora_dim,
                                     self.max_b_seq_len)
            return
        tabs = (ia.a_start, ia.a_len, ia.a_loc, self._bins)
        dispatch_bgmv(d, input, key, *tabs, 3, ia.a_scaling)
        dispatch_bgmv(o, d, val, *tabs, 3, ia.a_scaling)
