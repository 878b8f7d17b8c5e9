"""Synthetic multi-LoRA workloads built directly on the device: a unified paged
pool per layer (adapter pages scattered among KV pages), the adapter index
tables and a batch.  Used by the benchmark and by the full-size GPU tests.

The shapes follow the reference's dummy configurations (slora/mprophet/
model_config.py:117-130, lora_config.py:107-146) and its scattered-pool
micro-benchmark fixture (slora/models/peft/triton_kernel/tests/bench_ops.py:118-126):
pool pages are handed out from a seeded random permutation, the same page ids
for every layer, exactly as InferAdapter copies one adapter into the same
``loc`` of every layer's buffer (infer_adapter.py:49-57).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List

import numpy as np
import torch


@dataclass
class DecodeWorkload:
    name: str
    hidden: int
    h_out: List[int]            # q, k, v, o output widths
    n_layers: int
    ranks: np.ndarray           # [n_adapters]
    bins_np: np.ndarray         # [batch] adapter of every token
    a_start_np: np.ndarray
    a_len_np: np.ndarray
    a_loc_np: np.ndarray
    scales_np: np.ndarray
    page_elems: int
    n_pages: int
    dtype: torch.dtype
    key_buffer: list = field(default_factory=list)    # per layer [n_pages, heads, head_dim]  (LoRA A + K cache)
    value_buffer: list = field(default_factory=list)  # per layer                             (LoRA B + V cache)
    a_start: torch.Tensor = None
    a_len: torch.Tensor = None
    a_loc: torch.Tensor = None
    a_scaling: torch.Tensor = None
    req_bins: torch.Tensor = None
    max_rank: int = 0

    @property
    def batch(self) -> int:
        return int(self.bins_np.size)

    # ---- algorithmic (compulsory) bytes, per call --------------------------------
    def distinct_adapters(self) -> np.ndarray:
        return np.unique(self.bins_np)

    def shrink_bytes(self, h_in=None) -> int:
        """sum_{a in U} r_a*H*s + B*H*s + sum_t r_t*s + index traffic."""
        s = 2
        h = h_in or self.hidden
        u = self.distinct_adapters()
        r_u = self.ranks[u]
        r_t = self.ranks[self.bins_np]
        return int(r_u.sum() * h * s + self.batch * h * s + r_t.sum() * s + self._index_bytes(u))

    def expand_bytes(self, h_out) -> int:
        """sum_{a in U} r_a*H_out*s + sum_t r_t*s + 2*B*H_out*s + index traffic."""
        s = 2
        u = self.distinct_adapters()
        r_u = self.ranks[u]
        r_t = self.ranks[self.bins_np]
        return int(r_u.sum() * h_out * s + r_t.sum() * s + 2 * self.batch * h_out * s + self._index_bytes(u))

    def _index_bytes(self, u) -> int:
        return int(self.batch * 8 + u.size * (16 + 2) + self.ranks[u].sum() * 8)

    def qkv_shrink_bytes(self) -> int:
        """One launch covering q, k and v: the three per-call figures with x read once."""
        return 3 * self.shrink_bytes() - 2 * self.batch * self.hidden * 2

    def qkv_expand_bytes(self) -> int:
        return sum(self.expand_bytes(h) for h in self.h_out[:3])

    def layer_bytes(self, fused: bool = False) -> int:
        if fused:
            return (self.qkv_shrink_bytes() + self.shrink_bytes() + self.qkv_expand_bytes() +
                    self.expand_bytes(self.h_out[3]))
        return sum(self.shrink_bytes() + self.expand_bytes(h) for h in self.h_out)

    def step_bytes(self, fused: bool = False) -> int:
        return self.n_layers * self.layer_bytes(fused)

    def gathered_layer_bytes(self) -> int:
        """Same formulas with every token fetching its own copy of the weights."""
        s = 2
        r_t = self.ranks[self.bins_np]
        tot = 0
        for h in self.h_out:
            tot += r_t.sum() * self.hidden * s + self.batch * self.hidden * s + r_t.sum() * s
            tot += r_t.sum() * h * s + r_t.sum() * s + 2 * self.batch * h * s
        return int(tot)


def zipf_ids(rng, n_adapters: int, batch: int, alpha: float) -> np.ndarray:
    p = 1.0 / np.arange(1, n_adapters + 1, dtype=np.float64) ** alpha
    return rng.choice(n_adapters, size=batch, p=p / p.sum()).astype(np.int64)


def build_decode_workload(name, device, *, hidden, n_layers, n_adapters, rank_choices, batch, n_pages,
                          dtype=torch.float16, h_out=None, ids="zipf", zipf_alpha=1.0, occupancy=0.6, heads=32,
                          lora_alpha=16.0, seed=2, fill_noise=True, placement="scattered") -> DecodeWorkload:
    """Allocate and fill the pools on ``device``.

    ``placement``: "scattered" -- every adapter page at a random place of the pool (what an
    allocator that hands out the first free pages of a fragmented map ends up with);
    "runs" -- each adapter's ``4 r`` pages one contiguous run at a random place (what
    ``MemoryAllocator.alloc_adapter`` asks for).

    Weights: A ~ N(0, 1/hidden), B ~ N(0, 1/r), scaling = lora_alpha / r; pages
    not owned by an adapter up to ``occupancy`` of the pool hold N(0,1) noise
    standing for KV-cache entries, the rest is left as allocated."""
    rng = np.random.default_rng(seed)
    ranks = rng.choice(np.asarray(rank_choices), size=n_adapters).astype(np.int64)
    if ids == "zipf":
        bins = zipf_ids(rng, n_adapters, batch, zipf_alpha)
    else:
        bins = rng.integers(0, n_adapters, size=batch).astype(np.int64)
    a_len = 4 * ranks
    a_start = np.zeros(n_adapters, dtype=np.int64)
    a_start[1:] = np.cumsum(a_len)[:-1]
    n_loc = int(a_len.sum())
    if n_loc > n_pages:
        raise ValueError(f"pool of {n_pages} pages cannot hold {n_loc} adapter pages")
    perm = rng.permutation(n_pages).astype(np.int64)
    n_kv = max(0, int(occupancy * n_pages) - n_loc)
    if placement == "scattered":
        a_loc = perm[:n_loc]
        kv_pages = perm[n_loc:n_loc + n_kv]
    elif placement == "runs":
        # the pool cut into slots of the largest adapter's size; adapters take random slots
        slot = int(a_len.max())
        slots = rng.permutation(n_pages // slot)[:n_adapters].astype(np.int64)
        if slots.size < n_adapters:
            raise ValueError(f"pool of {n_pages} pages has no room for {n_adapters} runs of {slot} pages")
        a_loc = np.concatenate([s0 * slot + np.arange(n, dtype=np.int64) for s0, n in zip(slots, a_len)])
        used = np.zeros(n_pages, dtype=bool)
        used[a_loc] = True
        kv_pages = perm[~used[perm]][:n_kv]
    else:
        raise ValueError(f"unknown placement {placement!r}")
    scales = (lora_alpha / ranks).astype(np.float32)
    h_out = list(h_out) if h_out is not None else [hidden] * 4
    w = DecodeWorkload(name=name, hidden=hidden, h_out=h_out, n_layers=n_layers, ranks=ranks, bins_np=bins,
                       a_start_np=a_start, a_len_np=a_len, a_loc_np=a_loc, scales_np=scales, page_elems=hidden,
                       n_pages=n_pages, dtype=dtype, max_rank=int(ranks.max()))
    w.a_start = torch.from_numpy(a_start).to(device)
    w.a_len = torch.from_numpy(a_len).to(device)
    w.a_loc = torch.from_numpy(a_loc).to(device)
    w.a_scaling = torch.from_numpy(scales).to(device=device, dtype=torch.float16)
    w.req_bins = torch.from_numpy(bins).to(device)
    # per-page standard deviation of the B side: page i of adapter a holds B^T entries ~ N(0, 1/r_a)
    page_rank = np.repeat(ranks, 4 * ranks)
    std_b = torch.from_numpy((1.0 / np.sqrt(page_rank)).astype(np.float32)).to(device).view(-1, 1, 1)
    kv_idx = torch.from_numpy(kv_pages).to(device)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    head_dim = hidden // heads
    for _ in range(n_layers):
        kb = torch.empty((n_pages, heads, head_dim), dtype=dtype, device=device)
        vb = torch.empty((n_pages, heads, head_dim), dtype=dtype, device=device)
        if fill_noise:
            # cheap deterministic fill for pages nobody reads; KV pages get N(0,1)
            kb.zero_()
            vb.zero_()
            if n_kv:
                kb[kv_idx] = torch.randn((n_kv, heads, head_dim), generator=gen, device=device, dtype=torch.float32).to(dtype)
                vb[kv_idx] = torch.randn((n_kv, heads, head_dim), generator=gen, device=device, dtype=torch.float32).to(dtype)
        a_vals = torch.randn((n_loc, heads, head_dim), generator=gen, device=device, dtype=torch.float32)
        kb[w.a_loc] = (a_vals / float(np.sqrt(hidden))).to(dtype)
        b_vals = torch.randn((n_loc, heads, head_dim), generator=gen, device=device, dtype=torch.float32)
        vb[w.a_loc] = (b_vals * std_b).to(dtype)
        w.key_buffer.append(kb)
        w.value_buffer.append(vb)
    return w


# The benchmark configurations (hidden sizes and rank mixes of the S2 / S4 / S6
# dummy setups).
def s2_decode(device, n_layers=32, batch=256, n_pages=65536, dtype=torch.float16, seed=2, placement="scattered"):
    return build_decode_workload("S2 decode BGMV: hidden 4096, ranks {64,32,16,8}, 200 adapters, Zipf(1), batch 256",
                                 device, hidden=4096, n_layers=n_layers, n_adapters=200, rank_choices=[64, 32, 16, 8],
                                 batch=batch, n_pages=n_pages, dtype=dtype, ids="zipf", zipf_alpha=1.0, seed=seed,
                                 placement=placement)


def s4_decode(device, n_layers=40, batch=512, n_pages=262144, dtype=torch.float16, seed=4, placement="scattered"):
    return build_decode_workload("S4 decode: hidden 5120, ranks {64,32,16}, 1000 adapters, Zipf(0.9), batch 512",
                                 device, hidden=5120, n_layers=n_layers, n_adapters=1000, rank_choices=[64, 32, 16],
                                 batch=batch, n_pages=n_pages, dtype=dtype, ids="zipf", zipf_alpha=0.9, heads=40,
                                 seed=seed, placement=placement)


def s6_decode(device, n_layers=8, batch=1024, n_adapters=2000, n_pages=None, dtype=torch.bfloat16, seed=6,
              placement="scattered"):
    n_pages = n_pages or (n_adapters * 256 + 4096)
    return build_decode_workload("S6 decode: hidden 8192, rank 64, 2000 adapters, uniform ids, batch 1024, GQA k/v 1024",
                                 device, hidden=8192, n_layers=n_layers, n_adapters=n_adapters, rank_choices=[64],
                                 batch=batch, n_pages=n_pages, dtype=dtype, h_out=[8192, 1024, 1024, 8192],
                                 ids="uniform", heads=64, seed=seed, occupancy=0.0, fill_noise=False,
                                 placement=placement)


# ---- prefill ------------------------------------------------------------------
@dataclass
class PrefillSegments:
    """Requests of a prefill batch laid end to end: request i owns token rows
    ``b_start_loc[i] + [0, b_seq_len[i])`` and uses adapter ``b_indicies[i]``."""
    lens_np: np.ndarray
    ids_np: np.ndarray
    b_start_loc: torch.Tensor = None  # int32
    b_seq_len: torch.Tensor = None    # int32
    b_indicies: torch.Tensor = None   # int64

    @property
    def n_tokens(self) -> int:
        return int(self.lens_np.sum())

    @property
    def max_len(self) -> int:
        return int(self.lens_np.max())

    # algorithmic bytes and flops of one call over pool workload ``w``
    def shrink_bytes(self, w) -> int:
        u = np.unique(self.ids_np)
        return int(self.n_tokens * w.hidden * 2 + self.n_tokens * w.max_rank * 2 + w.ranks[u].sum() * w.hidden * 2)

    def expand_bytes(self, w, h_out) -> int:
        u = np.unique(self.ids_np)
        return int(2 * self.n_tokens * h_out * 2 + self.n_tokens * w.max_rank * 2 + w.ranks[u].sum() * h_out * 2)

    def flops(self, w, h) -> int:
        return int(2 * h * (w.ranks[self.ids_np] * self.lens_np).sum())


def segments(device, lens, ids) -> PrefillSegments:
    """Requests of the given lengths and adapters laid end to end."""
    lens = np.asarray(lens, dtype=np.int32)
    ids = np.asarray(ids, dtype=np.int64)
    start = np.zeros(lens.size, np.int32)
    start[1:] = np.cumsum(lens)[:-1]
    seg = PrefillSegments(lens_np=lens, ids_np=ids)
    seg.b_start_loc = torch.from_numpy(start).to(device)
    seg.b_seq_len = torch.from_numpy(lens).to(device)
    seg.b_indicies = torch.from_numpy(ids).to(device)
    return seg


def c4_prefill_segments(w, device, seed=4) -> PrefillSegments:
    """The prefill half of the mixed S4 step: 4 requests of 256 tokens whose adapters are drawn
    like the decode tokens' (Zipf(0.9) over the workload's adapters)."""
    rng = np.random.default_rng(seed + 100)
    return segments(device, [256] * 4, np.sort(zipf_ids(rng, len(w.ranks), 4, 0.9)))


def c3_prefill(device, n_layers=4, n_pages=65536, seed=3):
    """64 requests of 8..512 tokens sorted by adapter, 100 adapters of ranks
    {64,32,16,8}, bfloat16, hidden 4096, pages scattered over the pool."""
    w = build_decode_workload("C3 prefill: hidden 4096, 64 requests of 8..512 tokens, 100 adapters ranks {64,32,16,8}, bf16",
                              device, hidden=4096, n_layers=n_layers, n_adapters=100, rank_choices=[64, 32, 16, 8],
                              batch=1, n_pages=n_pages, dtype=torch.bfloat16, seed=seed)
    rng = np.random.default_rng(seed)
    n_req = 64
    lens = rng.integers(8, 513, size=n_req).astype(np.int32)
    ids = np.sort(rng.integers(0, 100, size=n_req)).astype(np.int64)
    start = np.zeros(n_req, np.int32)
    start[1:] = np.cumsum(lens)[:-1]
    seg = PrefillSegments(lens_np=lens, ids_np=ids)
    seg.b_start_loc = torch.from_numpy(start).to(device)
    seg.b_seq_len = torch.from_numpy(lens).to(device)
    seg.b_indicies = torch.from_numpy(ids).to(device)
    return w, seg
