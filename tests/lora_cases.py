"""Seeded synthetic multi-LoRA cases shared by the CPU and GPU tests.

A case is built with the oracle's own packer/table builder so that the dense
matrices (A, B per adapter and projection) and the paged pool describe the same
adapters.  Arrays are float32 holding values representable in ``dtype``.
"""
from __future__ import annotations

import numpy as np

from oracle import lora_oracle as O


class Case:
    pass


def make_case(seed, hidden, ranks, batch, dtype="f16", n_pages=None, page_elems=None, h_out=None,
              bins=None, zipf_alpha=None, lora_alpha=16.0, scatter=True, x_scale=1.0, max_rank=None):
    rng = np.random.default_rng(seed)
    c = Case()
    c.dtype = dtype
    c.hidden = hidden
    c.page_elems = page_elems or hidden
    c.h_out = list(h_out) if h_out is not None else [hidden] * 4
    c.ranks = [int(r) for r in ranks]
    n_ad = len(c.ranks)
    need = sum(4 * r for r in c.ranks)
    c.n_pages = n_pages or (need * 2 + 7)
    assert c.n_pages >= need
    # pool noise everywhere (stands for KV pages), then adapters on scattered pages
    c.key = O.round_to(rng.standard_normal((c.n_pages, c.page_elems)).astype(np.float32), dtype)
    c.value = O.round_to(rng.standard_normal((c.n_pages, c.page_elems)).astype(np.float32), dtype)
    perm = rng.permutation(c.n_pages) if scatter else np.arange(c.n_pages)
    c.a_start, c.a_len, c.a_loc = O.build_tables(c.ranks, perm[:need])
    c.A, c.B = [], []
    for i, r in enumerate(c.ranks):
        A = [O.round_to(rng.standard_normal((hidden, r)).astype(np.float32) / np.sqrt(hidden), dtype) for _ in range(4)]
        B = [O.round_to(rng.standard_normal((r, c.h_out[p])).astype(np.float32) / np.sqrt(max(r, 1)), dtype)
             for p in range(4)]
        c.A.append(A)
        c.B.append(B)
        if r > 0:
            wc = O.pack_w_combined(A, B, c.page_elems)
            loc = c.a_loc[c.a_start[i]: c.a_start[i] + 4 * r]
            O.load_into_pool(c.key, c.value, wc, loc)
    sc = np.array([lora_alpha / r if r else 0.0 for r in c.ranks], dtype=np.float32)
    c.scales = O.round_to(sc, "f16")  # a_scaling is an fp16 table in the reference (infer_adapter.py:33)
    if bins is None:
        if zipf_alpha is not None:
            pz = 1.0 / np.arange(1, n_ad + 1) ** zipf_alpha
            bins = rng.choice(n_ad, size=batch, p=pz / pz.sum())
        else:
            bins = rng.integers(0, n_ad, size=batch)
    c.bins = np.asarray(bins, dtype=np.int64)
    c.batch = len(c.bins)
    c.x = O.round_to(rng.standard_normal((c.batch, hidden)).astype(np.float32) * x_scale, dtype)
    c.max_rank = max_rank or max(c.ranks + [8])
    return c


def make_segments(seed, n_req, lo, hi, n_adapters, sort_by_adapter=True):
    """Prefill batch: request lengths U[lo, hi], adapter per request, packed rows."""
    rng = np.random.default_rng(seed)
    lens = rng.integers(lo, hi + 1, size=n_req).astype(np.int32)
    ids = rng.integers(0, n_adapters, size=n_req).astype(np.int64)
    if sort_by_adapter:
        ids = np.sort(ids)
    start = np.zeros(n_req, dtype=np.int32)
    start[1:] = np.cumsum(lens)[:-1]
    return start, lens, ids
