"""The decode plan itself (slora_bgmv_plan_build), word for word, against a restatement of its
layout in numpy, for every builder kernel: batches of up to 1024 tokens, of up to 8192 (tokens
sorted by adapter in LDS) and beyond (one workgroup, scratch behind the records).  The kernels
that read a plan are tested elsewhere (planned calls equal stateless calls bit for bit)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

HEADER, WORDS, RB, TT, XCDS = 16, 48, 8, 4, 8
MAGIC_WORD, N_ITEMS, MAX_RANK, BATCH, TT_WORD, RANK_CAP, N_RUNS = range(7)


def expected_plan(bins, a_start, a_len, a_loc, n_pages, rank_cap):
    """Runs = up to four tokens of one adapter, in token order; runs ordered by (adapter, first
    token); a run of rank r has ceil(min(r, rank_cap) / 8) items; the items, in that order, are cut
    into 8 queues of equal length (a run stays in the queue its first item falls into), queue q's
    k-th item is record k * 8 + q, the queues are padded to the longest with empty records."""
    n_adapters, n_loc = len(a_start), len(a_loc)
    runs = []
    by_adapter = {}
    for b, a in enumerate(bins):
        if 0 <= a < n_adapters and a_len[a] // 4 > 0:
            by_adapter.setdefault(int(a), []).append(b)
    for a in sorted(by_adapter):
        toks = by_adapter[a]
        for c in range(0, len(toks), TT):
            runs.append((a, toks[c:c + TT]))
    n_it = [(min(int(a_len[a]) // 4, rank_cap) + RB - 1) // RB for a, _ in runs]
    before = np.concatenate([[0], np.cumsum(n_it)]).astype(np.int64)
    total = int(before[-1])
    queue = [min(XCDS - 1, int(before[i]) * XCDS // max(total, 1)) for i in range(len(runs))]
    qstart = [min([int(before[i]) for i in range(len(runs)) if queue[i] == q], default=0) for q in range(XCDS)]
    qlen = [sum(n_it[i] for i in range(len(runs)) if queue[i] == q) for q in range(XCDS)]
    n_items = XCDS * max(qlen) if runs else 0
    rec = np.zeros((n_items, WORDS), np.int32)
    rec[:, 8:40] = -1
    for i, (a, toks) in enumerate(runs):
        r = int(a_len[a]) // 4
        q = queue[i]
        for it in range(n_it[i]):
            row = rec[(int(before[i]) - qstart[q] + it) * XCDS + q]
            row[0:4] = (a, r, len(toks), it * RB)
            row[4:4 + len(toks)] = toks
            for p in range(4):
                for jr in range(RB):
                    j = it * RB + jr
                    li = int(a_start[a]) + p * r + j
                    if j < r and 0 <= li < n_loc and 0 <= a_loc[li] < n_pages:
                        row[8 + p * RB + jr] = a_loc[li]
            row[40:42] = np.array([int(a_start[a])], np.int64).view(np.int32)      # low word, high word
            row[42] = 1 if (it == n_it[i] - 1 and r > rank_cap) else 0
    max_rank = max([int(a_len[a]) // 4 for a, _ in runs], default=0)
    return n_items, len(runs), max_rank, rec


@pytest.mark.parametrize("batch,n_adapters,rank_cap,seed", [
    (1, 3, 64, 0), (5, 2, 64, 1), (300, 40, 64, 2), (1024, 200, 64, 3),        # one token per thread
    (64, 5, 16, 4),                                                            # ranks above the cap: `more`
    (1025, 200, 64, 5), (3000, 1500, 32, 6), (8192, 64, 64, 7), (5000, 5000, 8, 8),   # sorted in LDS
    (9000, 300, 64, 9),                                                        # one workgroup
    (2000, 600000, 64, 10),                                                    # adapter ids too large for the sorted keys
])
def test_plan_records_word_for_word(gpu, batch, n_adapters, rank_cap, seed):
    import slora_hip
    rng = np.random.default_rng(seed)
    ranks = rng.choice([8, 16, 32, 64, 24, 0], size=n_adapters, p=[.25, .2, .2, .2, .1, .05])
    if seed == 4:
        ranks = np.array([64, 8, 32, 128, 16])
    if n_adapters > 100000:       # a few adapters with weights among many without
        live = rng.choice(n_adapters, size=80, replace=False)
        keep = ranks[live]
        ranks = np.zeros(n_adapters, dtype=ranks.dtype)
        ranks[live] = keep
    a_len = (4 * ranks).astype(np.int64)
    a_start = np.concatenate([[0], np.cumsum(a_len)[:-1]]).astype(np.int64)
    n_loc = int(a_len.sum())
    n_pages = n_loc + 50
    a_loc = rng.permutation(n_pages)[:n_loc].astype(np.int64)
    a_loc[rng.integers(0, max(n_loc, 1), size=3)] = n_pages + 7          # page ids outside the pool
    if n_adapters > 100000:
        pool_ids = np.concatenate([np.nonzero(ranks)[0], rng.integers(0, n_adapters, size=20)])
        bins = rng.choice(pool_ids, size=batch).astype(np.int64)
    else:
        p = 1.0 / np.arange(1, n_adapters + 1)
        bins = rng.choice(n_adapters, size=batch, p=p / p.sum()).astype(np.int64)
    bins[rng.integers(0, batch, size=max(1, batch // 50))] = -1           # tokens without an adapter
    bins[rng.integers(0, batch, size=max(1, batch // 70))] = n_adapters + 3
    t = [torch.from_numpy(v).to(gpu) for v in (a_start, a_len, a_loc, bins)]
    plan = slora_hip.make_plan(*t, rank_cap, n_pages)
    buf = plan.buf.cpu().numpy().view(np.int32)
    n_items, n_runs, max_rank, rec = expected_plan(bins, a_start, a_len, a_loc, n_pages, rank_cap)
    assert (plan.n_items, plan.n_runs, plan.max_rank) == (n_items, n_runs, max_rank)
    head = buf[:HEADER]
    assert (head[N_ITEMS], head[MAX_RANK], head[BATCH], head[TT_WORD], head[RANK_CAP], head[N_RUNS]) == \
        (n_items, max_rank, batch, TT, rank_cap, n_runs)
    got = buf[HEADER:HEADER + n_items * WORDS].reshape(n_items, WORDS)
    bad = np.nonzero((got != rec).any(axis=1))[0]
    assert bad.size == 0, (bad[:5], got[bad[:2]], rec[bad[:2]])
    # and a plan rebuilt in place for another batch of the same size holds that batch's records
    bins2 = rng.permutation(bins)
    slora_hip.rebuild_plan(plan, t[0], t[1], t[2], torch.from_numpy(bins2).to(gpu), n_pages)
    n_items2, n_runs2, _, rec2 = expected_plan(bins2, a_start, a_len, a_loc, n_pages, rank_cap)
    buf2 = plan.buf.cpu().numpy().view(np.int32)
    assert buf2[N_ITEMS] == n_items2 and buf2[N_RUNS] == n_runs2
    assert np.array_equal(buf2[HEADER:HEADER + n_items2 * WORDS].reshape(n_items2, WORDS), rec2)
