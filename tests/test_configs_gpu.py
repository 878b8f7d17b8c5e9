"""The benchmark configurations at their real shapes, the dense ("S-LoRA-bmm")
semantics on the GPU, and outputs that live inside the pool.

* C5 (S6 shape): hidden 8192 = page, q/o out 8192, k/v out 1024 (grouped-query), rank 64,
  bf16, batch 1024 over 2000 adapters with uniform ids -- an oracle-sized cut against
  ``ref_bgmv_*`` and the full size through properties.
* C4 (S4 shape): hidden 5120, 1000 adapters of ranks {64,32,16}, Zipf(0.9): 512 decode
  tokens and 4 prefill requests of 256 tokens over one 262144-page pool.
* The north star states its tolerance (rtol 1e-2 / atol 1e-3) against the reference's bmm
  path (slora/models/bmm/lora_bmm_infer.py:285-299): both operator families against
  ``ref_bmm`` directly.
* ``y`` as a row slice of the very buffer passed as ``w`` (the reference's decode k/v
  outputs are views of the pool,
  slora/common/basemodel/layer_infer/template/transformer_layer_infer_template.py:39-41).

Everything goes through the C ABI of libslora_hip.so.
"""
import numpy as np
import pytest
import torch

from oracle import lora_oracle as O
from lora_cases import make_case
from test_bgmv_gpu import GpuCase, dev, host, oracle_chain, run_chain

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-3


@pytest.fixture(params=["cache", "stateless"])
def plan_cache_mode(request):
    """Calls that pass no plan are served by the automatic plan cache (the default) or,
    with the cache off, by the kernels that find their runs by themselves."""
    import slora_hip
    slora_hip.set_plan_cache_enabled(request.param == "cache")
    slora_hip.clear_plan_cache()
    yield request.param
    slora_hip.clear_plan_cache()
    slora_hip.set_plan_cache_enabled(True)


# ---------------------------------------------------------------------------
# C5
# ---------------------------------------------------------------------------
def test_c5_cut_matches_oracle(gpu, plan_cache_mode):
    """hidden 8192, page 8192, k/v out 1024, rank 64, bf16: 3 adapters and 16 tokens, all
    four projections against the paged oracle, single calls and the q/k/v launches."""
    from slora_hip import dispatch_bgmv_qkv_expand, dispatch_bgmv_qkv_shrink
    h_out = [8192, 1024, 1024, 8192]
    c = make_case(55, 8192, [64, 64, 64], 16, dtype="bf16", h_out=h_out,
                  bins=np.array([0, 1, 2, 0, 0, 1, 2, 2, 0, 0, 0, 1, 0, 2, 1, 0]))
    g = GpuCase(c, gpu, heads=64)
    R = 64
    deltas = []
    for p in range(4):
        y0 = O.round_to(np.random.default_rng(p).standard_normal((c.batch, h_out[p])).astype(np.float32), "bf16")
        d_gpu, y_gpu = run_chain(c, g, p, R, gpu, y0)
        d_ref, _ = oracle_chain(c, p, R)
        np.testing.assert_allclose(d_gpu, d_ref, rtol=RTOL, atol=ATOL)
        y_ref = O.ref_bgmv_expand(y0, d_gpu, c.value, c.a_start, c.a_len, c.a_loc, c.bins, p, c.scales, dtype="bf16")
        # y0 ~ N(0,1) plus an update of order 1: the bf16 sum may cancel, one ulp of the larger term is 2^-8
        np.testing.assert_allclose(y_gpu, y_ref, rtol=RTOL, atol=8e-3)
        yz_gpu = run_chain(c, g, p, R, gpu)[1]
        yz_ref = O.ref_bgmv_expand(np.zeros_like(y0), d_gpu, c.value, c.a_start, c.a_len, c.a_loc, c.bins, p,
                                   c.scales, dtype="bf16")
        np.testing.assert_allclose(yz_gpu, yz_ref, rtol=RTOL, atol=ATOL)
        deltas.append(d_gpu)
    t = (g.a_start, g.a_len, g.a_loc, g.bins)
    d_f = [torch.zeros((c.batch, R), dtype=g.tdt, device=gpu) for _ in range(3)]
    dispatch_bgmv_qkv_shrink(d_f[0], d_f[1], d_f[2], g.x, g.key, *t)
    y_f = [torch.zeros((c.batch, h_out[p]), dtype=g.tdt, device=gpu) for p in range(3)]
    dispatch_bgmv_qkv_expand(y_f[0], y_f[1], y_f[2], d_f[0], d_f[1], d_f[2], g.value, *t, g.scales)
    for p in range(3):
        assert np.array_equal(host(d_f[p]), deltas[p]), p
        assert np.array_equal(host(y_f[p]), run_chain(c, g, p, R, gpu)[1]), p


def check_decode_properties(w, gpu, projections=(0, 1, 2, 3), y_atol=ATOL):
    """One layer of a device-built decode workload, checked without the CPU oracle:
    dense torch float32 on the device from the adapters' pool pages (A^T rows, the flat
    B^T), doubling the scales doubles y, a token permutation permutes the results bit for
    bit, columns of delta beyond the rank do not matter, and the q/k/v launches equal the
    single calls."""
    from slora_hip import dispatch_bgmv, dispatch_bgmv_qkv_expand, dispatch_bgmv_qkv_shrink
    B, H, R = w.batch, w.hidden, w.max_rank
    t = (w.a_start, w.a_len, w.a_loc, w.req_bins)
    g = torch.Generator(device=gpu)
    g.manual_seed(5)
    x = torch.randn((B, H), generator=g, device=gpu).to(w.dtype)
    key, val = w.key_buffer[0], w.value_buffer[0]
    perm = torch.randperm(B, generator=g, device=gpu)
    t_perm = (w.a_start, w.a_len, w.a_loc, w.req_bins[perm].contiguous())
    ranks_t = torch.from_numpy(w.ranks[w.bins_np]).to(gpu)
    groups = {int(a): torch.from_numpy(np.nonzero(w.bins_np == a)[0]).to(gpu) for a in np.unique(w.bins_np)}
    ds, ys = {}, {}
    for p in projections:
        Ho = w.h_out[p]
        d = torch.zeros((B, R), dtype=w.dtype, device=gpu)
        dispatch_bgmv(d, x, key, *t, p, w.a_scaling)
        y = torch.zeros((B, Ho), dtype=w.dtype, device=gpu)
        dispatch_bgmv(y, d, val, *t, p, w.a_scaling)
        d_ref = torch.zeros((B, R), dtype=torch.float32, device=gpu)
        y_ref = torch.zeros((B, Ho), dtype=torch.float32, device=gpu)
        for a, rows in groups.items():
            r = int(w.ranks[a])
            loc = w.a_loc[int(w.a_start_np[a]) + p * r: int(w.a_start_np[a]) + (p + 1) * r]
            A_t = key[loc].reshape(r, H).float()
            Bt = val[loc].reshape(-1)[: Ho * r].reshape(Ho, r).float()
            d_ref[rows, :r] = x[rows].float() @ A_t.t()
            y_ref[rows] = (d[rows, :r].float() @ Bt.t()) * float(w.a_scaling[a])
        np.testing.assert_allclose(d.float().cpu().numpy(), d_ref.cpu().numpy(), rtol=RTOL, atol=ATOL)
        np.testing.assert_allclose(y.float().cpu().numpy(), y_ref.cpu().numpy(), rtol=RTOL, atol=y_atol)
        y2 = torch.zeros_like(y)
        dispatch_bgmv(y2, d, val, *t, p, (w.a_scaling * 2).contiguous())
        tiny = 2.0 ** -13 if w.dtype == torch.float16 else 2.0 ** -125
        normal = y.abs() >= tiny
        assert torch.equal(y2[normal], (y * 2)[normal])
        dp = torch.zeros_like(d)
        dispatch_bgmv(dp, x[perm].contiguous(), key, *t_perm, p, w.a_scaling)
        assert torch.equal(dp, d[perm])
        yp = torch.zeros_like(y)
        dispatch_bgmv(yp, dp, val, *t_perm, p, w.a_scaling)
        assert torch.equal(yp, y[perm])
        dg = d.clone()
        dg[torch.arange(R, device=gpu)[None, :] >= ranks_t[:, None]] = 77.0
        yg = torch.zeros_like(y)
        dispatch_bgmv(yg, dg, val, *t, p, w.a_scaling)
        assert torch.equal(yg, y)
        ds[p], ys[p] = d, y
    if all(p in ds for p in (0, 1, 2)):
        d_f = [torch.zeros((B, R), dtype=w.dtype, device=gpu) for _ in range(3)]
        dispatch_bgmv_qkv_shrink(d_f[0], d_f[1], d_f[2], x, key, *t)
        y_f = [torch.zeros((B, w.h_out[p]), dtype=w.dtype, device=gpu) for p in range(3)]
        dispatch_bgmv_qkv_expand(y_f[0], y_f[1], y_f[2], d_f[0], d_f[1], d_f[2], val, *t, w.a_scaling)
        for p in range(3):
            assert torch.equal(d_f[p], ds[p]) and torch.equal(y_f[p], ys[p]), p


def test_full_size_c5_properties(gpu, plan_cache_mode):
    """The S6-shape decode itself: hidden 8192, rank 64, 2000 adapters on 516096 pages of
    8192 elements, batch 1024 with uniform adapter ids (about 800 distinct), k/v out 1024,
    bf16, one layer.  y of the dense check is a bf16 sum of 64 terms of order 1/8 scaled by
    0.25: atol 1e-3 holds."""
    import workloads
    w = workloads.s6_decode(gpu, n_layers=1)
    assert (w.hidden, w.h_out, w.batch, w.dtype) == (8192, [8192, 1024, 1024, 8192], 1024, torch.bfloat16)
    check_decode_properties(w, gpu)


# ---------------------------------------------------------------------------
# C4
# ---------------------------------------------------------------------------
def test_full_size_c4_mixed_step(gpu, plan_cache_mode):
    """The S4-shape mixed step on one layer of its 262144-page pool (hidden 5120, 1000
    adapters of ranks {64,32,16}, Zipf(0.9)): 512 decode tokens through dispatch_bgmv and 4
    prefill requests of 256 tokens through the segmented operators (the reference takes
    them at max_b_seq_len >= 200, max_lora_dim >= 64, 2 or more requests,
    slora/models/peft/lora_unordered_batch_infer.py:334), against dense torch float32 on
    the device, and the prefill requests also through dispatch_bgmv with per-token bins
    (the reference's other branch, :349-355)."""
    import workloads
    from slora_hip import dispatch_bgmv, lora_get_qkvo_fwd_expand, lora_get_qkvo_fwd_shrink
    w = workloads.s4_decode(gpu, n_layers=1)
    assert (w.hidden, w.batch, w.n_pages, w.ranks.size) == (5120, 512, 262144, 1000)
    check_decode_properties(w, gpu)

    H, R = w.hidden, w.max_rank
    rng = np.random.default_rng(44)
    ids = np.sort(workloads.zipf_ids(rng, 1000, 4, 0.9))
    lens = np.full(4, 256, np.int32)
    starts = np.arange(4, dtype=np.int32) * 256
    T = 1024
    st, ln, rq = dev(starts, torch.int32, gpu), dev(lens, torch.int32, gpu), dev(ids, torch.int64, gpu)
    g = torch.Generator(device=gpu)
    g.manual_seed(9)
    x = torch.randn((T, H), generator=g, device=gpu).to(w.dtype)
    key, val = w.key_buffer[0], w.value_buffer[0]
    t = (w.a_loc, w.a_start, w.a_len, st, ln, rq)
    tok_bins = torch.repeat_interleave(rq, ln.long())
    for p in range(4):
        d = torch.full((T, R), 9.0, dtype=w.dtype, device=gpu)
        lora_get_qkvo_fwd_shrink(x, key.view(-1, H), d, *t, H, p, R, 256)
        y0 = torch.randn((T, H), generator=g, device=gpu).to(w.dtype)
        y = y0.clone()
        lora_get_qkvo_fwd_expand(d, val.view(-1, H), y, w.a_scaling, *t, H, p, R, 256)
        d_ref = torch.zeros((T, R), dtype=torch.float32, device=gpu)
        y_ref = y0.float().clone()
        for i, a in enumerate(ids):
            r = int(w.ranks[a])
            loc = w.a_loc[int(w.a_start_np[a]) + p * r: int(w.a_start_np[a]) + (p + 1) * r]
            rows = slice(i * 256, (i + 1) * 256)
            d_ref[rows, :r] = x[rows].float() @ key[loc].reshape(r, H).float().t()
            y_ref[rows] += (d[rows, :r].float() @ val[loc].reshape(H, r).float().t()) * float(w.a_scaling[a])
        np.testing.assert_allclose(host(d), d_ref.cpu().numpy(), rtol=RTOL, atol=ATOL)
        # y0 ~ N(0,1) plus an update of order 1 in fp16: one ulp of a sum near 4 is 4e-3
        np.testing.assert_allclose(host(y), y_ref.cpu().numpy(), rtol=RTOL, atol=4e-3)
        # the same tokens through the decode operator with per-token adapter ids
        d2 = torch.zeros((T, R), dtype=w.dtype, device=gpu)
        dispatch_bgmv(d2, x, key, w.a_start, w.a_len, w.a_loc, tok_bins, p, w.a_scaling)
        np.testing.assert_allclose(host(d2), d_ref.cpu().numpy(), rtol=RTOL, atol=ATOL)
        y2 = y0.clone()
        dispatch_bgmv(y2, d2, val, w.a_start, w.a_len, w.a_loc, tok_bins, p, w.a_scaling)
        np.testing.assert_allclose(host(y2), y_ref.cpu().numpy(), rtol=RTOL, atol=8e-3)


# ---------------------------------------------------------------------------
# the bmm semantics, directly
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("hidden,ranks,batch,lora_alpha", [
    (4096, [8] * 8, 32, 16.0),                    # C1: 8 adapters of rank 8, 32 tokens, scaling 2.0
    (1024, [64, 32, 16, 8, 8, 16], 48, 12.0),     # mixed ranks, scalings that are not powers of two
])
def test_decode_and_prefill_match_ref_bmm(gpu, plan_cache_mode, dtype, hidden, ranks, batch, lora_alpha):
    """Both operator families against the gather + zero-padded bmm + scatter-add of the
    reference's bmm engine (``ref_bmm``, slora/models/bmm/lora_bmm_infer.py:285-299).

    Stage by stage at exactly rtol 1e-2 / atol 1e-3: the shrink output against the
    engine's rounded ``x @ A``, and the expand against the engine fed with the GPU's own
    shrink output (``ref_bmm`` with x = delta and A = the identity, whose ``x @ A`` is delta
    exactly), from a zero y.

    The whole chain shrink -> expand against ``ref_bmm(x, A, B)``: rtol 1e-2 / atol 1e-3 for
    every output but a counted few -- at most 1 in 10 000 may lie outside, and then by no more
    than what ONE storage-type rounding flip of ONE delta entry moves that output by,
    ``ulp(max|delta_t|) * scale * max_d |B[d, n]|``.  The intermediate delta is rounded to
    fp16/bf16 by the engine and by the kernels alike, from float sums taken in different
    orders; where a sum lies within a float ulp of a rounding boundary the two round apart,
    whatever the kernel does.  (Measured: 5 of 131072 outputs of the C1 case differ by up to
    2e-3 where y is near zero.)  From a random y every output is also allowed one rounding
    step of the storage type at the magnitude of the larger operand of ``y0 + update``: the
    reference's ``+=`` rounds the update (product, then times scaling) and the sum at that
    magnitude, the kernels round scale * sum once, and where y0 and the update cancel that
    step is larger than any tolerance relative to the small result."""
    from slora_hip import dispatch_bgmv, lora_get_qkvo_fwd_expand, lora_get_qkvo_fwd_shrink
    n_ad = len(ranks)
    rng = np.random.default_rng(3)
    if lora_alpha == 16.0:
        bins = rng.integers(0, n_ad, size=batch)              # C1: every token's adapter uniform in [0, 8)
    else:
        bins = np.repeat(rng.integers(0, n_ad, size=8), 6)    # requests of 6 tokens
    c = make_case(10 + hidden, hidden, ranks, batch, dtype=dtype, bins=bins, lora_alpha=lora_alpha)
    # the prefill operators see the same batch as requests: maximal runs of tokens with one adapter
    cut = np.flatnonzero(np.diff(c.bins)) + 1
    start = np.concatenate([[0], cut]).astype(np.int32)
    lens = np.diff(np.concatenate([start, [batch]])).astype(np.int32)
    ids = c.bins[start]
    g = GpuCase(c, gpu)
    R = max(ranks)
    st, ln, rq = dev(start, torch.int32, gpu), dev(lens, torch.int32, gpu), dev(ids, torch.int64, gpu)
    t = (g.a_start, g.a_len, g.a_loc, g.bins)
    tp = (g.a_loc, g.a_start, g.a_len, st, ln, rq)
    mant = 10 if dtype == "f16" else 7
    eye = [np.eye(R, r, dtype=np.float32) for r in ranks]
    for p in range(4):
        A_p, B_p = [a[p] for a in c.A], [b[p] for b in c.B]
        zero = np.zeros((batch, hidden), np.float32)
        y0 = O.round_to(np.random.default_rng(p).standard_normal((batch, hidden)).astype(np.float32), dtype)
        xa = np.zeros((batch, R), np.float32)
        for tkn in range(batch):
            a = c.bins[tkn]
            xa[tkn, : ranks[a]] = O.round_to(c.x[tkn] @ A_p[a], dtype)
        # per output: what one rounding flip of one delta entry of the token can move it by
        ulp_d = 2.0 ** (np.floor(np.log2(np.abs(xa).max(axis=1) + 1e-30)) - mant)
        flip = np.stack([ulp_d[tkn] * c.scales[c.bins[tkn]] * np.abs(B_p[c.bins[tkn]]).max(axis=0)
                         for tkn in range(batch)])

        def close(got, want, start=None):
            err = np.abs(got - want)
            tol = RTOL * np.abs(want) + ATOL
            if start is not None:   # one step of the storage type at the magnitude of y0 or of the update
                big = np.maximum(np.abs(start), np.abs(want - start))
                tol = tol + 2.0 ** (np.floor(np.log2(big + 1e-30)) - mant)
            bad = err > tol
            assert bad.sum() <= max(1, int(1e-4 * bad.size)), (p, int(bad.sum()), bad.size, float((err - tol).max()))
            assert np.all(err[bad] <= tol[bad] + flip[bad]), (p, float((err - tol - flip)[bad].max()))

        # ---- decode
        d = torch.zeros((batch, R), dtype=g.tdt, device=gpu)
        dispatch_bgmv(d, g.x, g.key, *t, p, g.scales)
        np.testing.assert_allclose(host(d), xa, rtol=RTOL, atol=ATOL)
        y = torch.zeros((batch, hidden), dtype=g.tdt, device=gpu)
        dispatch_bgmv(y, d, g.value, *t, p, g.scales)
        np.testing.assert_allclose(host(y), O.ref_bmm(zero, host(d), eye, B_p, c.scales, c.bins, dtype),
                                   rtol=RTOL, atol=ATOL)
        close(host(y), O.ref_bmm(zero, c.x, A_p, B_p, c.scales, c.bins, dtype))
        y = dev(y0, g.tdt, gpu)
        dispatch_bgmv(y, d, g.value, *t, p, g.scales)
        close(host(y), O.ref_bmm(y0, c.x, A_p, B_p, c.scales, c.bins, dtype), y0)
        # ---- prefill
        o = torch.zeros((batch, R), dtype=g.tdt, device=gpu)
        lora_get_qkvo_fwd_shrink(g.x, g.key.view(c.n_pages, hidden), o, *tp, hidden, p, R, int(lens.max()))
        np.testing.assert_allclose(host(o), xa, rtol=RTOL, atol=ATOL)
        y2 = torch.zeros((batch, hidden), dtype=g.tdt, device=gpu)
        lora_get_qkvo_fwd_expand(o, g.value.view(c.n_pages, hidden), y2, g.scales, *tp, hidden, p, R, int(lens.max()))
        np.testing.assert_allclose(host(y2), O.ref_bmm(zero, host(o), eye, B_p, c.scales, c.bins, dtype),
                                   rtol=RTOL, atol=ATOL)
        close(host(y2), O.ref_bmm(zero, c.x, A_p, B_p, c.scales, c.bins, dtype))
        y2 = dev(y0, g.tdt, gpu)
        lora_get_qkvo_fwd_expand(o, g.value.view(c.n_pages, hidden), y2, g.scales, *tp, hidden, p, R, int(lens.max()))
        close(host(y2), O.ref_bmm(y0, c.x, A_p, B_p, c.scales, c.bins, dtype), y0)


# ---------------------------------------------------------------------------
# y inside the pool
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_output_rows_inside_the_pool_passed_as_w(gpu, plan_cache_mode, dtype):
    """The reference's decode step writes k and v straight into pool rows: ``y`` is a
    contiguous row slice of the buffer that the same call reads adapter pages from (other
    rows).  Results must be bitwise those of a call whose y is a separate tensor, for the
    single call, the q/k/v launch and the prefill operator."""
    from slora_hip import (dispatch_bgmv, dispatch_bgmv_qkv_expand, lora_get_qkvo_fwd_expand)
    H, ranks, B = 1024, [64, 8, 32, 16], 70
    c = make_case(91, H, ranks, B, dtype=dtype, zipf_alpha=1.0)
    g = GpuCase(c, gpu)
    R = 64
    t = (g.a_start, g.a_len, g.a_loc, g.bins)
    gen = torch.Generator(device=gpu)
    gen.manual_seed(2)
    kv_rows = torch.randn((3 * B, 4, H // 4), generator=gen, device=gpu).to(g.tdt)
    pool = torch.cat([g.value, kv_rows]).contiguous()       # adapter pages first, then the rows the step writes
    n_pages = pool.size(0)
    deltas = []
    for p in range(3):
        d = torch.zeros((B, R), dtype=g.tdt, device=gpu)
        dispatch_bgmv(d, g.x, g.key, *t, p, g.scales)
        deltas.append(d)

    def slot(buf, i):
        return buf[c.n_pages + i * B: c.n_pages + (i + 1) * B].view(B, H)

    # separate outputs
    want = []
    for p in range(3):
        y = slot(pool, p).clone()
        dispatch_bgmv(y, deltas[p], pool, *t, p, g.scales)
        want.append(y)
    # outputs inside the buffer passed as w, one call per projection
    inside = pool.clone()
    for p in range(3):
        dispatch_bgmv(slot(inside, p), deltas[p], inside, *t, p, g.scales)
    torch.cuda.synchronize()
    for p in range(3):
        assert torch.equal(slot(inside, p), want[p]), p
    assert torch.equal(inside[: c.n_pages], pool[: c.n_pages])
    # the q/k/v launch
    inside = pool.clone()
    dispatch_bgmv_qkv_expand(slot(inside, 0), slot(inside, 1), slot(inside, 2), *deltas, inside, *t, g.scales)
    torch.cuda.synchronize()
    for p in range(3):
        assert torch.equal(slot(inside, p), want[p]), p
    # the prefill operator over the same tokens as one request per token run
    ids = c.bins.copy()
    st = dev(np.arange(B, dtype=np.int32), torch.int32, gpu)
    ln = torch.ones(B, dtype=torch.int32, device=gpu)
    rq = dev(ids, torch.int64, gpu)
    sep = slot(pool, 1).clone()
    lora_get_qkvo_fwd_expand(deltas[1], pool.view(n_pages, H), sep, g.scales, g.a_loc, g.a_start, g.a_len, st, ln, rq,
                             H, 1, R, 1)
    inside = pool.clone()
    lora_get_qkvo_fwd_expand(deltas[1], inside.view(n_pages, H), slot(inside, 1), g.scales, g.a_loc, g.a_start,
                             g.a_len, st, ln, rq, H, 1, R, 1)
    torch.cuda.synchronize()
    assert torch.equal(slot(inside, 1), sep)
