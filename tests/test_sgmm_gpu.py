"""Prefill segmented shrink / expand on the GPU against the CPU oracle, through
the C ABI.  Tolerance: rtol 1e-2, atol 1e-3 (fp16 and bf16)."""
import numpy as np
import pytest
import torch

from oracle import lora_oracle as O
from lora_cases import make_case, make_segments
from test_bgmv_gpu import GpuCase, dev, host, RTOL, ATOL, TDT

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["cache", "no-plan"])
def prefill_plan_mode(request):
    """Every test runs twice: with shrink calls served by the automatic per-batch plan
    (the default) and with the cache off, which sends them to the kernel that works out
    its share of the batch by itself."""
    import slora_hip
    slora_hip.set_plan_cache_enabled(request.param == "cache")
    slora_hip.clear_prefill_plan_cache()
    yield request.param
    slora_hip.clear_prefill_plan_cache()
    slora_hip.set_plan_cache_enabled(True)


def seg_case(seed, hidden, ranks, n_req, lo, hi, dtype, h_out=None, sort=True):
    start, lens, ids = make_segments(seed, n_req, lo, hi, len(ranks), sort_by_adapter=sort)
    T = int(lens.sum())
    c = make_case(seed, hidden, ranks, batch=T, dtype=dtype, bins=np.repeat(ids, lens), h_out=h_out)
    c.start, c.lens, c.ids = start, lens, ids
    return c


def run_prefill(c, g, p, R, device, o0, y0):
    from slora_hip import lora_get_qkvo_fwd_shrink, lora_get_qkvo_fwd_expand
    start = dev(c.start, torch.int32, device)
    lens = dev(c.lens, torch.int32, device)
    ids = dev(c.ids, torch.int64, device)
    max_len = int(c.lens.max()) if len(c.lens) else 0
    delta = dev(o0, g.tdt, device)
    w_a = g.key.view(c.n_pages, c.page_elems)
    w_b = g.value.view(c.n_pages, c.page_elems)
    lora_get_qkvo_fwd_shrink(g.x, w_a, delta, g.a_loc, g.a_start, g.a_len, start, lens, ids, c.hidden, p, R, max_len)
    y = dev(y0, g.tdt, device)
    lora_get_qkvo_fwd_expand(delta, w_b, y, g.scales, g.a_loc, g.a_start, g.a_len, start, lens, ids, c.h_out[p], p, R,
                             max_len)
    torch.cuda.synchronize()
    return host(delta), host(y)


def check(c, g, p, R, device, seed=0):
    rng = np.random.default_rng(seed)
    T = c.batch
    o0 = O.round_to(rng.standard_normal((T, R)).astype(np.float32), c.dtype)  # garbage that must be overwritten
    y0 = O.round_to(rng.standard_normal((T, c.h_out[p])).astype(np.float32), c.dtype)
    d_gpu, y_gpu = run_prefill(c, g, p, R, device, o0, y0)
    d_ref = O.ref_prefill_shrink(o0, c.x, c.key, c.a_loc, c.a_start, c.a_len, c.start, c.lens, c.ids, p, R, c.dtype)
    np.testing.assert_allclose(d_gpu, d_ref, rtol=RTOL, atol=ATOL)
    y_ref = O.ref_prefill_expand(y0, d_gpu, c.value, c.scales, c.a_loc, c.a_start, c.a_len, c.start, c.lens, c.ids, p,
                                 R, c.dtype)
    np.testing.assert_allclose(y_gpu, y_ref, rtol=RTOL, atol=ATOL)
    return d_gpu, y_gpu


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("hidden,ranks,n_req,lo,hi", [
    (256, [8, 16, 32, 64], 9, 1, 70),
    (1024, [64, 8, 16], 6, 8, 200),
    (4096, [64, 32, 16, 8], 8, 8, 300),
    (5120, [64, 32, 16], 4, 100, 256),
    (512, [128, 8], 5, 1, 40),
])
def test_prefill_chain_matches_oracle(gpu, dtype, hidden, ranks, n_req, lo, hi):
    c = seg_case(200 + hidden + n_req, hidden, ranks, n_req, lo, hi, dtype)
    g = GpuCase(c, gpu)
    R = max(ranks)
    for p in range(4):
        check(c, g, p, R, gpu, seed=p)


@pytest.mark.parametrize("n_req,lo,hi", [(257, 1, 9), (300, 1, 40), (700, 1, 6), (64, 60, 70)])
def test_prefill_many_requests(gpu, n_req, lo, hi):
    """More requests than the shrink kernel describes at a time (256), unsorted
    adapters, request lengths around the unit (16) and tile (64) sizes."""
    c = seg_case(500 + n_req, 256, [8, 16, 32, 64, 24], n_req, lo, hi, "bf16", sort=False)
    g = GpuCase(c, gpu)
    for p in (0, 3):
        check(c, g, p, 64, gpu, seed=p)


@pytest.mark.parametrize("lens", [
    [1500] + [3] * 40,                 # one long request among short ones
    [2049],                            # a single request cut into many chunks
    [700, 1, 64, 65, 128, 129, 16, 15, 17, 32, 33],   # lengths around the unit, tile and chunk sizes
    [5] * 256,                         # as many requests as one pass describes
    [40] * 255 + [900],                # ... with a long one at the end
], ids=["skewed", "single", "boundaries", "256-short", "255-and-long"])
def test_prefill_work_split(gpu, lens):
    """Request mixes that exercise how the kernels share out the work: per-request
    chunks (shrink), even shares of row tiles walked across request boundaries
    (expand), both with fewer requests than workgroups and with more."""
    lens = np.asarray(lens, dtype=np.int32)
    ranks = [64, 8, 32, 16]
    rng = np.random.default_rng(int(lens.sum()))
    ids = np.sort(rng.integers(0, len(ranks), size=len(lens))).astype(np.int64)
    start = np.zeros(len(lens), dtype=np.int32)
    start[1:] = np.cumsum(lens)[:-1]
    c = make_case(77, 320, ranks, batch=int(lens.sum()), dtype="bf16", bins=np.repeat(ids, lens))
    c.start, c.lens, c.ids = start, lens, ids
    g = GpuCase(c, gpu)
    for p in (1, 3):
        check(c, g, p, 64, gpu, seed=p)


@pytest.mark.parametrize("seed", range(10))
def test_prefill_random_configurations(gpu, seed):
    """Seeded random shapes for the segmented kernels: hidden any multiple of 8 up
    to 4096, ranks of every kind, 1 to 90 requests of 1 to 300 tokens, sorted by
    adapter or not, either dtype, all four projections against the oracle."""
    rng = np.random.default_rng(3000 + seed)
    hidden = int(rng.integers(2, 65)) * 8 * int(rng.choice([1, 2, 8]))
    ranks = [int(rng.choice([8, 16, 32, 64, 24, 40, 4, 12, 128])) for _ in range(int(rng.integers(1, 6)))]
    hidden = max(hidden, (max(ranks) + 15) // 8 * 8)
    n_req = int(rng.choice([1, 3, 17, 90]))
    hi = int(rng.choice([2, 40, 300]))
    dtype = str(rng.choice(["f16", "bf16"]))
    c = seg_case(3100 + seed, hidden, ranks, n_req, 1, hi, dtype, sort=bool(rng.integers(0, 2)))
    g = GpuCase(c, gpu)
    R = (max(ranks) + 7) // 8 * 8
    for p in range(4):
        check(c, g, p, R, gpu, seed=p)


def test_full_size_c3_against_dense_and_decode(gpu):
    """The C3 configuration itself (bf16, hidden 4096, 64 requests of 8..512 tokens,
    100 adapters of ranks {64,32,16,8}, 65536-page pool), one layer: shrink and
    expand against torch float32 on the device from the unpacked A, B (rtol 1e-2;
    atol 1e-3 for the shrink output, 2e-2 for y, which is a bf16 sum of order-1
    terms that may cancel), zero-fill of the columns beyond each rank, and rows
    that belong to no request left alone."""
    import workloads
    from slora_hip import lora_get_qkvo_fwd_shrink, lora_get_qkvo_fwd_expand
    w, seg = workloads.c3_prefill(gpu, n_layers=1)
    T, H, R = seg.n_tokens, w.hidden, w.max_rank
    g = torch.Generator(device=gpu)
    g.manual_seed(3)
    x = torch.randn((T + 5, H), generator=g, device=gpu).to(w.dtype)       # 5 rows owned by no request
    key, val = w.key_buffer[0], w.value_buffer[0]
    t = (w.a_loc, w.a_start, w.a_len, seg.b_start_loc, seg.b_seq_len, seg.b_indicies)
    starts = np.concatenate([[0], np.cumsum(seg.lens_np)[:-1]])
    for p in (0, 3):
        d = torch.full((T + 5, R), 9.0, dtype=w.dtype, device=gpu)
        lora_get_qkvo_fwd_shrink(x, key.view(-1, H), d, *t, H, p, R, seg.max_len)
        y0 = torch.randn((T + 5, H), generator=g, device=gpu).to(w.dtype)
        y = y0.clone()
        lora_get_qkvo_fwd_expand(d, val.view(-1, H), y, w.a_scaling, *t, H, p, R, seg.max_len)
        d_ref = torch.zeros((T, R), dtype=torch.float32, device=gpu)
        y_ref = y0[:T].float().clone()
        for i, a in enumerate(seg.ids_np):
            r = int(w.ranks[a])
            loc = w.a_loc[int(w.a_start_np[a]) + p * r: int(w.a_start_np[a]) + (p + 1) * r]
            rows = slice(int(starts[i]), int(starts[i]) + int(seg.lens_np[i]))
            d_ref[rows, :r] = x[rows].float() @ key[loc].reshape(r, H).float().t()
            y_ref[rows] += (d[rows, :r].float() @ val[loc].reshape(H, r).float().t()) * float(w.scales_np[a])
        np.testing.assert_allclose(d[:T].float().cpu().numpy(), d_ref.cpu().numpy(), rtol=RTOL, atol=ATOL)
        np.testing.assert_allclose(y[:T].float().cpu().numpy(), y_ref.cpu().numpy(), rtol=RTOL, atol=2e-2)
        assert torch.equal(d[T:], torch.full((5, R), 9.0, dtype=w.dtype, device=gpu))
        assert torch.equal(y[T:], y0[T:])


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_prefill_gather_bit_exact(gpu, dtype):
    rng = np.random.default_rng(5)
    H, ranks = 256, [8, 16, 32, 64]
    c = seg_case(5, H, ranks, 7, 1, 50, dtype, sort=False)
    for i, r in enumerate(ranks):
        c.A[i] = [rng.integers(-2, 3, (H, r)).astype(np.float32) for _ in range(4)]
        c.B[i] = [rng.integers(-2, 3, (r, H)).astype(np.float32) for _ in range(4)]
        loc = c.a_loc[c.a_start[i]: c.a_start[i] + 4 * r]
        O.load_into_pool(c.key, c.value, O.pack_w_combined(c.A[i], c.B[i], H), loc)
    x = np.zeros((c.batch, H), np.float32)
    for t in range(c.batch):
        idx = rng.choice(H, size=3, replace=False)
        x[t, idx] = rng.integers(-2, 3, 3)
    c.x = x
    c.scales = np.array([1.0, 2.0, 0.5, 0.25], np.float32)
    g = GpuCase(c, gpu)
    for p in range(4):
        o0 = np.full((c.batch, 64), 9.0, np.float32)
        y0 = np.zeros((c.batch, H), np.float32)
        d_gpu, y_gpu = run_prefill(c, g, p, 64, gpu, o0, y0)
        for t in range(c.batch):
            a = c.bins[t]
            d = c.x[t] @ c.A[a][p]
            assert np.array_equal(d_gpu[t, : ranks[a]], d), (p, t)
            assert np.all(d_gpu[t, ranks[a]:] == 0), (p, t)      # zero fill up to max_rank
            assert np.array_equal(y_gpu[t], O.round_to((d @ c.B[a][p]) * c.scales[a], dtype)), (p, t)


def test_prefill_unowned_rows_and_empty_requests(gpu):
    """Rows no request owns stay as they were; zero-length requests do nothing."""
    c = make_case(6, 256, [8, 16], batch=40, dtype="f16", bins=np.zeros(40, np.int64))
    c.start = np.array([3, 20, 30], np.int32)
    c.lens = np.array([5, 0, 7], np.int32)
    c.ids = np.array([1, 0, 0], np.int64)
    c.bins[3:8] = 1
    g = GpuCase(c, gpu)
    o0 = np.full((40, 16), 5.0, np.float32)
    y0 = np.full((40, 256), 2.0, np.float32)
    d_gpu, y_gpu = run_prefill(c, g, 1, 16, gpu, o0, y0)
    owned = np.zeros(40, bool)
    owned[3:8] = True
    owned[30:37] = True
    assert np.all(d_gpu[~owned] == 5.0) and np.all(y_gpu[~owned] == 2.0)
    d_ref = O.ref_prefill_shrink(o0, c.x, c.key, c.a_loc, c.a_start, c.a_len, c.start, c.lens, c.ids, 1, 16, "f16")
    np.testing.assert_allclose(d_gpu, d_ref, rtol=RTOL, atol=ATOL)


def test_prefill_strided_views_and_odd_layouts(gpu):
    """x / o as row-strided views (the reference passes strides), a rank that
    is not a multiple of 8 and an output width that is not a multiple of 8
    (element-wise path)."""
    from slora_hip import lora_get_qkvo_fwd_shrink, lora_get_qkvo_fwd_expand
    c = seg_case(7, 256, [12, 8, 20], 5, 3, 40, "f16")
    g = GpuCase(c, gpu)
    R = 24
    T = c.batch
    start, lens, ids = dev(c.start, torch.int32, gpu), dev(c.lens, torch.int32, gpu), dev(c.ids, torch.int64, gpu)
    max_len = int(c.lens.max())
    x_wide = torch.zeros((T, 256 + 24), dtype=torch.float16, device=gpu)
    x_wide[:, :256] = g.x
    xv = x_wide[:, :256]
    d_wide = torch.zeros((T, R + 3), dtype=torch.float16, device=gpu)
    dv = d_wide[:, :R]
    lora_get_qkvo_fwd_shrink(xv, g.key.view(c.n_pages, 256), dv, g.a_loc, g.a_start, g.a_len, start, lens, ids, 256, 2,
                             R, max_len)
    d_ref = O.ref_prefill_shrink(np.zeros((T, R), np.float32), c.x, c.key, c.a_loc, c.a_start, c.a_len, c.start,
                                 c.lens, c.ids, 2, R, "f16")
    np.testing.assert_allclose(host(dv), d_ref, rtol=RTOL, atol=ATOL)
    assert torch.all(d_wide[:, R:] == 0)
    y_wide = torch.ones((T, 256 + 5), dtype=torch.float16, device=gpu)
    yv = y_wide[:, :256]
    lora_get_qkvo_fwd_expand(dv, g.value.view(c.n_pages, 256), yv, g.scales, g.a_loc, g.a_start, g.a_len, start, lens,
                             ids, 256, 2, R, max_len)
    y_ref = O.ref_prefill_expand(np.ones((T, 256), np.float32), host(dv), c.value, c.scales, c.a_loc, c.a_start,
                                 c.a_len, c.start, c.lens, c.ids, 2, R, "f16")
    np.testing.assert_allclose(host(yv), y_ref, rtol=RTOL, atol=ATOL)
    assert torch.all(y_wide[:, 256:] == 1)


def test_prefill_matches_decode_kernels(gpu):
    """The two operator families must agree where the reference treats them as
    interchangeable (lora_unordered_batch_infer.py:334-355)."""
    from slora_hip import dispatch_bgmv
    c = seg_case(8, 1024, [64, 16, 32], 6, 5, 90, "f16")
    g = GpuCase(c, gpu)
    R = 64
    d_gpu, y_gpu = run_prefill(c, g, 0, R, gpu, np.zeros((c.batch, R), np.float32), np.zeros((c.batch, 1024), np.float32))
    delta = torch.zeros((c.batch, R), dtype=torch.float16, device=gpu)
    dispatch_bgmv(delta, g.x, g.key, g.a_start, g.a_len, g.a_loc, g.bins, 0, g.scales)
    y = torch.zeros((c.batch, 1024), dtype=torch.float16, device=gpu)
    dispatch_bgmv(y, delta, g.value, g.a_start, g.a_len, g.a_loc, g.bins, 0, g.scales)
    np.testing.assert_allclose(host(delta), d_gpu, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(host(y), y_gpu, rtol=2 * RTOL, atol=4 * ATOL)


def _shrink_args(c, g, device):
    start = dev(c.start, torch.int32, device)
    lens = dev(c.lens, torch.int32, device)
    ids = dev(c.ids, torch.int64, device)
    return start, lens, ids, int(c.lens.max())


@pytest.mark.parametrize("hidden,ranks,n_req,lo,hi", [
    (256, [8, 16, 32, 64], 9, 1, 70),       # small batch: rank columns shared by 4 workgroups
    (1024, [64, 8, 16], 40, 30, 200),       # one chunk or a few per request
    (320, [128, 24], 5, 1, 300),            # two passes over the rank, odd rank (element-wise path)
    (256, [16, 32], 300, 1, 9),             # more requests than a plan describes: the plain kernel runs
])
def test_prefill_plan_gives_the_plain_kernels_bits(gpu, hidden, ranks, n_req, lo, hi):
    """An explicit plan, the automatic one and no plan at all: identical outputs."""
    from slora_hip import lora_get_qkvo_fwd_shrink, make_prefill_plan
    c = seg_case(900 + n_req, hidden, ranks, n_req, lo, hi, "bf16")
    g = GpuCase(c, gpu)
    start, lens, ids, max_len = _shrink_args(c, g, gpu)
    R = (max(ranks) + 7) // 8 * 8
    plan = make_prefill_plan(g.a_start, g.a_len, start, lens, ids, c.batch, R, max_len)
    assert plan.usable == (n_req <= 256)
    w_a = g.key.view(c.n_pages, c.page_elems)
    for p in range(4):
        outs = []
        for how in (False, plan, None):
            o = torch.full((c.batch, R), 7.0, dtype=g.tdt, device=gpu)
            lora_get_qkvo_fwd_shrink(g.x, w_a, o, g.a_loc, g.a_start, g.a_len, start, lens, ids, c.hidden, p, R,
                                     max_len, plan=how)
            outs.append(o)
        torch.cuda.synchronize()
        assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2]), p


def test_prefill_plan_cache_follows_the_index_tensors(gpu, prefill_plan_mode):
    import slora_hip
    from slora_hip import lora_get_qkvo_fwd_shrink
    if prefill_plan_mode != "cache":
        pytest.skip("cache switched off")
    c = seg_case(31, 256, [16, 8, 32], 12, 1, 90, "f16")
    g = GpuCase(c, gpu)
    start, lens, ids, max_len = _shrink_args(c, g, gpu)
    w_a = g.key.view(c.n_pages, c.page_elems)
    slora_hip.plan_cache_stats(reset=True)

    def stats():
        s = slora_hip.plan_cache_stats()
        return s["prefill_builds"], s["prefill_hits"]

    def both(lens_t, ids_t):
        o0 = torch.full((c.batch, 32), 3.0, dtype=g.tdt, device=gpu)  # rows of no request keep this value
        o1 = o0.clone()
        lora_get_qkvo_fwd_shrink(g.x, w_a, o0, g.a_loc, g.a_start, g.a_len, start, lens_t, ids_t, c.hidden, 2, 32,
                                 max_len, plan=False)
        lora_get_qkvo_fwd_shrink(g.x, w_a, o1, g.a_loc, g.a_start, g.a_len, start, lens_t, ids_t, c.hidden, 2, 32,
                                 max_len)
        torch.cuda.synchronize()
        assert torch.equal(o0, o1)

    both(lens, ids)
    both(lens, ids)
    assert stats() == (1, 1)
    ids.copy_(torch.flip(ids, dims=[0]))          # in place: the version changes, the plan is rebuilt
    both(lens, ids)
    assert stats()[0] == 2
    lens2 = lens.clone()                          # another object with the same values: rebuilt as well
    both(lens2, ids)
    assert stats()[0] == 3
    lens2[0] = 0                                  # a request dropped in place
    both(lens2, ids)
    assert stats()[0] == 4
    # a caller that makes new tensors for every call gets no plan after a few useless builds
    for _ in range(8 + 3):
        both(lens2.clone(), ids)
    assert stats()[0] <= 4 + 8
    built = stats()[0]
    both(lens2.clone(), ids)                      # paused: no build
    assert stats()[0] == built


def test_prefill_plan_of_another_batch_is_rejected(gpu):
    from slora_hip import lora_get_qkvo_fwd_shrink, make_prefill_plan
    c = seg_case(32, 256, [16, 8], 6, 1, 50, "f16")
    g = GpuCase(c, gpu)
    start, lens, ids, max_len = _shrink_args(c, g, gpu)
    plan = make_prefill_plan(g.a_start, g.a_len, start, lens, ids, c.batch, 16, max_len)
    o = torch.zeros((c.batch, 32), dtype=g.tdt, device=gpu)
    with pytest.raises(RuntimeError, match="another batch"):
        lora_get_qkvo_fwd_shrink(g.x, g.key.view(c.n_pages, c.page_elems), o, g.a_loc, g.a_start, g.a_len, start, lens,
                                 ids, c.hidden, 0, 32, max_len, plan=plan)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("hidden,ranks,n_req,lo,hi,sort", [
    (256, [8, 16, 32, 64], 9, 1, 70, True),        # small batch: rank columns shared by 4 workgroups
    (1024, [64, 8, 16], 40, 30, 200, True),        # a few chunks per request
    (4096, [64, 32, 16, 8], 12, 8, 300, True),     # the hidden size of the headline configurations
    (320, [128, 24], 5, 1, 300, False),            # two passes over the rank; rank 24 takes the element-wise path
    (256, [16, 32], 300, 1, 9, False),             # more requests than a plan describes
    (200, [8, 40, 16], 7, 1, 90, False),           # hidden size that is no multiple of 64: ragged last k block
    (64, [8], 3, 1, 20, True),                     # a single k block per row
    (128, [16, 8], 4, 1, 30, True),                # two k blocks: fewer blocks than wavefronts
    # larger batches (more row parts than workgroups of a launch)
    (256, [16, 8, 64, 32], 45, 90, 130, True),
    (200, [8, 40, 16], 50, 80, 120, False),        # ragged last k block, a rank on the element-wise path
    (320, [128, 24], 300, 10, 22, False),          # two passes over the rank, more requests than a plan describes
])
def test_prefill_qkv_shrink_gives_the_three_calls_bits(gpu, dtype, hidden, ranks, n_req, lo, hi, sort):
    """lora_get_qkvo_fwd_shrink_qkv (x read once for q, k and v) against the three calls
    the reference issues (lora_unordered_batch_infer.py:334-347 and the k, v blocks after
    it): identical bits, with a plan and without; rows of no request and the columns
    beyond max_rank stay as they were."""
    from slora_hip import lora_get_qkvo_fwd_shrink, lora_get_qkvo_fwd_shrink_qkv
    c = seg_case(1200 + hidden + n_req, hidden, ranks, n_req, lo, hi, dtype, sort=sort)
    g = GpuCase(c, gpu)
    start, lens, ids, max_len = _shrink_args(c, g, gpu)
    R = (max(ranks) + 7) // 8 * 8
    w_a = g.key.view(c.n_pages, c.page_elems)
    T = c.batch
    x = torch.cat([g.x, torch.ones((3, c.hidden), dtype=g.tdt, device=gpu)])     # 3 rows owned by no request
    t = (g.a_loc, g.a_start, g.a_len, start, lens, ids)
    single = []
    for p in range(3):
        o = torch.full((T + 3, R + 8), 7.0, dtype=g.tdt, device=gpu)
        lora_get_qkvo_fwd_shrink(x, w_a, o[:, :R], *t, c.hidden, p, R, max_len, plan=False)
        single.append(o)
    for how in (False, None):
        fused = [torch.full((T + 3, R + 8), 7.0, dtype=g.tdt, device=gpu) for _ in range(3)]
        lora_get_qkvo_fwd_shrink_qkv(x, w_a, fused[0][:, :R], fused[1][:, :R], fused[2][:, :R], *t, c.hidden, R, max_len,
                                     plan=how)
        torch.cuda.synchronize()
        for p in range(3):
            assert torch.equal(fused[p], single[p]), (p, how)
    d_ref = O.ref_prefill_shrink(np.zeros((T, R), np.float32), c.x, c.key, c.a_loc, c.a_start, c.a_len, c.start,
                                 c.lens, c.ids, 1, R, c.dtype)
    np.testing.assert_allclose(host(single[1][:T, :R]), d_ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("hidden,ranks,n_req,lo,hi,sort,x_pad,o_off", [
    (256, [8, 16, 32, 64], 60, 60, 110, True, 0, 0),      # whole and partial 64-row tiles of every tile count
    (512, [128, 24, 40], 50, 80, 130, False, 0, 0),       # two passes over the rank; ranks that end inside a 16-column tile
    (256, [64, 8], 70, 1, 150, False, 64, 8),             # strided x, output columns at an aligned offset of a wider buffer
    (128, [32, 16], 40, 100, 140, True, 8, 4),            # output rows that are not 16-byte aligned: element-wise stores
    (128, [64, 16], 20, 900, 1100, True, 0, 0),           # more than 64 rows per workgroup: several tiles in one stream of blocks
])
def test_prefill_shrink_above_4096_tokens(gpu, dtype, hidden, ranks, n_req, lo, hi, sort, x_pad, o_off):
    """Batches of more than 4096 tokens take the kernels whose K loop streams through LDS (whole
    64-k blocks, 64-row tiles, the wavefronts splitting the outputs): single projection and
    q/k/v in one launch against the oracle at rtol 1e-2 / atol 1e-3, the fused launch bit for bit
    the three calls, with and without a plan; columns outside [0, max_rank) of a wider output
    buffer and rows of no request keep what they held."""
    from slora_hip import lora_get_qkvo_fwd_shrink, lora_get_qkvo_fwd_shrink_qkv
    c = seg_case(2000 + hidden + n_req, hidden, ranks, n_req, lo, hi, dtype, sort=sort)
    assert c.batch > 4096
    g = GpuCase(c, gpu)
    start, lens, ids, max_len = _shrink_args(c, g, gpu)
    R = (max(ranks) + 7) // 8 * 8
    T = c.batch
    w_a = g.key.view(c.n_pages, c.page_elems)
    xb = torch.zeros((T + 2, hidden + x_pad), dtype=g.tdt, device=gpu)
    xb[:T, :hidden] = g.x
    x = xb[:, :hidden]
    t = (g.a_loc, g.a_start, g.a_len, start, lens, ids)
    outs = {}
    for how in (False, None):
        single = []
        for p in range(3):
            ob = torch.full((T + 2, R + 16), 7.0, dtype=g.tdt, device=gpu)
            lora_get_qkvo_fwd_shrink(x, w_a, ob[:, o_off:o_off + R], *t, hidden, p, R, max_len, plan=how)
            single.append(ob)
        fused = [torch.full((T + 2, R + 16), 7.0, dtype=g.tdt, device=gpu) for _ in range(3)]
        lora_get_qkvo_fwd_shrink_qkv(x, w_a, *[f[:, o_off:o_off + R] for f in fused], *t, hidden, R, max_len, plan=how)
        torch.cuda.synchronize()
        for p in range(3):
            assert torch.equal(fused[p], single[p]), (p, how)
        outs[how] = single
    for p in range(3):
        assert torch.equal(outs[False][p], outs[None][p]), p
        ob = outs[None][p]
        d_ref = O.ref_prefill_shrink(np.full((T, R), 7.0, np.float32), c.x, c.key, c.a_loc, c.a_start, c.a_len, c.start,
                                     c.lens, c.ids, p, R, c.dtype)
        np.testing.assert_allclose(host(ob[:T, o_off:o_off + R]), d_ref, rtol=RTOL, atol=ATOL)
        keep = torch.full((1,), 7.0, dtype=g.tdt, device=gpu)
        assert torch.all(ob[:, :o_off] == keep) and torch.all(ob[:, o_off + R:] == keep) and torch.all(ob[T:] == keep)


def test_prefill_qkv_shrink_rejects_mismatched_outputs(gpu):
    from slora_hip import lora_get_qkvo_fwd_shrink_qkv
    c = seg_case(33, 256, [16, 8], 6, 1, 50, "f16")
    g = GpuCase(c, gpu)
    start, lens, ids, max_len = _shrink_args(c, g, gpu)
    o = [torch.zeros((c.batch, 16), dtype=g.tdt, device=gpu) for _ in range(2)]
    wide = torch.zeros((c.batch, 24), dtype=g.tdt, device=gpu)
    with pytest.raises(RuntimeError, match="share dtype, shape and row stride"):
        lora_get_qkvo_fwd_shrink_qkv(g.x, g.key.view(c.n_pages, c.page_elems), o[0], o[1], wide, g.a_loc, g.a_start,
                                     g.a_len, start, lens, ids, c.hidden, 16, max_len)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("hidden,h_kv,ranks,n_req,lo,hi", [
    (512, 512, [64, 8, 16, 32], 9, 1, 120),        # q, k and v as wide as a page
    (1024, 256, [64, 16], 6, 8, 200),              # grouped-query widths: k and v a quarter of a page
    (512, 128, [8, 32], 5, 1, 40),                 # k and v narrower than one output group of a workgroup
    (256, 256, [16, 32], 300, 1, 9),               # more requests than one workgroup describes
    (256, 256, [12, 8, 20], 5, 3, 40),             # ranks that take the element-wise path
    (4096, 4096, [64, 32, 16, 8], 12, 100, 600),   # C3's widths
])
def test_prefill_qkv_expand_gives_the_three_calls_bits(gpu, dtype, hidden, h_kv, ranks, n_req, lo, hi):
    """lora_get_qkvo_fwd_expand_qkv (one launch for q, k and v) against the three calls the reference
    issues (lora_unordered_batch_infer.py:349-372 and the k, v blocks after it): identical bits,
    also in rows that belong to no request and in the columns beyond the outputs' widths; one of
    the three results is checked against the oracle."""
    from slora_hip import lora_get_qkvo_fwd_expand, lora_get_qkvo_fwd_expand_qkv
    c = seg_case(2300 + hidden + n_req, hidden, ranks, n_req, lo, hi, dtype, h_out=[hidden, h_kv, h_kv, hidden])
    g = GpuCase(c, gpu)
    start, lens, ids = dev(c.start, torch.int32, gpu), dev(c.lens, torch.int32, gpu), dev(c.ids, torch.int64, gpu)
    max_len = int(c.lens.max())
    R = (max(ranks) + 7) // 8 * 8
    T = c.batch
    rng = np.random.default_rng(5)
    w_b = g.value.view(c.n_pages, c.page_elems)
    t = (g.a_loc, g.a_start, g.a_len, start, lens, ids)
    widths = [hidden, h_kv, h_kv]
    deltas = [dev(O.round_to(rng.standard_normal((T + 2, R)).astype(np.float32), c.dtype), g.tdt, gpu) for _ in range(3)]
    y0 = [O.round_to(rng.standard_normal((T + 2, widths[p] + 8)).astype(np.float32), c.dtype) for p in range(3)]
    single = [dev(y0[p], g.tdt, gpu) for p in range(3)]
    for p in range(3):
        lora_get_qkvo_fwd_expand(deltas[p], w_b, single[p][:, :widths[p]], g.scales, *t, widths[p], p, R, max_len)
    fused = [dev(y0[p], g.tdt, gpu) for p in range(3)]
    lora_get_qkvo_fwd_expand_qkv(deltas[0], deltas[1], deltas[2], w_b, fused[0][:, :hidden], fused[1][:, :h_kv],
                                 fused[2][:, :h_kv], g.scales, *t, hidden, h_kv, R, max_len)
    torch.cuda.synchronize()
    for p in range(3):
        assert torch.equal(fused[p], single[p]), p
        assert torch.equal(fused[p][T:], dev(y0[p], g.tdt, gpu)[T:])           # rows of no request
        assert torch.equal(fused[p][:, widths[p]:], dev(y0[p], g.tdt, gpu)[:, widths[p]:])
    y_ref = O.ref_prefill_expand(y0[2][:T, :h_kv], host(deltas[2])[:T], c.value, c.scales, c.a_loc, c.a_start, c.a_len,
                                 c.start, c.lens, c.ids, 2, R, c.dtype)
    np.testing.assert_allclose(host(fused[2][:T, :h_kv]), y_ref, rtol=RTOL, atol=ATOL)


def test_prefill_qkv_expand_rejects_mismatched_tensors(gpu):
    from slora_hip import lora_get_qkvo_fwd_expand_qkv
    c = seg_case(34, 256, [16, 8], 6, 1, 50, "f16")
    g = GpuCase(c, gpu)
    start, lens, ids = dev(c.start, torch.int32, gpu), dev(c.lens, torch.int32, gpu), dev(c.ids, torch.int64, gpu)
    d = [torch.zeros((c.batch, 16), dtype=g.tdt, device=gpu) for _ in range(3)]
    y = [torch.zeros((c.batch, 256), dtype=g.tdt, device=gpu) for _ in range(2)]
    narrow = torch.zeros((c.batch, 128), dtype=g.tdt, device=gpu)
    t = (g.a_loc, g.a_start, g.a_len, start, lens, ids)
    with pytest.raises(RuntimeError, match="o_k and o_v must share shape"):
        lora_get_qkvo_fwd_expand_qkv(d[0], d[1], d[2], g.value.view(c.n_pages, 256), y[0], y[1], narrow, g.scales, *t,
                                     256, 256, 16, int(c.lens.max()))
    with pytest.raises(RuntimeError, match="x_q, x_k and x_v must share shape"):
        lora_get_qkvo_fwd_expand_qkv(d[0], d[1], d[2][:, :8], g.value.view(c.n_pages, 256), y[0], y[1], y[1], g.scales,
                                     *t, 256, 256, 16, int(c.lens.max()))
