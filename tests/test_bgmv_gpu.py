"""Decode shrink / expand on the GPU against the CPU oracle.

Everything goes through the C ABI of libslora_hip.so (``slora_hip.dispatch_bgmv`` is the
compiled extension's check-and-call in front of it).  Tolerance for floating point is the one
the task states: rtol 1e-2, atol 1e-3 in fp16 and bf16.  Gather/index work is
checked bit-exactly with integer-valued cases.
"""
import numpy as np
import pytest
import torch

from oracle import lora_oracle as O
from lora_cases import make_case

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-3
TDT = {"f16": torch.float16, "bf16": torch.bfloat16}


@pytest.fixture(autouse=True, params=["cache", "stateless"])
def plan_cache_mode(request):
    """Every test runs twice: with calls that pass no plan served by the
    automatic plan cache (the default), and with the cache off, which sends the
    same calls to the kernels that find their runs by themselves."""
    import slora_hip
    slora_hip.set_plan_cache_enabled(request.param == "cache")
    slora_hip.clear_plan_cache()
    yield request.param
    slora_hip.clear_plan_cache()
    slora_hip.set_plan_cache_enabled(True)


def dev(a, dtype, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device=device, dtype=dtype)


def host(t):
    return t.detach().to(torch.float32).cpu().numpy()


class GpuCase:
    def __init__(self, c, device, heads=None):
        tdt = TDT[c.dtype]
        heads = heads or (4 if c.page_elems % 4 == 0 else 1)
        self.key = dev(c.key, tdt, device).view(c.n_pages, heads, c.page_elems // heads)
        self.value = dev(c.value, tdt, device).view(c.n_pages, heads, c.page_elems // heads)
        self.a_start = dev(c.a_start, torch.int64, device)
        self.a_len = dev(c.a_len, torch.int64, device)
        self.a_loc = dev(c.a_loc, torch.int64, device)
        self.bins = dev(c.bins, torch.int64, device)
        self.scales = dev(c.scales, torch.float16, device)
        self.x = dev(c.x, tdt, device)
        self.tdt = tdt


def run_chain(c, g, p, R, device, y0=None):
    from slora_hip import dispatch_bgmv
    delta = torch.zeros((c.batch, R), dtype=g.tdt, device=device)
    dispatch_bgmv(delta, g.x, g.key, g.a_start, g.a_len, g.a_loc, g.bins, p, g.scales)
    y = torch.zeros((c.batch, c.h_out[p]), dtype=g.tdt, device=device) if y0 is None else dev(y0, g.tdt, device)
    dispatch_bgmv(y, delta, g.value, g.a_start, g.a_len, g.a_loc, g.bins, p, g.scales)
    torch.cuda.synchronize()
    return host(delta), host(y)


def assert_close_but_for_rounding_flips(got, want, rtol, atol, dtype):
    """rtol / atol as stated, except that at most 2 in 100 000 elements may differ by one rounding
    step of the storage type at the magnitude of the values that were summed (2^-8 of the largest
    |value| for bf16, 2^-11 for fp16): y = T(y0 + T(scale * sum)) rounds twice at the magnitude of
    y0, the kernel and the oracle add up the fp32 sum in different orders, and where y0 and the
    delta cancel, one flipped rounding is larger than any tolerance relative to the small result."""
    bad = np.abs(got - want) > atol + rtol * np.abs(want)
    if not bad.any():
        return
    step = float(np.abs(want).max()) * (2.0 ** -8 if dtype == "bf16" else 2.0 ** -11)
    assert bad.sum() <= max(1, int(2e-5 * bad.size)), f"{bad.sum()} of {bad.size} elements outside rtol/atol"
    assert np.abs(got - want)[bad].max() <= step, (np.abs(got - want)[bad].max(), step)


def oracle_chain(c, p, R, y0=None):
    delta = O.ref_bgmv_shrink(np.zeros((c.batch, R), np.float32), c.x, c.key, c.a_start, c.a_len, c.a_loc, c.bins, p,
                              dtype=c.dtype)
    y0 = np.zeros((c.batch, c.h_out[p]), np.float32) if y0 is None else y0
    y = O.ref_bgmv_expand(y0, delta, c.value, c.a_start, c.a_len, c.a_loc, c.bins, p, c.scales, dtype=c.dtype)
    return delta, y


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("hidden,ranks,batch", [
    (256, [8, 16, 32, 64], 37),
    (1024, [8, 16], 128),          # shape of test_kernel_correctness_multi_rank.py
    (4096, [64, 32, 16, 8, 64, 8], 64),
    (5120, [64, 32, 16], 19),
    (768, [128, 8], 9),
    (4608, [16, 32], 40),          # page widths of the shrink's wider straight-line paths, whole and
    (6144, [32, 16], 23),          # partial last vector columns, runs of up to four tokens
    (5632, [16, 32], 30),
    (8192, [16, 32], 21),
    (7168, [16], 11),
    (8704, [32, 16], 9),           # wider than any of them: the general path
])
def test_decode_chain_matches_oracle(gpu, dtype, hidden, ranks, batch):
    c = make_case(100 + hidden + batch, hidden, ranks, batch, dtype=dtype, zipf_alpha=1.0)
    g = GpuCase(c, gpu)
    R = max(ranks)
    for p in range(4):
        y0 = O.round_to(np.random.default_rng(p).standard_normal((batch, hidden)).astype(np.float32), dtype)
        d_gpu, y_gpu = run_chain(c, g, p, R, gpu, y0)
        d_ref, y_ref = oracle_chain(c, p, R, y0)
        np.testing.assert_allclose(d_gpu, d_ref, rtol=RTOL, atol=ATOL)
        # expand is checked on the GPU's own shrink output so one rounding flip in delta is not amplified
        y_ref2 = O.ref_bgmv_expand(y0, d_gpu, c.value, c.a_start, c.a_len, c.a_loc, c.bins, p, c.scales, dtype=dtype)
        assert_close_but_for_rounding_flips(y_gpu, y_ref2, RTOL, ATOL, dtype)
        assert_close_but_for_rounding_flips(y_gpu, y_ref, 2 * RTOL, 4 * ATOL, dtype)


def test_reference_kernel_test_shapes(gpu):
    """The fixture of test/kernel/test_kernel_correctness.py:57-95: H=4096,
    R=128, N=128, 2 adapters back to back, identity a_loc, scaling 1, qkvo=1,
    expand; checked against that script's closed form."""
    rng = np.random.default_rng(42)
    H, R, N, n_ad, qkvo = 4096, 128, 128, 2, 1
    key = O.round_to(rng.standard_normal((R * 4 * n_ad, H)).astype(np.float32), "f16")
    a_len = np.full(n_ad, R * 4, np.int64)
    a_start = np.array([0, R * 4], np.int64)
    a_loc = np.arange(R * 4 * n_ad, dtype=np.int64)
    bins = np.repeat(np.arange(n_ad), N // n_ad).astype(np.int64)
    x = O.round_to(rng.standard_normal((N, R)).astype(np.float32), "f16")
    ref = np.zeros((N, H))
    for i in range(N):
        a = bins[i]
        a_w = key[a_start[a] + qkvo * R: a_start[a] + (qkvo + 1) * R].reshape(H, R).T
        ref[i] = x[i].astype(np.float64) @ a_w.astype(np.float64)
    from slora_hip import dispatch_bgmv
    y = torch.zeros((N, H), dtype=torch.float16, device=gpu)
    dispatch_bgmv(y, dev(x, torch.float16, gpu), dev(key, torch.float16, gpu).view(-1, 32, H // 32),
                  dev(a_start, torch.int64, gpu), dev(a_len, torch.int64, gpu), dev(a_loc, torch.int64, gpu),
                  dev(bins, torch.int64, gpu), qkvo, torch.ones(n_ad, dtype=torch.float16, device=gpu))
    np.testing.assert_allclose(host(y), ref, rtol=RTOL, atol=2e-2)  # |ref| ~ 11, fp16 ulp there is 8e-3


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_gather_is_bit_exact(gpu, dtype):
    """Integer-valued weights and activations: every partial sum is exact in
    fp32 and the results are exact in the storage type, so equality is
    bitwise.  Any wrong page / offset / split shows."""
    rng = np.random.default_rng(7)
    H, ranks, batch = 512, [8, 16, 32, 8, 64], 96
    c = make_case(7, H, ranks, batch, dtype=dtype, zipf_alpha=0.8)
    for i, r in enumerate(ranks):
        c.A[i] = [rng.integers(-2, 3, (H, r)).astype(np.float32) for _ in range(4)]
        c.B[i] = [rng.integers(-2, 3, (r, H)).astype(np.float32) for _ in range(4)]
        loc = c.a_loc[c.a_start[i]: c.a_start[i] + 4 * r]
        O.load_into_pool(c.key, c.value, O.pack_w_combined(c.A[i], c.B[i], H), loc)
    # sparse small-integer activations keep |delta| and |y| small enough to be exact in bf16 too
    x = np.zeros((batch, H), np.float32)
    for t in range(batch):
        idx = rng.choice(H, size=3, replace=False)
        x[t, idx] = rng.integers(-2, 3, 3)
    c.x = x
    c.scales = np.array([1.0, 2.0, 0.5, 1.0, 0.25], np.float32)
    g = GpuCase(c, gpu)
    for p in range(4):
        d_gpu, y_gpu = run_chain(c, g, p, 64, gpu)
        for t in range(batch):
            a = c.bins[t]
            d = c.x[t] @ c.A[a][p]
            assert np.array_equal(d_gpu[t, : ranks[a]], d), (p, t)
            assert np.all(d_gpu[t, ranks[a]:] == 0)
            want = O.round_to((d @ c.B[a][p]) * c.scales[a], dtype)
            assert np.array_equal(y_gpu[t], want), (p, t)


def test_shrink_leaves_columns_beyond_rank_untouched(gpu):
    c = make_case(8, 256, [8, 16], 20, dtype="f16")
    g = GpuCase(c, gpu)
    from slora_hip import dispatch_bgmv
    delta = torch.full((c.batch, 32), 3.0, dtype=torch.float16, device=gpu)
    dispatch_bgmv(delta, g.x, g.key, g.a_start, g.a_len, g.a_loc, g.bins, 2, g.scales)
    d = host(delta)
    for t in range(c.batch):
        r = c.ranks[c.bins[t]]
        assert np.all(d[t, r:] == 3.0)
        assert not np.any(d[t, :r] == 3.0)


def test_expand_ignores_garbage_beyond_rank_and_scale_zero(gpu):
    c = make_case(9, 256, [8, 16, 32], 33, dtype="f16")
    g = GpuCase(c, gpu)
    from slora_hip import dispatch_bgmv
    R = 32
    delta = torch.zeros((c.batch, R), dtype=torch.float16, device=gpu)
    dispatch_bgmv(delta, g.x, g.key, g.a_start, g.a_len, g.a_loc, g.bins, 1, g.scales)
    y1 = torch.zeros((c.batch, 256), dtype=torch.float16, device=gpu)
    dispatch_bgmv(y1, delta, g.value, g.a_start, g.a_len, g.a_loc, g.bins, 1, g.scales)
    junk = delta.clone()
    for t in range(c.batch):
        junk[t, c.ranks[c.bins[t]]:] = 1000.0
    y2 = torch.zeros_like(y1)
    dispatch_bgmv(y2, junk, g.value, g.a_start, g.a_len, g.a_loc, g.bins, 1, g.scales)
    assert torch.equal(y1, y2)
    y3 = torch.randn_like(y1)
    y3_before = y3.clone()
    dispatch_bgmv(y3, delta, g.value, g.a_start, g.a_len, g.a_loc, g.bins, 1, torch.zeros_like(g.scales))
    assert torch.equal(y3, y3_before)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_gqa_narrow_kv_and_wide_pages(gpu, dtype):
    """Output narrower than a page (k/v of grouped-query attention): hidden
    1024, k/v width 256, page = 1024 elements."""
    c = make_case(11, 1024, [64, 16, 8], 40, dtype=dtype, h_out=[1024, 256, 256, 1024])
    g = GpuCase(c, gpu)
    for p in range(4):
        d_gpu, y_gpu = run_chain(c, g, p, 64, gpu)
        y_ref = O.ref_bgmv_expand(np.zeros((c.batch, c.h_out[p]), np.float32), d_gpu, c.value, c.a_start, c.a_len,
                                  c.a_loc, c.bins, p, c.scales, dtype=dtype)
        np.testing.assert_allclose(y_gpu, y_ref, rtol=RTOL, atol=ATOL)


def test_odd_rank_and_rank_above_columns(gpu):
    """Ranks that are not a multiple of 8 take the element-wise path; an
    adapter whose rank exceeds the delta width uses only the columns there are."""
    c = make_case(12, 256, [4, 12, 8, 24], 30, dtype="f16")
    g = GpuCase(c, gpu)
    for p in (0, 3):
        for R in (24, 16):
            d_gpu, y_gpu = run_chain(c, g, p, R, gpu)
            d_ref, _ = oracle_chain(c, p, R)
            np.testing.assert_allclose(d_gpu, d_ref, rtol=RTOL, atol=ATOL)
            y_ref = O.ref_bgmv_expand(np.zeros((c.batch, 256), np.float32), d_gpu, c.value, c.a_start, c.a_len,
                                      c.a_loc, c.bins, p, c.scales, dtype="f16")
            np.testing.assert_allclose(y_gpu, y_ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("batch", [1, 7, 513, 1500])
def test_ragged_batches_and_popular_adapter(gpu, batch):
    """Batches that do not fill a workgroup group, batches longer than one
    scan chunk, and one adapter owning most tokens (long runs)."""
    bins = np.random.default_rng(batch).choice(4, size=batch, p=[0.85, 0.05, 0.05, 0.05])
    c = make_case(13 + batch, 512, [16, 8, 64, 32], batch, dtype="f16", bins=bins)
    g = GpuCase(c, gpu)
    d_gpu, y_gpu = run_chain(c, g, 0, 64, gpu)
    d_ref, _ = oracle_chain(c, 0, 64)
    np.testing.assert_allclose(d_gpu, d_ref, rtol=RTOL, atol=ATOL)
    y_ref = O.ref_bgmv_expand(np.zeros((batch, 512), np.float32), d_gpu, c.value, c.a_start, c.a_len, c.a_loc,
                              c.bins, 0, c.scales, dtype="f16")
    np.testing.assert_allclose(y_gpu, y_ref, rtol=RTOL, atol=ATOL)


def test_empty_batch_and_zero_rank(gpu):
    from slora_hip import dispatch_bgmv
    c = make_case(14, 256, [8, 0, 16], 12, dtype="f16", bins=np.array([0, 1, 2] * 4))
    g = GpuCase(c, gpu)
    d_gpu, y_gpu = run_chain(c, g, 0, 16, gpu)
    assert np.all(d_gpu[1::3] == 0) and np.all(y_gpu[1::3] == 0)  # rank-0 adapter: nothing happens
    d_ref, _ = oracle_chain(c, 0, 16)
    np.testing.assert_allclose(d_gpu, d_ref, rtol=RTOL, atol=ATOL)
    e = torch.zeros((0, 256), dtype=torch.float16, device=gpu)
    d = torch.zeros((0, 16), dtype=torch.float16, device=gpu)
    dispatch_bgmv(d, e, g.key, g.a_start, g.a_len, g.a_loc, g.bins[:0], 0, g.scales)
    dispatch_bgmv(e, d, g.value, g.a_start, g.a_len, g.a_loc, g.bins[:0], 0, g.scales)
    torch.cuda.synchronize()


def test_out_of_range_indices_are_skipped_not_faulted(gpu):
    """Adapter ids or page ids outside the tables: the token / row is skipped."""
    from slora_hip import dispatch_bgmv
    c = make_case(15, 256, [8, 16], 8, dtype="f16", bins=np.array([0, 1, 0, 1, 0, 1, 0, 1]))
    g = GpuCase(c, gpu)
    bad_bins = g.bins.clone()
    bad_bins[3] = 99
    bad_bins[4] = -1
    delta = torch.full((8, 16), 5.0, dtype=torch.float16, device=gpu)
    dispatch_bgmv(delta, g.x, g.key, g.a_start, g.a_len, g.a_loc, bad_bins, 0, g.scales)
    d = host(delta)
    assert np.all(d[3] == 5.0) and np.all(d[4] == 5.0)
    bad_loc = g.a_loc.clone()
    bad_loc[0] = c.n_pages + 5  # adapter 0, projection q, row 0
    delta.fill_(5.0)
    dispatch_bgmv(delta, g.x, g.key, g.a_start, g.a_len, bad_loc, g.bins, 0, g.scales)
    d = host(delta)
    assert np.all(d[0::2, 0] == 5.0)
    d_ref, _ = oracle_chain(c, 0, 16)
    np.testing.assert_allclose(d[0::2, 1:8], d_ref[0::2, 1:8], rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_fused_qkv_equals_three_calls(gpu, dtype):
    from slora_hip import dispatch_bgmv, dispatch_bgmv_qkv_shrink, dispatch_bgmv_qkv_expand
    c = make_case(16, 1024, [64, 8, 32, 16], 70, dtype=dtype, h_out=[1024, 256, 256, 1024], zipf_alpha=1.0)
    g = GpuCase(c, gpu)
    R = 64
    sep = [torch.zeros((c.batch, R), dtype=g.tdt, device=gpu) for _ in range(3)]
    fus = [torch.zeros((c.batch, R), dtype=g.tdt, device=gpu) for _ in range(3)]
    for p in range(3):
        dispatch_bgmv(sep[p], g.x, g.key, g.a_start, g.a_len, g.a_loc, g.bins, p, g.scales)
    dispatch_bgmv_qkv_shrink(fus[0], fus[1], fus[2], g.x, g.key, g.a_start, g.a_len, g.a_loc, g.bins)
    for p in range(3):
        assert torch.equal(sep[p], fus[p])
    y0 = [torch.randn((c.batch, c.h_out[p]), dtype=g.tdt, device=gpu) for p in range(3)]
    ys = [t.clone() for t in y0]
    yf = [t.clone() for t in y0]
    for p in range(3):
        dispatch_bgmv(ys[p], sep[p], g.value, g.a_start, g.a_len, g.a_loc, g.bins, p, g.scales)
    dispatch_bgmv_qkv_expand(yf[0], yf[1], yf[2], fus[0], fus[1], fus[2], g.value, g.a_start, g.a_len, g.a_loc,
                             g.bins, g.scales)
    for p in range(3):
        assert torch.equal(ys[p], yf[p])


def test_scaling_table_read_in_its_own_dtype(gpu):
    """bf16 activations with the fp16 scaling table the reference keeps
    (infer_adapter.py:33): the table must be read as fp16."""
    c = make_case(17, 256, [8, 16], 10, dtype="bf16")
    g = GpuCase(c, gpu)
    d_gpu, y_gpu = run_chain(c, g, 0, 16, gpu)
    y_ref = O.ref_bgmv_expand(np.zeros((10, 256), np.float32), d_gpu, c.value, c.a_start, c.a_len, c.a_loc, c.bins, 0,
                              c.scales, dtype="bf16")
    np.testing.assert_allclose(y_gpu, y_ref, rtol=RTOL, atol=ATOL)


def test_denormal_weights_are_not_flushed(gpu):
    """The reference's dummy adapters are U(-1e-3, 1e-3) (lora_layer_weight.py:41-56):
    a good part of such weights is subnormal in fp16 and must still count."""
    c = make_case(18, 1024, [8, 16], 16, dtype="f16")
    rng = np.random.default_rng(18)
    for i, r in enumerate(c.ranks):
        c.A[i] = [O.round_to(rng.uniform(-6e-5, 6e-5, (1024, r)).astype(np.float32), "f16") for _ in range(4)]
        loc = c.a_loc[c.a_start[i]: c.a_start[i] + 4 * r]
        O.load_into_pool(c.key, c.value, O.pack_w_combined(c.A[i], c.B[i], 1024), loc)
    c.x = O.round_to(np.abs(c.x) * 8, "f16")
    g = GpuCase(c, gpu)
    d_gpu, _ = run_chain(c, g, 0, 16, gpu)
    d_ref, _ = oracle_chain(c, 0, 16)
    np.testing.assert_allclose(d_gpu, d_ref, rtol=RTOL, atol=1e-5)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("hidden,ranks,batch,h_out,rank_cap", [
    (1024, [64, 8, 32, 16], 70, [1024, 256, 256, 1024], 64),
    (4096, [64, 32, 16, 8, 8, 16], 256, None, 64),
    (512, [16, 8, 64, 32], 1500, None, 64),
    (256, [4, 12, 8, 24], 30, None, 24),       # element-wise expand path
    (512, [64, 8, 128], 40, None, 32),          # ranks above rank_cap keep using a_loc
])
def test_planned_calls_equal_stateless_calls(gpu, dtype, hidden, ranks, batch, h_out, rank_cap):
    """A plan changes how a call finds its pages, never what it computes: the
    results must be bitwise those of the stateless calls (single and q/k/v-fused)."""
    import slora_hip
    from slora_hip import dispatch_bgmv, dispatch_bgmv_qkv_shrink, dispatch_bgmv_qkv_expand
    bins = None
    if batch == 1500:
        bins = np.random.default_rng(3).choice(4, size=batch, p=[0.85, 0.05, 0.05, 0.05])
    c = make_case(300 + hidden + batch, hidden, ranks, batch, dtype=dtype, h_out=h_out, zipf_alpha=1.0, bins=bins)
    g = GpuCase(c, gpu)
    R = max(ranks)
    t = (g.a_start, g.a_len, g.a_loc, g.bins)
    plan = slora_hip.make_plan(*t, rank_cap, c.n_pages)
    assert 0 < plan.n_runs <= batch and plan.n_items >= plan.n_runs
    assert plan.max_rank == max(ranks[i] for i in np.unique(c.bins))
    for readback in (plan, slora_hip.make_plan(*t, rank_cap, c.n_pages, readback=False)):
        d_s = [torch.zeros((batch, R), dtype=g.tdt, device=gpu) for _ in range(4)]
        d_p = [torch.zeros((batch, R), dtype=g.tdt, device=gpu) for _ in range(4)]
        for p in range(4):
            dispatch_bgmv(d_s[p], g.x, g.key, *t, p, g.scales, plan=False)
            dispatch_bgmv(d_p[p], g.x, g.key, *t, p, g.scales, plan=readback)
            assert torch.equal(d_s[p], d_p[p]), p
        y0 = [torch.randn((batch, c.h_out[p]), dtype=g.tdt, device=gpu) for p in range(4)]
        y_s = [v.clone() for v in y0]
        y_p = [v.clone() for v in y0]
        for p in range(4):
            dispatch_bgmv(y_s[p], d_s[p], g.value, *t, p, g.scales, plan=False)
            dispatch_bgmv(y_p[p], d_s[p], g.value, *t, p, g.scales, plan=readback)
            assert torch.equal(y_s[p], y_p[p]), p
        # fused q/k/v with a plan
        d_f = [torch.zeros((batch, R), dtype=g.tdt, device=gpu) for _ in range(3)]
        dispatch_bgmv_qkv_shrink(d_f[0], d_f[1], d_f[2], g.x, g.key, *t, plan=readback)
        y_f = [v.clone() for v in y0[:3]]
        dispatch_bgmv_qkv_expand(y_f[0], y_f[1], y_f[2], d_f[0], d_f[1], d_f[2], g.value, *t, g.scales, plan=readback)
        for p in range(3):
            assert torch.equal(d_f[p], d_s[p]) and torch.equal(y_f[p], y_s[p]), p


def test_automatic_plan_cache_follows_the_index_tensors(gpu, plan_cache_mode):
    """Calls without a plan reuse one built at the first call for the same index
    tensors; an in-place change of a tensor or a new tensor object rebuilds it,
    and the results always equal those of the plan-free kernels."""
    import slora_hip
    from slora_hip import dispatch_bgmv
    if plan_cache_mode != "cache":
        pytest.skip("cache switched off")
    c = make_case(77, 512, [16, 8, 32], 40, dtype="f16")
    g = GpuCase(c, gpu)
    slora_hip.plan_cache_stats(reset=True)

    def stats():
        s = slora_hip.plan_cache_stats()
        return s["builds"], s["hits"]

    def both(bins):
        t = (g.a_start, g.a_len, g.a_loc, bins)
        d0 = torch.zeros((c.batch, 32), dtype=g.tdt, device=gpu)
        d1 = torch.zeros_like(d0)
        dispatch_bgmv(d0, g.x, g.key, *t, 1, g.scales, plan=False)
        dispatch_bgmv(d1, g.x, g.key, *t, 1, g.scales)
        assert torch.equal(d0, d1)
        y0 = torch.zeros((c.batch, 512), dtype=g.tdt, device=gpu)
        y1 = torch.zeros_like(y0)
        dispatch_bgmv(y0, d0, g.value, *t, 1, g.scales, plan=False)
        dispatch_bgmv(y1, d0, g.value, *t, 1, g.scales)
        assert torch.equal(y0, y1)

    both(g.bins)
    assert stats() == (1, 1)                       # shrink built it, expand reused it
    both(g.bins)
    assert stats() == (1, 3)
    g.bins.copy_(torch.flip(g.bins, dims=[0]))     # new batch written in place: version changes
    both(g.bins)
    assert stats()[0] == 2
    both(g.bins.clone())                           # same contents in a new tensor object
    assert stats()[0] == 3
    torch.cuda.synchronize()
    with torch.cuda.stream(torch.cuda.Stream()):   # another stream never sees this stream's plan
        both(g.bins)
    assert stats()[0] == 4
    # a new tensor object that lands at the address (and version) of a freed one is another tensor
    slora_hip.clear_plan_cache()
    slora_hip.plan_cache_stats(reset=True)
    for k in range(3):
        b = torch.roll(g.bins, k).contiguous()
        both(b)
        del b
    assert stats()[0] == 3
    # a table rewritten through this library's own raw-pointer writers invalidates the plan
    from slora_hip.infer_adapter import launch_var_len_copy
    slora_hip.clear_plan_cache()
    slora_hip.plan_cache_stats(reset=True)
    loc = g.a_loc.clone()
    t2 = (g.a_start, g.a_len, loc, g.bins)
    d_a = torch.zeros((c.batch, 32), dtype=g.tdt, device=gpu)
    dispatch_bgmv(d_a, g.x, g.key, *t2, 1, g.scales)
    # move every adapter's page list to where another adapter's was: same tensor object, new contents
    new_loc = torch.flip(g.a_loc, dims=[0]).contiguous()
    launch_var_len_copy(torch.zeros(1, dtype=torch.int64, device=gpu),
                        torch.full((1,), loc.numel(), dtype=torch.int64, device=gpu), new_loc,
                        torch.zeros(1, dtype=torch.int64, device=gpu), loc)
    d_b = torch.zeros_like(d_a)
    dispatch_bgmv(d_b, g.x, g.key, *t2, 1, g.scales)
    d_c = torch.zeros_like(d_a)
    dispatch_bgmv(d_c, g.x, g.key, *t2, 1, g.scales, plan=False)
    assert torch.equal(d_b, d_c) and not torch.equal(d_a, d_b)
    assert stats()[0] == 2


@pytest.mark.parametrize("seed", range(12))
def test_random_configurations(gpu, seed):
    """Seeded random shapes: hidden and output widths that are any multiple of 8,
    ranks that are powers of two, other multiples of 8, or odd, batches from 1 to
    700, pages wider than the rows, either dtype.  Every way of calling (no plan,
    plan, q/k/v in one launch) against the oracle and against each other bit for bit."""
    import slora_hip
    from slora_hip import dispatch_bgmv, dispatch_bgmv_qkv_expand, dispatch_bgmv_qkv_shrink
    rng = np.random.default_rng(1000 + seed)
    hidden = int(rng.integers(1, 129)) * 8 * int(rng.choice([1, 1, 4]))
    n_ad = int(rng.integers(1, 7))
    ranks = [int(rng.choice([8, 16, 32, 64, 24, 40, 4, 12, 5, 128])) for _ in range(n_ad)]
    batch = int(rng.choice([1, 2, 5, 33, 64, 257, 700]))
    wide = int(rng.choice([1, 1, 2]))
    h_out = [int(rng.integers(1, 65)) * 8 * wide for _ in range(4)] if rng.random() < 0.5 else None
    if h_out is not None:
        h_out = [max(h, max(ranks) + 8) for h in h_out]
    hidden = max(hidden, max(ranks) + 8)          # shrink means delta narrower than x
    page_elems = max([hidden] + (h_out or [])) * int(rng.choice([1, 1, 2]))
    dtype = str(rng.choice(["f16", "bf16"]))
    c = make_case(2000 + seed, hidden, ranks, batch, dtype=dtype, h_out=h_out, page_elems=page_elems,
                  zipf_alpha=float(rng.choice([0.0, 1.0, 2.0])))
    g = GpuCase(c, gpu, heads=1)
    R = (max(ranks) + 7) // 8 * 8
    t = (g.a_start, g.a_len, g.a_loc, g.bins)
    plan = slora_hip.make_plan(*t, R, c.n_pages)
    y0 = [torch.randn((batch, c.h_out[p]), dtype=g.tdt, device=gpu) for p in range(4)]
    d_s, y_s = [], []
    for p in range(4):
        d = torch.zeros((batch, R), dtype=g.tdt, device=gpu)
        dispatch_bgmv(d, g.x, g.key, *t, p, g.scales, plan=False)
        y = y0[p].clone()
        dispatch_bgmv(y, d, g.value, *t, p, g.scales, plan=False)
        d_ref, _ = oracle_chain(c, p, R)
        np.testing.assert_allclose(host(d), d_ref, rtol=RTOL, atol=ATOL)
        # against the oracle from a zero start (a random start adds a rounding of the sum to
        # the storage type that cancellation can turn into more than 1 % of the result)
        yz = torch.zeros_like(y)
        dispatch_bgmv(yz, d, g.value, *t, p, g.scales, plan=False)
        y_ref = O.ref_bgmv_expand(np.zeros((batch, c.h_out[p]), np.float32), host(d), c.value, c.a_start, c.a_len,
                                  c.a_loc, c.bins, p, c.scales, dtype=c.dtype)
        np.testing.assert_allclose(host(yz), y_ref, rtol=RTOL, atol=ATOL)
        d_s.append(d)
        y_s.append(y)
        d_p = torch.zeros_like(d)
        dispatch_bgmv(d_p, g.x, g.key, *t, p, g.scales, plan=plan)
        y_p = y0[p].clone()
        dispatch_bgmv(y_p, d_p, g.value, *t, p, g.scales, plan=plan)
        assert torch.equal(d_p, d) and torch.equal(y_p, y), ("planned", p)
    for planned in (None, plan):
        kw = {"plan": planned} if planned is not None else {"plan": False}
        d_f = [torch.zeros((batch, R), dtype=g.tdt, device=gpu) for _ in range(3)]
        y_f = [y0[p].clone() for p in range(3)]
        dispatch_bgmv_qkv_shrink(d_f[0], d_f[1], d_f[2], g.x, g.key, *t, **kw)
        dispatch_bgmv_qkv_expand(y_f[0], y_f[1], y_f[2], d_f[0], d_f[1], d_f[2], g.value, *t, g.scales, **kw)
        for p in range(3):
            assert torch.equal(d_f[p], d_s[p]) and torch.equal(y_f[p], y_s[p]), ("q/k/v", planned is not None, p)


def test_full_size_s2_properties(gpu, plan_cache_mode):
    """The benchmark's own configuration (hidden 4096, 200 adapters of ranks
    {64,32,16,8}, Zipf(1) batch of 256, 65536-page pool), one layer, checked through
    properties that do not need the CPU oracle at this size:
    * against torch float32 on the same device from the adapters' unpacked A, B
      (dense closed form, rtol 1e-2 / atol 1e-3 on the final y with the kernel's
      own fp16 delta as input of the second product);
    * doubling every scale doubles y exactly (power of two, zero start) wherever
      y is a normal fp16 number;
    * permuting the tokens permutes the results bit for bit (other runs, other
      workgroups, same sums);
    * garbage in delta columns beyond an adapter's rank changes nothing."""
    import workloads
    from slora_hip import dispatch_bgmv
    w = workloads.s2_decode(gpu, n_layers=1)
    B, H, R = w.batch, w.hidden, w.max_rank
    t = (w.a_start, w.a_len, w.a_loc, w.req_bins)
    g = torch.Generator(device=gpu)
    g.manual_seed(5)
    x = torch.randn((B, H), generator=g, device=gpu).to(w.dtype)
    key, val = w.key_buffer[0], w.value_buffer[0]
    perm = torch.randperm(B, generator=g, device=gpu)
    t_perm = (w.a_start, w.a_len, w.a_loc, w.req_bins[perm].contiguous())
    ranks_t = torch.from_numpy(w.ranks[w.bins_np]).to(gpu)
    for p in range(4):
        d = torch.zeros((B, R), dtype=w.dtype, device=gpu)
        dispatch_bgmv(d, x, key, *t, p, w.a_scaling)
        y = torch.zeros((B, H), dtype=w.dtype, device=gpu)
        dispatch_bgmv(y, d, val, *t, p, w.a_scaling)
        # dense float32 closed form per adapter in the batch
        d_ref = torch.zeros((B, R), dtype=torch.float32, device=gpu)
        y_ref = torch.zeros((B, H), dtype=torch.float32, device=gpu)
        for a in np.unique(w.bins_np):
            r = int(w.ranks[a])
            loc = w.a_loc[int(w.a_start_np[a]) + p * r: int(w.a_start_np[a]) + (p + 1) * r]
            rows = torch.from_numpy(np.nonzero(w.bins_np == a)[0]).to(gpu)
            A = key[loc].reshape(r, H).float()                      # [r, H] = A^T
            Bt = val[loc].reshape(H, r).float()                     # [H, r] = B^T
            d_ref[rows, :r] = x[rows].float() @ A.t()
            y_ref[rows] = (d[rows, :r].float() @ Bt.t()) * float(w.scales_np[a])
        np.testing.assert_allclose(d.float().cpu().numpy(), d_ref.cpu().numpy(), rtol=RTOL, atol=ATOL)
        np.testing.assert_allclose(y.float().cpu().numpy(), y_ref.cpu().numpy(), rtol=RTOL, atol=ATOL)
        # scale x 2  ->  y x 2, exactly
        y2 = torch.zeros_like(y)
        dispatch_bgmv(y2, d, val, *t, p, (w.a_scaling * 2).contiguous())
        normal = y.abs() >= 2.0 ** -13   # below, fp16 is subnormal and rounding does not commute with doubling
        assert torch.equal(y2[normal], (y * 2)[normal])
        assert (y2[~normal].float() - 2 * y[~normal].float()).abs().max() <= 2.0 ** -23
        # token permutation
        dp = torch.zeros_like(d)
        dispatch_bgmv(dp, x[perm].contiguous(), key, *t_perm, p, w.a_scaling)
        assert torch.equal(dp, d[perm])
        yp = torch.zeros_like(y)
        dispatch_bgmv(yp, dp, val, *t_perm, p, w.a_scaling)
        assert torch.equal(yp, y[perm])
        # columns beyond the rank do not matter
        dg = d.clone()
        cols = torch.arange(R, device=gpu)[None, :] >= ranks_t[:, None]
        dg[cols] = 77.0
        yg = torch.zeros_like(y)
        dispatch_bgmv(yg, dg, val, *t, p, w.a_scaling)
        assert torch.equal(yg, y)


def test_plan_is_rejected_for_another_batch_size(gpu):
    import slora_hip
    c = make_case(19, 256, [8, 16], 12, dtype="f16")
    g = GpuCase(c, gpu)
    plan = slora_hip.make_plan(g.a_start, g.a_len, g.a_loc, g.bins, 16, c.n_pages)
    d = torch.zeros((6, 16), dtype=torch.float16, device=gpu)
    with pytest.raises(RuntimeError, match="plan was built for"):
        slora_hip.dispatch_bgmv(d, g.x[:6], g.key, g.a_start, g.a_len, g.a_loc, g.bins[:6], 0, g.scales, plan=plan)


def test_golden_fixture_decode_and_prefill(gpu):
    """The committed closed-form fixture (tests/golden/lora_small.npz) through
    both operator families."""
    from test_oracle import load_golden
    from slora_hip import dispatch_bgmv, lora_get_qkvo_fwd_shrink, lora_get_qkvo_fwd_expand
    g = load_golden()
    f16 = torch.float16
    key = torch.from_numpy(g["key"]).to(gpu)
    value = torch.from_numpy(g["value"]).to(gpu)
    n_pages = key.shape[0]
    a_start, a_len, a_loc, bins = (torch.from_numpy(g[k]).to(gpu) for k in ("a_start", "a_len", "a_loc", "bins"))
    st, ln, rq = (torch.from_numpy(g[k]).to(gpu) for k in ("b_start_loc", "b_seq_len", "b_indicies"))
    scales = torch.from_numpy(g["scales"]).to(gpu)
    x = torch.from_numpy(g["x"]).to(gpu)
    T = x.shape[0]
    for p in range(4):
        d = torch.zeros((T, 32), dtype=f16, device=gpu)
        dispatch_bgmv(d, x, key.view(n_pages, 4, 32), a_start, a_len, a_loc, bins, p, scales)
        np.testing.assert_allclose(host(d), g["delta64"][p], rtol=2e-3, atol=2e-3)
        y = torch.from_numpy(g["y0"][p]).to(gpu)
        dispatch_bgmv(y, d, value.view(n_pages, 4, 32), a_start, a_len, a_loc, bins, p, scales)
        np.testing.assert_allclose(host(y), g["y64"][p], rtol=1e-2, atol=1e-2)
        o = torch.ones((T, 32), dtype=f16, device=gpu)
        lora_get_qkvo_fwd_shrink(x, key, o, a_loc, a_start, a_len, st, ln, rq, 128, p, 32, int(g["b_seq_len"].max()))
        np.testing.assert_allclose(host(o), g["delta64"][p], rtol=2e-3, atol=2e-3)
        y2 = torch.from_numpy(g["y0"][p]).to(gpu)
        lora_get_qkvo_fwd_expand(o, value, y2, scales, a_loc, a_start, a_len, st, ln, rq, 128, p, 32,
                                 int(g["b_seq_len"].max()))
        np.testing.assert_allclose(host(y2), g["y64"][p], rtol=1e-2, atol=1e-2)
