"""Pins the CPU oracle (oracle/lora_oracle.py) without a GPU.

The reference stores no golden vectors for this path; its executable specs are
the two closed-form loops of test/kernel/test_kernel_correctness.py:87-95 and
test_kernel_correctness_multi_rank.py:97-106, restated here verbatim in numpy.
Everything else is pinned by mathematics: the pool layout by its inverse taken
from a different reference file, the paged index arithmetic by the dense closed
form in float64 and by integer-exact cases, the rounding helpers by torch's own
conversions.
"""
import numpy as np
import pytest
import torch

from oracle import lora_oracle as O
from lora_cases import make_case, make_segments


# ---------------------------------------------------------------------------
# rounding helpers against an independent library routine
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,tdt", [("f16", torch.float16), ("bf16", torch.bfloat16)])
def test_round_to_matches_torch(dtype, tdt):
    rng = np.random.default_rng(0)
    a = np.concatenate([
        rng.standard_normal(4096).astype(np.float32) * 10.0 ** rng.integers(-8, 5, 4096),
        np.array([0.0, -0.0, 1.0, 65504.0, 65519.9, 6e-8, 5.96e-8, 2.98e-8, 1e-40, 3.3895e38], dtype=np.float32),
        # exact ties
        np.array([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8], dtype=np.float32),
    ])
    want = torch.from_numpy(a).to(tdt).to(torch.float32).numpy()
    got = O.round_to(a, dtype)
    finite = np.isfinite(want)
    assert np.array_equal(got[finite], want[finite])
    assert np.array_equal(np.isinf(got), np.isinf(want))


# ---------------------------------------------------------------------------
# pool layout
# ---------------------------------------------------------------------------
def test_pack_layout_elementwise():
    """w_combined element by element: [0, p*r+j, k] = A_p[k, j];
    flat element n*r+d of [1, p*r:(p+1)*r] = B_p[d, n]."""
    rng = np.random.default_rng(1)
    H, r = 16, 8
    A = [rng.integers(-50, 50, (H, r)).astype(np.float32) for _ in range(4)]
    B = [rng.integers(-50, 50, (r, H)).astype(np.float32) for _ in range(4)]
    wc = O.pack_w_combined(A, B, H)
    assert wc.shape == (2, 4 * r, H)
    for p in range(4):
        for j in range(r):
            for k in range(H):
                assert wc[0, p * r + j, k] == A[p][k, j]
        flat = wc[1, p * r:(p + 1) * r].reshape(-1)
        for n in range(H):
            for d in range(r):
                assert flat[n * r + d] == B[p][d, n]


def test_pack_matches_torch_view_semantics():
    """The packer is written in the reference with torch views:
    ``A.T.reshape(rank, heads, -1)`` and ``B.T.reshape(rank, heads, -1)`` on
    transposed-contiguous tensors (lora_layer_weight.py:84-93).  Replay those
    torch expressions literally and compare."""
    g = torch.Generator().manual_seed(2)
    H, r, heads = 32, 8, 4
    mats = {}
    for name in "qkvo":
        # load_dummy_weights: rand((rank, H)).transpose(0,1).contiguous() -> (H, r); rand((H, rank)).T.contiguous() -> (r, H)
        mats[name + "A"] = torch.rand((r, H), generator=g).transpose(0, 1).contiguous()
        mats[name + "B"] = torch.rand((H, r), generator=g).transpose(0, 1).contiguous()
    combined = torch.concat([mats[n + "A"].T.reshape(r, heads, -1) for n in "qkvo"] +
                            [mats[n + "B"].T.reshape(r, heads, -1) for n in "qkvo"]).reshape(2, 4 * r, heads, -1)
    wc = O.pack_w_combined([mats[n + "A"].numpy() for n in "qkvo"], [mats[n + "B"].numpy() for n in "qkvo"], H)
    assert np.array_equal(combined.reshape(2, 4 * r, H).numpy(), wc)


@pytest.mark.parametrize("ranks", [[8], [8, 16, 64, 32], [16, 16, 8]])
def test_pack_load_unpack_roundtrip(ranks):
    """pack (lora_layer_weight.py) -> load (infer_adapter.py) -> unpack
    (lora_single_batch_infer.py) is the identity on scattered pages."""
    c = make_case(3, 64, ranks, batch=4)
    for i, r in enumerate(ranks):
        loc = c.a_loc[c.a_start[i]: c.a_start[i] + c.a_len[i]]
        A, B = O.unpack_from_pool(c.key, c.value, loc, c.hidden, c.h_out)
        for p in range(4):
            assert np.array_equal(A[p], c.A[i][p])
            assert np.array_equal(B[p], c.B[i][p])


def test_build_tables():
    a_start, a_len, a_loc = O.build_tables([8, 16, 8], np.arange(100, 228))
    assert a_len.tolist() == [32, 64, 32]
    assert a_start.tolist() == [0, 32, 96]
    assert a_loc.tolist() == list(range(100, 228))
    assert a_start.dtype == a_len.dtype == a_loc.dtype == np.int64


def test_gqa_pack_narrow_output():
    """k/v narrower than a page: B^T fills the first r*h_kv/page_elems pages of the slot."""
    c = make_case(4, 64, [16], batch=2, h_out=[64, 16, 16, 64])
    loc = c.a_loc[:64]
    A, B = O.unpack_from_pool(c.key, c.value, loc, 64, c.h_out)
    for p in range(4):
        assert np.array_equal(B[p], c.B[0][p])
        assert B[p].shape == (16, c.h_out[p])


# ---------------------------------------------------------------------------
# the reference's own executable specs
# ---------------------------------------------------------------------------
def _reference_test_setup(rng, H, R, N):
    """Fixture of test/kernel/test_kernel_correctness*.py: adapters stored back
    to back, identity a_loc, scaling 1, tokens split evenly over adapters."""
    n_ad = len(R)
    key_buffer = O.round_to(rng.standard_normal((sum(R) * 4, H)).astype(np.float32), "f16")
    a_len = np.array([r * 4 for r in R], dtype=np.int64)
    a_start = np.zeros_like(a_len)
    a_start[1:] = np.cumsum(a_len[:-1])
    a_loc = np.arange(sum(R) * 4, dtype=np.int64)
    a_scaling = np.ones(n_ad, dtype=np.float32)
    per = (N + n_ad - 1) // n_ad
    bins = np.concatenate([np.full(per, i, dtype=np.int64) for i in range(n_ad)])[:N]
    return key_buffer, a_start, a_len, a_loc, a_scaling, bins


@pytest.mark.parametrize("R,H,qkvo", [([128, 128], 4096, 1), ([8, 16], 1024, 0), ([8, 16], 1024, 3)])
def test_expand_against_reference_test_loop(R, H, qkvo):
    """part == "B" of test_kernel_correctness.py:87-95 / _multi_rank.py:97-106:
    ``a_w = key_buffer[a_start + qkvo*R : a_start + (qkvo+1)*R].reshape(H, R).T``
    and ``ref = x[i:i+1, :R] @ a_w``."""
    rng = np.random.default_rng(42)
    N, max_r = 32, max(R)
    key_buffer, a_start, a_len, a_loc, a_scaling, bins = _reference_test_setup(rng, H, R, N)
    x = O.round_to(rng.standard_normal((N, max_r)).astype(np.float32), "f16")
    results = []
    for i in range(N):
        a = bins[i]
        a_w = key_buffer[a_start[a] + qkvo * R[a]: a_start[a] + (qkvo + 1) * R[a]]
        a_w = a_w.reshape(H, R[a]).T
        results.append(x[i:i + 1, :R[a]].astype(np.float64) @ a_w.astype(np.float64))
    ref = np.concatenate(results)
    got = O.ref_bgmv_expand(np.zeros((N, H), np.float32), x, key_buffer, a_start, a_len, a_loc, bins, qkvo,
                            a_scaling, dtype="f32")
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("R,H,qkvo", [([128, 128], 4096, 1), ([8, 16], 1024, 2)])
def test_shrink_against_reference_test_loop(R, H, qkvo):
    """part == "A" of the same scripts: ``a_w.reshape(R, H).T``; ``x[i] @ a_w``."""
    rng = np.random.default_rng(43)
    N, max_r = 32, max(R)
    key_buffer, a_start, a_len, a_loc, a_scaling, bins = _reference_test_setup(rng, H, R, N)
    x = O.round_to(rng.standard_normal((N, H)).astype(np.float32), "f16")
    got = O.ref_bgmv_shrink(np.zeros((N, max_r), np.float32), x, key_buffer, a_start, a_len, a_loc, bins, qkvo,
                            dtype="f32")
    for i in range(N):
        a = bins[i]
        a_w = key_buffer[a_start[a] + qkvo * R[a]: a_start[a] + (qkvo + 1) * R[a]].reshape(R[a], H).T
        ref = x[i:i + 1].astype(np.float64) @ a_w.astype(np.float64)
        np.testing.assert_allclose(got[i, :R[a]], ref[0], rtol=1e-5, atol=1e-4)
        assert np.all(got[i, R[a]:] == 0.0)  # untouched (the kernel returns early for j >= r)


# ---------------------------------------------------------------------------
# paged semantics against the dense closed form
# ---------------------------------------------------------------------------
def _paged_chain(c, p, dtype, y0=None, max_rank=None):
    R = max_rank or c.max_rank
    delta = O.ref_bgmv_shrink(np.zeros((c.batch, R), np.float32), c.x, c.key, c.a_start, c.a_len, c.a_loc, c.bins,
                              p, dtype=dtype)
    y0 = np.zeros((c.batch, c.h_out[p]), np.float32) if y0 is None else y0
    return O.ref_bgmv_expand(y0, delta, c.value, c.a_start, c.a_len, c.a_loc, c.bins, p, c.scales, dtype=dtype), delta


@pytest.mark.parametrize("seed,ranks", [(10, [8, 16, 32, 64]), (11, [8, 8]), (12, [24, 40, 8])])
def test_paged_chain_equals_dense_f64(seed, ranks):
    c = make_case(seed, 128, ranks, batch=24, dtype="f32")
    for p in range(4):
        y0 = np.random.default_rng(seed + p).standard_normal((c.batch, 128)).astype(np.float32)
        got, _ = _paged_chain(c, p, "f32", y0=y0)
        want = O.dense_lora_f64(y0, c.x, [a[p] for a in c.A], [b[p] for b in c.B], c.scales, c.bins)
        np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-5)


def test_bmm_equals_dense_f64_and_paged():
    c = make_case(20, 128, [8, 16, 32], batch=20, dtype="f32")
    for p in range(4):
        y0 = np.zeros((c.batch, 128), np.float32)
        bmm = O.ref_bmm(y0, c.x, [a[p] for a in c.A], [b[p] for b in c.B], c.scales, c.bins, dtype="f32")
        want = O.dense_lora_f64(y0, c.x, [a[p] for a in c.A], [b[p] for b in c.B], c.scales, c.bins)
        paged, _ = _paged_chain(c, p, "f32")
        np.testing.assert_allclose(bmm, want, rtol=2e-5, atol=2e-5)
        np.testing.assert_allclose(bmm, paged, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_16bit_paths_within_stated_tolerance_of_bmm(dtype):
    """The stated tolerance (rtol 1e-2, atol 1e-3... scaled by the bf16 epsilon
    for bf16, see the GPU tests) between the paged and the bmm rounding chains."""
    c = make_case(21, 256, [8, 16, 64], batch=16, dtype=dtype)
    p = 0
    paged, _ = _paged_chain(c, p, dtype)
    bmm = O.ref_bmm(np.zeros((c.batch, 256), np.float32), c.x, [a[p] for a in c.A], [b[p] for b in c.B], c.scales,
                    c.bins, dtype=dtype)
    atol = 1e-3 if dtype == "f16" else 8e-3
    rtol = 1e-2 if dtype == "f16" else 3e-2
    np.testing.assert_allclose(paged, bmm, rtol=rtol, atol=atol * np.abs(bmm).max())


def test_integer_exact_gather():
    """Small-integer weights and one-hot / small-integer activations: every
    value is exact in fp16, so a wrong page, a wrong r*qkvo offset or a wrong
    n*r+d split changes the result.  Dense integer matmul is the truth."""
    rng = np.random.default_rng(30)
    H, ranks = 32, [8, 16, 8]
    c = make_case(30, H, ranks, batch=12, dtype="f16")
    # overwrite with integers
    for i, r in enumerate(ranks):
        c.A[i] = [rng.integers(-3, 4, (H, r)).astype(np.float32) for _ in range(4)]
        c.B[i] = [rng.integers(-3, 4, (r, H)).astype(np.float32) for _ in range(4)]
        loc = c.a_loc[c.a_start[i]: c.a_start[i] + 4 * r]
        O.load_into_pool(c.key, c.value, O.pack_w_combined(c.A[i], c.B[i], H), loc)
    c.x = rng.integers(-2, 3, (c.batch, H)).astype(np.float32)
    c.scales = np.array([1.0, 2.0, 0.5], dtype=np.float32)
    for p in range(4):
        got, delta = _paged_chain(c, p, "f16")
        for t in range(c.batch):
            a = c.bins[t]
            d = c.x[t] @ c.A[a][p]
            assert np.array_equal(delta[t, : ranks[a]], d)
            assert np.array_equal(got[t], (d @ c.B[a][p]) * c.scales[a])


def test_special_cases():
    c = make_case(40, 64, [8, 16], batch=10, dtype="f32")
    p = 2
    y0 = np.random.default_rng(1).standard_normal((c.batch, 64)).astype(np.float32)
    base, delta = _paged_chain(c, p, "f32", y0=y0)
    # scale = 0 leaves y unchanged
    zero = O.ref_bgmv_expand(y0, delta, c.value, c.a_start, c.a_len, c.a_loc, c.bins, p, np.zeros(2, np.float32), "f32")
    assert np.array_equal(zero, y0)
    # linear in scale
    dbl = O.ref_bgmv_expand(y0, delta, c.value, c.a_start, c.a_len, c.a_loc, c.bins, p, 2 * c.scales, "f32")
    np.testing.assert_allclose(dbl - y0, 2 * (base - y0), rtol=1e-5, atol=1e-6)
    # garbage in delta[:, r:] does not matter (bgmv_impl.cuh:186-188)
    junk = delta.copy()
    for t in range(c.batch):
        junk[t, c.ranks[c.bins[t]]:] = 1e4
    again = O.ref_bgmv_expand(y0, junk, c.value, c.a_start, c.a_len, c.a_loc, c.bins, p, c.scales, "f32")
    assert np.array_equal(again, base)
    # token permutation equivariance
    perm = np.random.default_rng(2).permutation(c.batch)
    d2 = O.ref_bgmv_shrink(np.zeros_like(delta), c.x[perm], c.key, c.a_start, c.a_len, c.a_loc, c.bins[perm], p, "f32")
    assert np.array_equal(d2, delta[perm])
    # single adapter, identity pages: plain x @ A @ B
    s = make_case(41, 32, [8], batch=5, dtype="f32", scatter=False)
    out, _ = _paged_chain(s, 0, "f32")
    want = s.scales[0] * (s.x.astype(np.float64) @ s.A[0][0].astype(np.float64)) @ s.B[0][0].astype(np.float64)
    np.testing.assert_allclose(out, want, rtol=2e-5, atol=2e-6)


def test_prefill_equals_decode_on_repeated_bins():
    """The reference itself falls back from the segmented kernels to BGMV with
    ``repeat_interleave(req_bins, b_seq_len)`` (lora_unordered_batch_infer.py:66,
    349-355): same numbers, except that the segmented shrink writes zeros in
    columns r..max_rank."""
    ranks = [8, 16, 32]
    start, lens, ids = make_segments(50, 6, 1, 9, len(ranks))
    T = int(lens.sum())
    c = make_case(50, 64, ranks, batch=T, dtype="f16", bins=np.repeat(ids, lens))
    R = 32
    for p in range(4):
        o0 = np.full((T, R), 7.0, np.float32)
        sh = O.ref_prefill_shrink(o0, c.x, c.key, c.a_loc, c.a_start, c.a_len, start, lens, ids, p, R, "f16")
        dec = O.ref_bgmv_shrink(np.zeros((T, R), np.float32), c.x, c.key, c.a_start, c.a_len, c.a_loc, c.bins, p, "f16")
        assert np.array_equal(sh, dec)  # zeros beyond r in both (decode started from zeros)
        y0 = np.random.default_rng(p).standard_normal((T, 64)).astype(np.float32)
        y0 = O.round_to(y0, "f16")
        ex = O.ref_prefill_expand(y0, sh, c.value, c.scales, c.a_loc, c.a_start, c.a_len, start, lens, ids, p, R, "f16")
        dex = O.ref_bgmv_expand(y0, dec, c.value, c.a_start, c.a_len, c.a_loc, c.bins, p, c.scales, "f16")
        # rounding points differ (scale inside vs after the sum; T add vs float add)
        np.testing.assert_allclose(ex, dex, rtol=1e-2, atol=1e-3 * max(1.0, np.abs(dex).max()))


def test_prefill_leaves_unowned_rows_alone():
    ranks = [8]
    c = make_case(51, 32, ranks, batch=10, dtype="f32", bins=np.zeros(10, np.int64))
    start = np.array([2, 7], np.int32)
    lens = np.array([3, 0], np.int32)
    ids = np.array([0, 0], np.int64)
    o = O.ref_prefill_shrink(np.full((10, 8), 5.0, np.float32), c.x, c.key, c.a_loc, c.a_start, c.a_len, start, lens,
                             ids, 0, 8, "f32")
    assert np.all(o[:2] == 5.0) and np.all(o[5:] == 5.0) and not np.any(o[2:5] == 5.0)


def test_var_len_copy():
    old_loc = np.arange(1000, 1300, dtype=np.int64)
    old_start = np.array([0, 32, 96], np.int64)
    lens = np.array([32, 64, 204], np.int64)
    keep = [0, 2]
    new_len = lens[keep]
    new_start = np.array([0, 32], np.int64)
    out = O.ref_var_len_copy(old_start[keep], new_len, old_loc, new_start, int(new_len.sum()))
    assert out.tolist() == list(range(1000, 1032)) + list(range(1096, 1300))


def test_offload_tables_explicit_and_invariants():
    """Hand-written expected tables for a 4-adapter case, then on random cases the
    properties that fix the result: kept adapters keep order, lengths, scaling and
    their exact page lists; starts are the running sum; kept + removed pages are
    the old pages, each exactly once."""
    a_len = np.array([8, 4, 12, 4], np.int64)
    a_start = np.array([0, 8, 12, 24], np.int64)
    a_loc = np.arange(100, 128, dtype=np.int64)[::-1].copy()   # 127 .. 100
    scal = np.array([2.0, 4.0, 1.0, 8.0], np.float32)
    ns, nl, nloc, nsc, rem = O.ref_offload_tables(a_start, a_len, a_loc, scal, [True, False, True, False])
    assert ns.tolist() == [0, 8] and nl.tolist() == [8, 12] and nsc.tolist() == [2.0, 1.0]
    assert nloc.tolist() == list(range(127, 119, -1)) + list(range(115, 103, -1))
    assert rem.tolist() == list(range(119, 115, -1)) + list(range(103, 99, -1))
    # nothing kept / everything kept
    ns, nl, nloc, nsc, rem = O.ref_offload_tables(a_start, a_len, a_loc, scal, [False] * 4)
    assert ns.size == nl.size == nloc.size == nsc.size == 0 and rem.tolist() == a_loc.tolist()
    ns, nl, nloc, nsc, rem = O.ref_offload_tables(a_start, a_len, a_loc, scal, [True] * 4)
    assert ns.tolist() == a_start.tolist() and nloc.tolist() == a_loc.tolist() and rem.size == 0
    rng = np.random.default_rng(5)
    for _ in range(20):
        n = int(rng.integers(1, 40))
        ranks = rng.choice([2, 8, 16, 64, 70], size=n)
        a_start, a_len, a_loc = O.build_tables(ranks, rng.permutation(100000)[: int(4 * ranks.sum())])
        scal = rng.standard_normal(n).astype(np.float32)
        keep = rng.random(n) < 0.6
        ns, nl, nloc, nsc, rem = O.ref_offload_tables(a_start, a_len, a_loc, scal, keep)
        left = np.nonzero(keep)[0]
        assert nl.tolist() == a_len[left].tolist() and nsc.tolist() == scal[left].tolist()
        assert ns.tolist() == (np.cumsum(nl) - nl).tolist()
        for k, i in enumerate(left):
            assert nloc[ns[k]: ns[k] + nl[k]].tolist() == a_loc[a_start[i]: a_start[i] + a_len[i]].tolist()
        assert sorted(np.concatenate([nloc, rem]).tolist()) == sorted(a_loc.tolist())


def test_merge_adapter_closed_form_and_round_trip():
    """ref_merge_adapter against the dense closed form in float64 (one rounding
    chain apart), exactly on integer-valued cases, and merge followed by unmerge
    gives W back exactly where every intermediate is exactly representable."""
    rng = np.random.default_rng(4)
    H, Ho, r = 48, 40, 8
    W = O.round_to(rng.standard_normal((H, Ho)).astype(np.float32), "f16")
    A = O.round_to(rng.standard_normal((H, r)).astype(np.float32) / 8, "f16")
    B = O.round_to(rng.standard_normal((r, Ho)).astype(np.float32) / 4, "f16")
    got = O.ref_merge_adapter(W, A, B, 2.0, 1.0, "f16")
    exact = W.astype(np.float64) + 2.0 * A.astype(np.float64) @ B.astype(np.float64)
    np.testing.assert_allclose(got, exact, rtol=2e-3, atol=2e-3)
    Wi = rng.integers(-8, 9, size=(H, Ho)).astype(np.float32)
    Ai = rng.integers(-2, 3, size=(H, r)).astype(np.float32)
    Bi = rng.integers(-2, 3, size=(r, Ho)).astype(np.float32)
    m = O.ref_merge_adapter(Wi, Ai, Bi, 2.0, 1.0, "f16")
    assert np.array_equal(m, Wi + 2.0 * Ai @ Bi)
    assert np.array_equal(O.ref_merge_adapter(m, Ai, Bi, 2.0, -1.0, "f16"), Wi)
    assert np.array_equal(O.ref_merge_adapter(Wi, Ai, Bi, 0.0, 1.0, "bf16"), Wi)


def test_allocator_against_brute_force():
    """ref_alloc / ref_alloc_contiguous / ref_free against the plain definitions:
    the first n free pages in index order; the smallest s with pages s..s+n-1 all
    free (tried one start at a time)."""
    rng = np.random.default_rng(9)
    for _ in range(200):
        tot = int(rng.integers(1, 60))
        state = (rng.random(tot) < rng.random()).astype(np.uint8)
        need = int(rng.integers(0, tot + 2))
        free = [i for i in range(tot) if state[i]]
        s1 = state.copy()
        got = O.ref_alloc(s1, need)
        assert got.tolist() == free[:need]
        exp = state.copy()
        exp[free[:need]] = 0
        assert np.array_equal(s1, exp)
        if need >= 1:
            s2 = state.copy()
            res = O.ref_alloc_contiguous(s2, need)
            starts = [s for s in range(0, tot - need + 1) if all(state[s + k] for k in range(need))]
            if not starts:
                assert res is None and np.array_equal(s2, state)
            else:
                sel, a, b = res
                assert (a, b) == (starts[0], starts[0] + need) and sel.tolist() == list(range(a, b))
                assert s2[a:b].sum() == 0 and np.array_equal(np.delete(s2, np.arange(a, b)), np.delete(state, np.arange(a, b)))
        s3 = s1.copy()
        O.ref_free(s3, got)
        assert np.array_equal(s3, state)


# ---------------------------------------------------------------------------
# committed fixture (closed form in float64 on the dense matrices) and CPU baseline
# ---------------------------------------------------------------------------
def load_golden():
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "lora_small.npz"))
    return {k: g[k] for k in g.files}


def test_oracle_matches_golden_fixture():
    g = load_golden()
    key, value, x = (g[k].astype(np.float32) for k in ("key", "value", "x"))
    scales = g["scales"].astype(np.float32)
    T = x.shape[0]
    for p in range(4):
        d = O.ref_bgmv_shrink(np.zeros((T, 32), np.float32), x, key, g["a_start"], g["a_len"], g["a_loc"], g["bins"], p,
                              "f16")
        np.testing.assert_allclose(d, g["delta64"][p], rtol=2e-3, atol=2e-3)
        y = O.ref_bgmv_expand(g["y0"][p].astype(np.float32), d, value, g["a_start"], g["a_len"], g["a_loc"], g["bins"],
                              p, scales, "f16")
        np.testing.assert_allclose(y, g["y64"][p], rtol=1e-2, atol=1e-2)
        o = O.ref_prefill_shrink(np.ones((T, 32), np.float32), x, key, g["a_loc"], g["a_start"], g["a_len"],
                                 g["b_start_loc"], g["b_seq_len"], g["b_indicies"], p, 32, "f16")
        np.testing.assert_allclose(o, g["delta64"][p], rtol=2e-3, atol=2e-3)
        y2 = O.ref_prefill_expand(g["y0"][p].astype(np.float32), o, value, scales, g["a_loc"], g["a_start"], g["a_len"],
                                  g["b_start_loc"], g["b_seq_len"], g["b_indicies"], p, 32, "f16")
        np.testing.assert_allclose(y2, g["y64"][p], rtol=1e-2, atol=1e-2)


def test_cpu_baseline_layer_matches_ref_bmm():
    c = make_case(60, 128, [8, 16, 32], batch=22, dtype="f32")
    layer = O.BmmCpuLayer(c.A, c.B, c.scales, c.bins, threads=2)
    rng = np.random.default_rng(61)
    x_att = rng.standard_normal((22, 128)).astype(np.float32)
    ys = [torch.zeros((22, 128)) for _ in range(4)]
    layer.decode(torch.from_numpy(c.x), torch.from_numpy(x_att), ys)
    for p in range(4):
        xin = c.x if p < 3 else x_att
        want = O.ref_bmm(np.zeros((22, 128), np.float32), xin, [a[p] for a in c.A], [b[p] for b in c.B], c.scales,
                         c.bins, "f32")
        np.testing.assert_allclose(ys[p].numpy(), want, rtol=1e-4, atol=1e-5)
