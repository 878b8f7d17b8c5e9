"""Adapter load / offload helpers on the GPU against the CPU oracle, through the
C ABI.  Byte and index movement: everything is compared bit for bit."""
import numpy as np
import pytest
import torch

from oracle import lora_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n_layers,heads,head_dim,rank", [(3, 4, 32, 8), (40, 2, 20, 3), (2, 32, 128, 64)])
def test_load_rows_into_pool_equals_index_put(gpu, dtype, n_layers, heads, head_dim, rank):
    """``buffer[loc] = rows`` for key and value buffers of every layer in one call
    equals the oracle's load_into_pool (= the reference's per-layer index_put);
    pages not named by loc keep their bytes; a page id outside the pool is skipped."""
    from slora_hip.infer_adapter import load_rows_into_pool
    rng = np.random.default_rng(n_layers * 100 + rank)
    n_rows = 4 * rank
    n_pages = n_rows + 41
    loc_np = rng.permutation(n_pages)[:n_rows].astype(np.int64)
    g = torch.Generator(device=gpu)
    g.manual_seed(1)
    bufs = [torch.randn((n_pages, heads, head_dim), generator=g, device=gpu).to(dtype) for _ in range(2 * n_layers)]
    rows = [torch.randn((n_rows, heads, head_dim), generator=g, device=gpu).to(dtype) for _ in range(2 * n_layers)]
    before = [b.clone() for b in bufs]
    loc = torch.from_numpy(loc_np).to(gpu)
    load_rows_into_pool(bufs, rows, loc)
    torch.cuda.synchronize()
    for l in range(n_layers):
        kb = before[2 * l].view(torch.uint8).cpu().numpy().reshape(n_pages, -1).copy()
        vb = before[2 * l + 1].view(torch.uint8).cpu().numpy().reshape(n_pages, -1).copy()
        w = np.stack([rows[2 * l].view(torch.uint8).cpu().numpy().reshape(n_rows, -1),
                      rows[2 * l + 1].view(torch.uint8).cpu().numpy().reshape(n_rows, -1)])
        O.load_into_pool(kb, vb, w, loc_np)
        assert np.array_equal(bufs[2 * l].view(torch.uint8).cpu().numpy().reshape(n_pages, -1), kb)
        assert np.array_equal(bufs[2 * l + 1].view(torch.uint8).cpu().numpy().reshape(n_pages, -1), vb)
    # out-of-range page ids are skipped
    bad = loc.clone()
    bad[0], bad[1] = n_pages, -5
    snap = bufs[0].clone()
    load_rows_into_pool(bufs[:1], [rows[0] + 1], bad)
    torch.cuda.synchronize()
    same = (bufs[0] == snap).view(n_pages, -1).all(dim=1).cpu().numpy()
    assert same[loc_np[0]] and same[loc_np[1]] and not same[loc_np[2]]


def test_load_rows_then_decode_uses_them(gpu):
    """pack -> scatter into the pool -> dispatch_bgmv equals the dense LoRA."""
    from slora_hip import dispatch_bgmv
    from slora_hip.infer_adapter import load_rows_into_pool
    rng = np.random.default_rng(11)
    H, r, n_pages, B = 256, 16, 200, 9
    A = [rng.standard_normal((H, r)).astype(np.float32) / 16 for _ in range(4)]
    Bm = [rng.standard_normal((r, H)).astype(np.float32) / 4 for _ in range(4)]
    w = O.round_to(O.pack_w_combined(A, Bm, H), "f16")
    a_start, a_len, a_loc = O.build_tables([r], rng.permutation(n_pages)[: 4 * r])
    key = torch.zeros((n_pages, 4, H // 4), dtype=torch.float16, device=gpu)
    val = torch.zeros_like(key)
    load_rows_into_pool([key, val], [torch.from_numpy(w[0]).to(gpu, torch.float16).view(4 * r, 4, H // 4),
                                     torch.from_numpy(w[1]).to(gpu, torch.float16).view(4 * r, 4, H // 4)],
                        torch.from_numpy(a_loc).to(gpu))
    x = O.round_to(rng.standard_normal((B, H)).astype(np.float32), "f16")
    t = [torch.from_numpy(v).to(gpu) for v in (a_start, a_len, a_loc, np.zeros(B, np.int64))]
    scal = torch.tensor([2.0], dtype=torch.float16, device=gpu)
    for p in range(4):
        d = torch.zeros((B, r), dtype=torch.float16, device=gpu)
        y = torch.zeros((B, H), dtype=torch.float16, device=gpu)
        dispatch_bgmv(d, torch.from_numpy(x).to(gpu, torch.float16), key, *t, p, scal)
        dispatch_bgmv(y, d, val, *t, p, scal)
        ref = 2.0 * (x.astype(np.float64) @ O.round_to(A[p], "f16").astype(np.float64)) @ \
            O.round_to(Bm[p], "f16").astype(np.float64)
        np.testing.assert_allclose(y.float().cpu().numpy(), ref, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("n,ranks", [(1, [8]), (5, [8, 64, 70, 2]), (300, [16, 64, 128]), (2500, [2, 4])])
def test_var_len_copy_and_table_compaction(gpu, n, ranks):
    """launch_var_len_copy and compact_adapter_tables against the oracle, bit for
    bit; lists longer than 256 entries (where the reference's mask over-copies)
    included."""
    from slora_hip.infer_adapter import compact_adapter_tables, launch_var_len_copy
    rng = np.random.default_rng(n)
    r = rng.choice(ranks, size=n)
    a_start, a_len, a_loc = O.build_tables(r, rng.permutation(1 << 20)[: int(4 * r.sum())])
    scal = rng.standard_normal(n).astype(np.float16)
    for frac in (0.0, 0.5, 1.0):
        keep = rng.random(n) < frac
        ns, nl, nloc, nsc, rem = O.ref_offload_tables(a_start, a_len, a_loc, scal, keep)
        d = [torch.from_numpy(v).to(gpu) for v in (a_start, a_len, a_loc, scal, keep)]
        g_ns, g_nl, g_nloc, g_nsc, g_rem = compact_adapter_tables(*d)
        assert g_ns.cpu().numpy().tolist() == ns.tolist()
        assert g_nl.cpu().numpy().tolist() == nl.tolist()
        assert np.array_equal(g_nloc.cpu().numpy(), nloc)
        assert np.array_equal(g_nsc.cpu().numpy().view(np.uint16), nsc.view(np.uint16))
        assert np.array_equal(g_rem.cpu().numpy(), rem)
        # the reference's own sequence of calls: cumsum on the host side, then the copy kernel
        left = np.nonzero(keep)[0]
        if left.size:
            out = torch.full((int(nl.sum()),), -1, dtype=torch.int64, device=gpu)
            launch_var_len_copy(d[0][torch.from_numpy(left).to(gpu)], g_nl, d[2], g_ns, out)
            assert np.array_equal(out.cpu().numpy(), nloc)


@pytest.mark.parametrize("tot", [1, 37, 4096, 4097, 70000, 262144])
def test_page_allocator_equals_the_reference_allocator(gpu, tot):
    """alloc / alloc_contiguous / free on the device against the oracle's restatement
    of MemoryAllocator, bit for bit, over a random sequence of calls on maps that
    cross the kernels' 4096-page blocks."""
    from slora_hip.infer_adapter import PageAllocator
    rng = np.random.default_rng(tot)
    pa = PageAllocator(tot, gpu)
    state = np.ones(tot, np.uint8)
    held = []
    for step in range(40):
        free_now = int(state.sum())
        op = rng.integers(0, 4)
        if op == 0 and free_now:
            need = int(rng.integers(0, min(free_now, max(1, tot // 3)) + 1))
            exp = O.ref_alloc(state, need)
            got = pa.alloc(need)
            assert np.array_equal(got.cpu().numpy(), exp), (step, "alloc", need)
            held.append(exp)
        elif op == 1 and free_now:
            need = int(rng.integers(1, min(free_now, max(1, tot // 8)) + 1))
            exp = O.ref_alloc_contiguous(state, need)
            got = pa.alloc_contiguous(need)
            if exp is None:
                assert got is None, (step, "contiguous", need)
            else:
                assert got is not None and (got[1], got[2]) == (exp[1], exp[2]), (step, "contiguous", need)
                assert np.array_equal(got[0].cpu().numpy(), exp[0])
                held.append(exp[0])
        elif held:
            # give back a random half of one earlier allocation, scattered
            blk = held.pop(int(rng.integers(0, len(held))))
            if blk.size:
                pick = rng.permutation(blk)[: max(1, blk.size // 2)]
                rest = np.setdiff1d(blk, pick)
                O.ref_free(state, pick)
                pa.free(torch.from_numpy(pick).to(gpu))
                if rest.size:
                    held.append(rest)
        assert np.array_equal(pa.mem_state.cpu().numpy().astype(np.uint8), state), step
        assert pa.can_use_mem_size == int(state.sum())
    with pytest.raises(Exception, match="no enough pool space"):
        pa.alloc(pa.can_use_mem_size + 1)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("hidden,h_out,rank", [(256, [256, 64, 64, 256], 16), (512, [512] * 4, 64), (128, [128] * 4, 12)])
def test_merge_and_unmerge_adapter(gpu, dtype, hidden, h_out, rank):
    """gather_lora_a is the exact transpose-gather; merge_adapter equals the
    oracle's restatement of the reference within rtol 1e-2 and an absolute term of
    one storage-type rounding of the update A B * scaling (the reference rounds the
    update before adding it, the kernel adds the float sum: where W and the update
    cancel, the difference is that rounding, not a fraction of the result) --
    1e-3 in fp16, 8e-3 in bf16 at these magnitudes; exactly on integer-valued
    weights, where merge + unmerge also returns the base weights bit for bit."""
    from slora_hip.infer_adapter import gather_lora_a, load_rows_into_pool, merge_adapter, unmerge_adapter
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    rng = np.random.default_rng(hidden + rank)
    n_pages, heads = 4 * rank * 3 + 17, 4
    ranks = [8, rank, 8]
    a_start, a_len, a_loc = O.build_tables(ranks, rng.permutation(n_pages)[: 4 * sum(ranks)])
    scal = np.array([1.0, 2.0, 0.5], np.float32)
    key = torch.zeros((n_pages, heads, hidden // heads), dtype=tdt, device=gpu)
    val = torch.zeros_like(key)
    for integer in (False, True):
        if integer:
            A = [rng.integers(-2, 3, size=(hidden, rank)).astype(np.float32) for _ in range(4)]
            Bm = [rng.integers(-2, 3, size=(rank, h_out[p])).astype(np.float32) for p in range(4)]
            W0 = [rng.integers(-8, 9, size=(hidden, h_out[p])).astype(np.float32) for p in range(4)]
        else:
            A = [O.round_to(rng.standard_normal((hidden, rank)).astype(np.float32) / 16, dtype) for _ in range(4)]
            Bm = [O.round_to(rng.standard_normal((rank, h_out[p])).astype(np.float32) / 4, dtype) for p in range(4)]
            W0 = [O.round_to(rng.standard_normal((hidden, h_out[p])).astype(np.float32), dtype) for p in range(4)]
        w = O.pack_w_combined(A, Bm, hidden)
        loc1 = a_loc[a_start[1]: a_start[1] + a_len[1]]
        load_rows_into_pool([key, val], [torch.from_numpy(w[0]).to(gpu, tdt).view(4 * rank, heads, -1),
                                         torch.from_numpy(w[1]).to(gpu, tdt).view(4 * rank, heads, -1)],
                            torch.from_numpy(loc1).to(gpu))
        t = [torch.from_numpy(v).to(gpu) for v in (a_start, a_len, a_loc)]
        scales = torch.from_numpy(scal).to(gpu, torch.float16)
        for p in range(4):
            a_p = gather_lora_a(key, t[2], int(a_start[1]) + p * rank, rank, hidden, (rank + 7) // 8 * 8)
            assert torch.equal(a_p[:, :rank], torch.from_numpy(A[p]).to(gpu, tdt))
            assert not a_p[:, rank:].any()
        Wg = [torch.from_numpy(v).to(gpu, tdt) for v in W0]
        merge_adapter(Wg, key, val, *t, scales, 1)
        for p in range(4):
            ref = O.ref_merge_adapter(W0[p], A[p], Bm[p], 2.0, 1.0, dtype)
            if integer:
                assert np.array_equal(Wg[p].float().cpu().numpy(), ref), p
            else:
                np.testing.assert_allclose(Wg[p].float().cpu().numpy(), ref, rtol=1e-2,
                                           atol=1e-3 if dtype == "f16" else 8e-3)
        unmerge_adapter(Wg, key, val, *t, scales, 1)
        for p in range(4):
            if integer:
                assert np.array_equal(Wg[p].float().cpu().numpy(), W0[p]), p
            else:
                np.testing.assert_allclose(Wg[p].float().cpu().numpy(), W0[p], rtol=1e-2,
                                           atol=4e-3 if dtype == "f16" else 3e-2)


def test_pool_ops_reject_bad_arguments(gpu):
    from slora_hip.infer_adapter import compact_adapter_tables, launch_var_len_copy, load_rows_into_pool
    buf = torch.zeros((10, 2, 8), dtype=torch.float16, device=gpu)
    rows = torch.zeros((3, 2, 8), dtype=torch.float16, device=gpu)
    loc = torch.arange(3, device=gpu)
    with pytest.raises(RuntimeError):
        load_rows_into_pool([buf], [rows, rows], loc)
    with pytest.raises(RuntimeError):
        load_rows_into_pool([buf], [rows.float()], loc)
    with pytest.raises(RuntimeError):
        load_rows_into_pool([buf], [rows], loc.int())
    with pytest.raises(RuntimeError):
        load_rows_into_pool([buf], [rows.cpu()], loc)
    with pytest.raises(RuntimeError):
        launch_var_len_copy(loc, loc[:2], loc, loc, loc.clone())
    with pytest.raises(RuntimeError):
        compact_adapter_tables(loc, loc, loc, torch.zeros(3, device=gpu, dtype=torch.float16),
                               torch.ones(2, device=gpu, dtype=torch.bool))


# ---------------------------------------------------------------------------
# the packer and the InferAdapter class
# ---------------------------------------------------------------------------
class _Adapter:
    """What InferAdapter.load_adapters needs of an adapter: name, rank, scaling and per layer
    the q, k, v, o matrices as the reference keeps them at home (A_p [hidden, r], B_p [r, h_out])."""

    def __init__(self, name, r, alpha, lora_A, lora_B):
        self.lora_dir, self.r, self.scaling = name, r, alpha / r
        self.lora_A, self.lora_B = lora_A, lora_B


class _RefStyleLayer:
    """A layer object with the reference's interface (lora_layer_weight.py:226-246): w_combined
    appears on load_to_gpu() and goes away on offload_from_gpu()."""

    def __init__(self, w_combined_home):
        self.home, self.w_combined = w_combined_home, None

    def load_to_gpu(self, prefetch=False):
        self.w_combined = self.home

    def offload_from_gpu(self):
        self.w_combined = None


def _np_mats(rng, hidden, h_out, r, n_layers, dtype):
    A = [[O.round_to(rng.standard_normal((hidden, r)).astype(np.float32) / 8, dtype) for _ in range(4)]
         for _ in range(n_layers)]
    B = [[O.round_to(rng.standard_normal((r, h_out[p])).astype(np.float32) / 4, dtype) for p in range(4)]
         for _ in range(n_layers)]
    return A, B


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("hidden,page_elems,h_out,rank,n_layers", [
    (256, 256, [256] * 4, 16, 3),
    (512, 512, [512, 64, 64, 512], 64, 2),      # grouped-query k/v: B^T fills part of its slot, zeros behind
    (192, 256, [256, 128, 128, 192], 8, 9),     # rows shorter than a page, more matrices than one launch takes
    (128, 128, [128] * 4, 12, 1),               # a rank that is no multiple of 8
])
def test_pack_lora_into_pool_equals_w_combined_index_put(gpu, dtype, hidden, page_elems, h_out, rank, n_layers):
    """A_p / B_p transposed straight into the pool pages give bit for bit what the oracle's
    ``pack_w_combined`` + ``load_into_pool`` (= the reference's host-side w_combined and its
    per-layer index_put) leave there; other pages keep their bytes."""
    from slora_hip.infer_adapter import pack_lora_into_pool
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    rng = np.random.default_rng(hidden + rank)
    n_pages = 4 * rank + 37
    loc_np = rng.permutation(n_pages)[: 4 * rank].astype(np.int64)
    A, B = _np_mats(rng, hidden, h_out, rank, n_layers, dtype)
    g = torch.Generator(device=gpu)
    g.manual_seed(3)
    keys = [torch.randn((n_pages, 2, page_elems // 2), generator=g, device=gpu).to(tdt) for _ in range(n_layers)]
    vals = [torch.randn((n_pages, 2, page_elems // 2), generator=g, device=gpu).to(tdt) for _ in range(n_layers)]
    want_k = [k.float().cpu().numpy().reshape(n_pages, page_elems).copy() for k in keys]
    want_v = [v.float().cpu().numpy().reshape(n_pages, page_elems).copy() for v in vals]
    for l in range(n_layers):
        O.load_into_pool(want_k[l], want_v[l], O.pack_w_combined(A[l], B[l], page_elems), loc_np)
    dA = [[torch.from_numpy(a).to(gpu, tdt) for a in A[l]] for l in range(n_layers)]
    dB = [[torch.from_numpy(b).to(gpu, tdt) for b in B[l]] for l in range(n_layers)]
    pack_lora_into_pool(keys, vals, dA, dB, torch.from_numpy(loc_np).to(gpu), rank)
    torch.cuda.synchronize()
    for l in range(n_layers):
        assert np.array_equal(keys[l].float().cpu().numpy().reshape(n_pages, page_elems), want_k[l]), l
        assert np.array_equal(vals[l].float().cpu().numpy().reshape(n_pages, page_elems), want_v[l]), l


@pytest.mark.parametrize("placement", [False, True])
def test_infer_adapter_load_offload_and_decode(gpu, placement):
    """InferAdapter over a MemoryAllocator: adapters arrive in three loads (device matrices, and
    objects with the reference's w_combined interface), some are dropped, one comes back.  After
    every step the four tables equal the oracle's (build_tables appended per load,
    ref_offload_tables per offload) with the page ids the oracle's allocator hands out, and
    dispatch_bgmv over the pool gives the dense LoRA of every loaded adapter."""
    from slora_hip import dispatch_bgmv
    from slora_hip.infer_adapter import InferAdapter, MemoryAllocator
    H, L, heads = 256, 2, 4
    rng = np.random.default_rng(5)
    mm = MemoryAllocator(600, 0, torch.float16, heads, H // heads, L, device=gpu)
    for b in mm.key_buffer + mm.value_buffer:
        b.zero_()
    # some KV pages are in use between the adapters' pages
    kv = mm.alloc(50)
    mm.free(kv[::2].contiguous())
    state = mm.mem_state.cpu().numpy().astype(np.uint8)
    ia = InferAdapter.init(mm, prefetch_stream=torch.cuda.Stream(), placement=placement, device=gpu)
    ranks = {"a": 8, "b": 16, "c": 32, "d": 8, "e": 64}
    mats, adapters = {}, {}
    for name, r in ranks.items():
        A, B = _np_mats(rng, H, [H] * 4, r, L, "f16")
        mats[name] = (A, B)
        if name in ("b", "d"):   # the reference's interface: per layer a w_combined [2, 4r, heads, head_dim]
            layers = [_RefStyleLayer(torch.from_numpy(O.pack_w_combined(A[l], B[l], H)).to(gpu, torch.float16)
                                     .view(2, 4 * r, heads, H // heads)) for l in range(L)]
            ad = _Adapter(name, r, 16.0, None, None)
            ad.layers = layers
        else:
            ad = _Adapter(name, r, 16.0, [[torch.from_numpy(a).to(gpu, torch.float16) for a in A[l]] for l in range(L)],
                          [[torch.from_numpy(b).to(gpu, torch.float16) for b in B[l]] for l in range(L)])
        adapters[name] = ad

    tables = dict(start=np.zeros(0, np.int64), len=np.zeros(0, np.int64), loc=np.zeros(0, np.int64),
                  scal=np.zeros(0, np.float32), dirs=[])

    def oracle_load(names):
        new = [n for n in names if n not in tables["dirs"]]
        if placement:
            locs = []
            for n in new:
                got = O.ref_alloc_contiguous(state, 4 * ranks[n])
                locs.append(got[0] if got is not None else O.ref_alloc(state, 4 * ranks[n]))
            new_loc = np.concatenate(locs)
        else:
            new_loc = O.ref_alloc(state, sum(4 * ranks[n] for n in new))
        s, ln, lc = O.build_tables([ranks[n] for n in new], new_loc)
        tables["start"] = np.concatenate([tables["start"], s + tables["loc"].size])
        tables["len"] = np.concatenate([tables["len"], ln])
        tables["loc"] = np.concatenate([tables["loc"], lc])
        tables["scal"] = np.concatenate([tables["scal"], [16.0 / ranks[n] for n in new]]).astype(np.float32)
        tables["dirs"] += new

    def oracle_offload(reserve):
        keep = np.array([d in reserve for d in tables["dirs"]])
        s, ln, lc, sc, removed = O.ref_offload_tables(tables["start"], tables["len"], tables["loc"], tables["scal"], keep)
        O.ref_free(state, removed)
        tables.update(start=s, len=ln, loc=lc, scal=sc, dirs=[d for d, k in zip(tables["dirs"], keep) if k])

    def check():
        torch.cuda.synchronize()
        assert ia.adapter_dirs == tables["dirs"]
        assert np.array_equal(ia.a_start.cpu().numpy(), tables["start"])
        assert np.array_equal(ia.a_len.cpu().numpy(), tables["len"])
        assert np.array_equal(ia.a_loc.cpu().numpy(), tables["loc"])
        assert np.array_equal(ia.a_scaling.float().cpu().numpy(), tables["scal"])
        assert np.array_equal(mm.mem_state.cpu().numpy().astype(np.uint8), state)
        assert mm.can_use_mem_size == int(state.sum())
        for i, d in enumerate(ia.adapter_dirs):
            assert ia.idx_map[d] == i
            assert ia.start_and_rank(d) == (int(tables["start"][i]), ranks[d])
        if not ia.adapter_dirs:
            return
        # one token per loaded adapter through the kernels, layer 1, every projection
        n = len(ia.adapter_dirs)
        x_np = O.round_to(rng.standard_normal((n, H)).astype(np.float32), "f16")
        x = torch.from_numpy(x_np).to(gpu, torch.float16)
        bins = torch.arange(n, dtype=torch.int64, device=gpu)
        for p in range(4):
            d = torch.zeros((n, 64), dtype=torch.float16, device=gpu)
            dispatch_bgmv(d, x, mm.key_buffer[1], ia.a_start, ia.a_len, ia.a_loc, bins, p, ia.a_scaling)
            y = torch.zeros((n, H), dtype=torch.float16, device=gpu)
            dispatch_bgmv(y, d, mm.value_buffer[1], ia.a_start, ia.a_len, ia.a_loc, bins, p, ia.a_scaling)
            want = np.stack([(x_np[i].astype(np.float64) @ mats[dn][0][1][p] @ mats[dn][1][1][p]) * 16.0 / ranks[dn]
                             for i, dn in enumerate(ia.adapter_dirs)])
            np.testing.assert_allclose(y.float().cpu().numpy(), want, rtol=2e-2, atol=2e-2)

    ia.load_adapters([adapters["a"], adapters["b"]])
    oracle_load(["a", "b"])
    check()
    ia.load_adapters([adapters["b"], adapters["c"], adapters["d"]], prefetch=True)   # b is there already
    torch.cuda.current_stream().wait_stream(ia.prefetch_stream)
    oracle_load(["c", "d"])
    check()
    ia.prefetch_tag.clear()                      # nothing is protected by a prefetch any more
    ia.offload_adapters(["a", "c"])
    oracle_offload(["a", "c"])
    check()
    ia.load_adapters([adapters["e"], adapters["b"]])
    oracle_load(["e", "b"])
    check()
    ia.offload_adapters(["a", "c", "e", "b"])     # everything reserved: nothing happens
    check()
    ia.offload_adapters([])
    oracle_offload([])
    check()
    assert mm.can_use_mem_size == 600 - 25


def test_prefetch_keeps_its_page_list_while_the_main_stream_allocates(gpu):
    """A prefetching load queues its pack kernels on the side stream and returns; the page list
    they read must stay theirs.  The side stream is kept busy first so that the kernels are still
    queued when the main stream allocates and overwrites int64 tensors of the page list's size
    (what the caching allocator would hand out if the list's block had been given back): every
    page must still hold the packed weights, bit for bit."""
    from slora_hip.infer_adapter import InferAdapter, MemoryAllocator, page_checksums
    H, L, heads, r = 256, 2, 4, 16
    rng = np.random.default_rng(11)
    mm = MemoryAllocator(400, 0, torch.float16, heads, H // heads, L, device=gpu)
    for b in mm.key_buffer + mm.value_buffer:
        b.zero_()
    side = torch.cuda.Stream()
    ia = InferAdapter.init(mm, prefetch_stream=side, device=gpu)
    A, B = _np_mats(rng, H, [H] * 4, r, L, "f16")
    ad = _Adapter("p", r, 16.0, [[torch.from_numpy(a).to(gpu, torch.float16) for a in A[l]] for l in range(L)],
                  [[torch.from_numpy(b).to(gpu, torch.float16) for b in B[l]] for l in range(L)])
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        torch.cuda._sleep(50_000_000)        # tens of milliseconds: the loads below queue behind it
    ia.load_adapters([ad], prefetch=True)
    junk = []
    for _ in range(64):                       # same size and dtype as the page list: the same allocator bin
        t = torch.empty(4 * r, dtype=torch.int64, device=gpu)
        t.fill_(399)                          # a valid page nobody owns
        junk.append(t)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    loc = ia.a_loc.cpu().numpy()
    assert np.array_equal(loc, np.arange(4 * r))          # first free pages of an empty map
    for l in range(L):
        w = O.pack_w_combined(A[l], B[l], H)               # [2, 4r, H]
        for side_i, buf in ((0, mm.key_buffer[l]), (1, mm.value_buffer[l])):
            want = O.round_to(w[side_i], "f16").astype(np.float16).view(np.uint32)
            got = page_checksums(buf, ia.a_loc).cpu().numpy().view(np.uint32)
            assert np.array_equal(got, np.bitwise_xor.reduce(want, axis=1)), (l, side_i)
            assert int(page_checksums(buf, torch.tensor([399], device=gpu)).item()) == 0
    assert len(junk) == 64


def test_memory_allocator_places_an_adapter_in_one_run(gpu):
    """alloc_adapter: one contiguous stretch when the map has one (the first such), the first
    free pages otherwise -- against the oracle's alloc_contiguous / alloc."""
    from slora_hip.infer_adapter import MemoryAllocator
    mm = MemoryAllocator(300, 0, torch.float16, 2, 8, 1, device=gpu)
    rng = np.random.default_rng(9)
    busy = rng.permutation(300)[:120].astype(np.int64)
    all_pages = mm.alloc(300)
    keep_free = np.setdiff1d(np.arange(300), busy)
    mm.free(torch.from_numpy(keep_free).to(gpu))
    state = np.zeros(300, np.uint8)
    state[keep_free] = 1
    for need in (3, 7, 2, 40, 5):
        got = mm.alloc_adapter(need).cpu().numpy()
        run = O.ref_alloc_contiguous(state, need)
        want = run[0] if run is not None else O.ref_alloc(state, need)
        assert np.array_equal(got, want), need
        assert np.array_equal(mm.mem_state.cpu().numpy().astype(np.uint8), state)
    assert all_pages.numel() == 300


@pytest.mark.parametrize("dtype,heads,head_dim", [(torch.float16, 32, 128), (torch.bfloat16, 4, 24)])
def test_page_checksums_equal_numpy_xor(gpu, dtype, heads, head_dim):
    """page_checksums against the xor of the pages' 32-bit words computed with numpy: exact;
    page ids outside the buffer give 0; an empty list gives an empty result."""
    from slora_hip.infer_adapter import page_checksums
    g = torch.Generator(device=gpu)
    g.manual_seed(9)
    buf = torch.randn((300, heads, head_dim), generator=g, device=gpu, dtype=torch.float32).to(dtype)
    rng = np.random.default_rng(9)
    loc = rng.integers(0, 300, size=1001).astype(np.int64)
    loc[5], loc[77] = -1, 300
    got = page_checksums(buf, torch.from_numpy(loc).to(gpu)).cpu().numpy().view(np.uint32)
    words = buf.cpu().view(torch.int16).numpy().reshape(300, -1).view(np.uint32)
    want = np.bitwise_xor.reduce(words, axis=1)
    ok = (loc >= 0) & (loc < 300)
    assert np.array_equal(got[ok], want[loc[ok]])
    assert np.all(got[~ok] == 0)
    assert page_checksums(buf, torch.empty(0, dtype=torch.int64, device=gpu)).numel() == 0


def test_page_xor_is_an_exact_in_place_xor(gpu):
    """page_xor against numpy: listed pages ^= key word by word, other pages and ids outside the
    buffer untouched, key 0 and an empty list change nothing."""
    from slora_hip.infer_adapter import page_xor
    rng = np.random.default_rng(13)
    words = rng.integers(0, 2 ** 32, size=(200, 640), dtype=np.uint64).astype(np.uint32)   # 2560-byte pages
    buf = torch.from_numpy(words.view(np.int32)).to(gpu)
    loc = rng.permutation(200)[:77].astype(np.int64)
    loc_dev = torch.from_numpy(np.concatenate([loc, [-1, 200]])).to(gpu)
    page_xor(buf, loc_dev, 0)
    page_xor(buf, torch.empty(0, dtype=torch.int64, device=gpu), 0x5a5a5a5a)
    assert np.array_equal(buf.cpu().numpy().view(np.uint32), words)
    page_xor(buf, loc_dev, 0x9e3779b9)
    want = words.copy()
    want[loc] ^= np.uint32(0x9e3779b9)
    assert np.array_equal(buf.cpu().numpy().view(np.uint32), want)
