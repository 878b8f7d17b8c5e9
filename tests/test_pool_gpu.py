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
