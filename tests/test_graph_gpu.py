"""The operators recorded into a HIP graph and replayed: every replay is checked against the
same calls made eagerly with ``plan=False``, with the batch (the per-token adapter ids, or the
request table) rewritten in place between the replays and eager work and synchronisations in
between.  Two forms: the explicit plan rebuilt inside the graph, and the calls exactly as the
reference issues them (no plan argument), for which the library builds the plan inside the
capture."""
import numpy as np
import pytest
import torch

from lora_cases import make_case
from test_bgmv_gpu import GpuCase
from test_sgmm_gpu import seg_case, _shrink_args

pytestmark = pytest.mark.gpu


def _capture(fn):
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        fn()                                   # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    return g


@pytest.mark.parametrize("how", ["explicit-plan", "drop-in"])
def test_decode_step_in_a_graph(gpu, how):
    import slora_hip
    from slora_hip import dispatch_bgmv, dispatch_bgmv_qkv_expand, dispatch_bgmv_qkv_shrink
    slora_hip.set_plan_cache_enabled(True)
    slora_hip.clear_plan_cache()
    c = make_case(909, 512, [16, 8, 32, 64], 57, dtype="f16", zipf_alpha=1.0)
    g = GpuCase(c, gpu)
    R, H = 64, 512
    t = (g.a_start, g.a_len, g.a_loc, g.bins)
    d = [torch.zeros((c.batch, R), dtype=g.tdt, device=gpu) for _ in range(3)]
    y0 = [torch.randn((c.batch, H), device=gpu).to(g.tdt) for _ in range(4)]
    y = [t_.clone() for t_ in y0]
    plan = slora_hip.make_plan(*t, R, c.n_pages) if how == "explicit-plan" else None

    def step():
        for i in range(4):
            y[i].copy_(y0[i])
        for b in d:
            b.zero_()                          # a fill kernel (no memset node)
        if how == "explicit-plan":
            slora_hip.rebuild_plan(plan, *t, c.n_pages)
            dispatch_bgmv_qkv_shrink(d[0], d[1], d[2], g.x, g.key, *t, plan=plan)
            dispatch_bgmv_qkv_expand(y[0], y[1], y[2], d[0], d[1], d[2], g.value, *t, g.scales, plan=plan)
            dispatch_bgmv(d[0], g.x, g.key, *t, 3, g.scales, plan=plan)
            dispatch_bgmv(y[3], d[0], g.value, *t, 3, g.scales, plan=plan)
        else:                                  # the reference's eight calls, nothing else
            for p in range(3):
                dispatch_bgmv(d[p], g.x, g.key, *t, p, g.scales)
                dispatch_bgmv(y[p], d[p], g.value, *t, p, g.scales)
            dispatch_bgmv(d[0], g.x, g.key, *t, 3, g.scales)
            dispatch_bgmv(y[3], d[0], g.value, *t, 3, g.scales)

    def eager():
        out = []
        for p in range(4):
            dd = torch.zeros((c.batch, R), dtype=g.tdt, device=gpu)
            yy = y0[p].clone()
            dispatch_bgmv(dd, g.x, g.key, *t, p, g.scales, plan=False)
            dispatch_bgmv(yy, dd, g.value, *t, p, g.scales, plan=False)
            out.append(yy)
        torch.cuda.synchronize()
        return out

    slora_hip.plan_cache_stats(reset=True)
    graph = _capture(step)
    if how == "drop-in":
        st = slora_hip.plan_cache_stats()
        # the warm-up run built one plan and the capture built its own; the other calls reused them
        assert st["builds"] == 2 and st["hits"] == 14, st
    rng = np.random.default_rng(5)
    for rep in range(4):
        if rep:                                # a new batch in the same tensor: the replay must follow it
            g.bins.copy_(torch.from_numpy(rng.integers(0, len(c.ranks), size=c.batch)).to(gpu))
        want = eager()
        graph.replay()
        torch.cuda.synchronize()
        for p in range(4):
            assert torch.equal(y[p], want[p]), (how, rep, p)
    slora_hip.clear_plan_cache()


@pytest.mark.parametrize("how", ["explicit-plan", "drop-in"])
def test_prefill_step_in_a_graph(gpu, how):
    import slora_hip
    from slora_hip import (lora_get_qkvo_fwd_expand, lora_get_qkvo_fwd_shrink, lora_get_qkvo_fwd_shrink_qkv,
                           make_prefill_plan)
    slora_hip.set_plan_cache_enabled(True)
    slora_hip.clear_prefill_plan_cache()
    c = seg_case(41, 256, [16, 8, 32, 64], 9, 3, 60, "bf16")
    g = GpuCase(c, gpu)
    start, lens, ids, max_len = _shrink_args(c, g, gpu)
    R, H = 64, 256
    T = c.batch
    seg = (g.a_loc, g.a_start, g.a_len, start, lens, ids)
    w_a, w_b = g.key.view(c.n_pages, H), g.value.view(c.n_pages, H)
    d = [torch.zeros((T, R), dtype=g.tdt, device=gpu) for _ in range(3)]
    y0 = [torch.randn((T, H), device=gpu).to(g.tdt) for _ in range(4)]
    y = [t_.clone() for t_ in y0]

    def step():
        for i in range(4):
            y[i].copy_(y0[i])
        if how == "explicit-plan":
            plan = make_prefill_plan(g.a_start, g.a_len, start, lens, ids, T, R, max_len)
            lora_get_qkvo_fwd_shrink_qkv(g.x, w_a, d[0], d[1], d[2], *seg, H, R, max_len, plan=plan)
            for p in range(3):
                lora_get_qkvo_fwd_expand(d[p], w_b, y[p], g.scales, *seg, H, p, R, max_len)
            lora_get_qkvo_fwd_shrink(g.x, w_a, d[0], *seg, H, 3, R, max_len, plan=plan)
            lora_get_qkvo_fwd_expand(d[0], w_b, y[3], g.scales, *seg, H, 3, R, max_len)
        else:
            for p in range(3):
                lora_get_qkvo_fwd_shrink(g.x, w_a, d[p], *seg, H, p, R, max_len)
                lora_get_qkvo_fwd_expand(d[p], w_b, y[p], g.scales, *seg, H, p, R, max_len)
            lora_get_qkvo_fwd_shrink(g.x, w_a, d[0], *seg, H, 3, R, max_len)
            lora_get_qkvo_fwd_expand(d[0], w_b, y[3], g.scales, *seg, H, 3, R, max_len)

    def eager():
        out = []
        for p in range(4):
            dd = torch.zeros((T, R), dtype=g.tdt, device=gpu)
            yy = y0[p].clone()
            lora_get_qkvo_fwd_shrink(g.x, w_a, dd, *seg, H, p, R, max_len, plan=False)
            lora_get_qkvo_fwd_expand(dd, w_b, yy, g.scales, *seg, H, p, R, max_len)
            out.append(yy)
        torch.cuda.synchronize()
        return out

    graph = _capture(step)
    rng = np.random.default_rng(6)
    for rep in range(3):
        if rep:                                # other adapters for the same requests, in place
            ids.copy_(torch.from_numpy(np.sort(rng.integers(0, len(c.ranks), size=ids.numel()))).to(gpu))
        want = eager()
        graph.replay()
        torch.cuda.synchronize()
        for p in range(4):
            assert torch.equal(y[p], want[p]), (how, rep, p)
    slora_hip.clear_prefill_plan_cache()


@pytest.mark.parametrize("kv_out", [256, 64])
def test_plan_without_item_count_walks_every_item(gpu, kv_out):
    """A plan whose item count the host does not have (readback=False, as after rebuild_plan or
    inside a capture) is launched with a quarter of its capacity in workgroups.  Here nearly
    every token has an adapter of its own, so the batch has close to the capacity in items and
    every workgroup walks several of them; with k/v narrower than a page the expand also
    uses its interleaved grid.  Bitwise the results of the plan-free calls."""
    import slora_hip
    from slora_hip import dispatch_bgmv, dispatch_bgmv_qkv_expand, dispatch_bgmv_qkv_shrink
    n_ad, batch, H, R = 300, 600, 256, 16
    rng = np.random.default_rng(3)
    bins = np.concatenate([np.arange(n_ad), rng.integers(0, n_ad, size=batch - n_ad)])
    rng.shuffle(bins)
    c = make_case(77, H, [R] * n_ad, batch, dtype="bf16", bins=bins, h_out=[H, kv_out, kv_out, H])
    g = GpuCase(c, gpu)
    t = (g.a_start, g.a_len, g.a_loc, g.bins)
    plan = slora_hip.make_plan(*t, R, c.n_pages, False)
    assert plan.n_items == 0
    d = [torch.zeros((batch, R), dtype=g.tdt, device=gpu) for _ in range(3)]
    y0 = [torch.randn((batch, h), device=gpu).to(g.tdt) for h in c.h_out]
    y = [t_.clone() for t_ in y0]
    dispatch_bgmv_qkv_shrink(d[0], d[1], d[2], g.x, g.key, *t, plan=plan)
    dispatch_bgmv_qkv_expand(y[0], y[1], y[2], d[0], d[1], d[2], g.value, *t, g.scales, plan=plan)
    do = torch.zeros((batch, R), dtype=g.tdt, device=gpu)
    dispatch_bgmv(do, g.x, g.key, *t, 3, g.scales, plan=plan)
    dispatch_bgmv(y[3], do, g.value, *t, 3, g.scales, plan=plan)
    torch.cuda.synchronize()
    head = plan.buf[:8].cpu().tolist()
    assert head[1] > (batch * 2) // 4          # more items than a quarter of the capacity (2 per token)
    for p in range(4):
        dd = torch.zeros((batch, R), dtype=g.tdt, device=gpu)
        yy = y0[p].clone()
        dispatch_bgmv(dd, g.x, g.key, *t, p, g.scales, plan=False)
        dispatch_bgmv(yy, dd, g.value, *t, p, g.scales, plan=False)
        assert torch.equal(d[p] if p < 3 else do, dd), p
        assert torch.equal(y[p], yy), p
