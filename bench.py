#!/usr/bin/env python3
"""Benchmark of the multi-LoRA batching hot path on one MI355X.

A "step" is one decode step's LoRA work at the S2 shape: for each of 32 layers,
q/k/v/o shrink and expand over the same batch of 256 tokens (200 adapters,
ranks {64,32,16,8}, Zipf(1) adapter popularity), reading adapter pages straight
from the per-layer unified pool.  The base-model matmuls are not part of it.
Inputs are resident in HBM before the timed region starts.

Prints ONE JSON line: LoRA tokens/s for the whole step, the roofline figure of
the dominant kernel (algorithmic bytes per launch / measured launch duration)
and the reference's torch bmm path timed on this box's host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "s-lora_amd"), os.path.join(ROOT, "tests")):  # tests/: the workload builder
    if _p not in sys.path:
        sys.path.insert(0, _p)

METRIC = "LoRA tokens/s + achieved HBM GB/s (% peak), S2 decode BGMV batch 256"
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the dominant kernel, from rocprofv3 counter runs of this
# file (FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter reads for
# a plain 256 MiB copy: 2.000 and 1.000); keyed by (workload, batch, mode, kernel).
# None where not measured.
TRAFFIC_BYTES = {
    ("s2", 256, "planned-fused", "bgmv_expand_kernel<F16, 3, true, 8>"): 81465122,  # 75173666 read + 6291456 written
    ("s2", 256, "planned-fused", "bgmv_shrink_kernel<F16, true, 8>"): 70979806,  # the q/k/v launch
    ("c3", "sgmm_expand_walk_kernel<BF16, 2, 1>"): 281689745,  # 155663826 read + 126025919 written
    ("c3", "sgmm_expand_walk_kernel<BF16, 2, 3>"): 860943997,  # 482866722 read + 378077275 written
    ("c3", "sgmm_shrink_planned_kernel<BF16, 1, false, true>"): 142557796,  # 140588644 read + 1969152 written
    ("c3", "sgmm_shrink_planned_kernel<BF16, 3, false, true>"): 174280962,  # 168373506 read + 5907456 written
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--batch", type=int, default=256)
    ap.add_argument("--workload", choices=["s2", "s4", "s6", "c3", "load", "streaming"], default="s2",
                    help="s2 (the metric's configuration), s4, s6: decode steps; c3: the prefill (segmented) kernels; "
                         "load: copying adapters into the pool; the last two are reported in the same format with "
                         "their own metric names")
    ap.add_argument("--mode", choices=["dropin", "fused", "planned", "planned-fused", "planned-lora"],
                    default="planned-fused",
                    help="dropin: 8 stateless dispatch_bgmv calls per layer exactly as the reference issues them; "
                         "fused: q/k/v shrink and q/k/v expand as one launch each (4 launches per layer); "
                         "planned*: the same with a per-step plan (built inside every timed step) passed as plan=; "
                         "planned-lora: shrink and expand of q/k/v in one launch and of o in one launch (2 per layer)")
    ap.add_argument("--all-modes", action="store_true", help="also time the other modes and report them under 'modes'")
    ap.add_argument("--launch", choices=["graph", "direct"], default="graph",
                    help="graph: the step is captured once into a HIP graph and replayed; direct: Python calls")
    ap.add_argument("--placement", choices=["scattered", "runs"], default="scattered",
                    help="where the adapters' pages lie in the pool -- scattered (the metric's configuration) "
                         "or one contiguous run per adapter (what MemoryAllocator.alloc_adapter asks for)")
    ap.add_argument("--keep-plan", action="store_true",
                    help="planned modes: build the plan once with its item count read back and do not rebuild it "
                         "inside the step (launches sized exactly; only right while the batch stays the same)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="leave out the 'modes' (reference call pattern, direct launches) and 'prefill_c3' blocks "
                         "that the default S2 run adds to its line")
    ap.add_argument("--cpu-reps", type=int, default=0, help="0 = as many as fit in about 15 s")
    ap.add_argument("--check", action="store_true", help="verify layer 0 against the oracle before timing")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain device copy of 256 MiB (read) + 256 MiB (write) so that a "
                         "counter run (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE) sees a kernel of known traffic")
    return ap.parse_args()


class StepBuffers:
    """Activations and outputs of every layer, distinct per layer so that no
    call finds its operands cached by the previous layer."""

    def __init__(self, w, device):
        import torch
        g = torch.Generator(device=device)
        g.manual_seed(123)
        B, H = w.batch, w.hidden
        self.x_in = [torch.randn((B, H), generator=g, device=device, dtype=torch.float32).to(w.dtype)
                     for _ in range(w.n_layers)]
        self.x_att = [torch.randn((B, H), generator=g, device=device, dtype=torch.float32).to(w.dtype)
                      for _ in range(w.n_layers)]
        self.y = [[torch.zeros((B, h), device=device, dtype=w.dtype) for h in w.h_out] for _ in range(w.n_layers)]
        self.delta = [torch.zeros((B, w.max_rank), device=device, dtype=w.dtype) for _ in range(3)]


def make_step(w, bufs, mode, keep_plan=False):
    """Returns (step, families).  `families` maps a label to (sweep, kernel
    name, launches per sweep, algorithmic bytes per launch): one sweep per kind
    of launch the step issues, over all layers, so that each kind's launch
    duration can be timed by itself.  With a planned mode the plan is rebuilt
    inside every step (one extra small launch, as a caller would do once per
    decode step); its item count was read back once when the plan was first
    made -- the synchronisation a caller pays per step, like the reference's own
    ``.item()`` at lora_unordered_batch_infer.py:64."""
    import torch
    import slora_hip
    bgmv = slora_hip.dispatch_bgmv
    t = (w.a_start, w.a_len, w.a_loc, w.req_bins)
    planned = mode.startswith("planned")
    one_launch = mode == "planned-lora"
    fused = mode.endswith("fused") or one_launch
    plan = slora_hip.make_plan(*t, w.max_rank, w.n_pages) if planned else None
    kw = {"plan": plan} if planned else {}
    L = w.n_layers
    ty = "F16" if w.dtype == torch.float16 else "BF16"
    pl = "true" if planned else "false"

    def qkv_shrink(l):
        slora_hip.dispatch_bgmv_qkv_shrink(bufs.delta[0], bufs.delta[1], bufs.delta[2], bufs.x_in[l],
                                           w.key_buffer[l], *t, **kw)

    def qkv_expand(l):
        slora_hip.dispatch_bgmv_qkv_expand(bufs.y[l][0], bufs.y[l][1], bufs.y[l][2], bufs.delta[0], bufs.delta[1],
                                           bufs.delta[2], w.value_buffer[l], *t, w.a_scaling, **kw)

    def shrink(l, p):
        bgmv(bufs.delta[p % 3], bufs.x_in[l] if p < 3 else bufs.x_att[l], w.key_buffer[l], *t, p, w.a_scaling, **kw)

    def expand(l, p):
        bgmv(bufs.y[l][p], bufs.delta[p % 3], w.value_buffer[l], *t, p, w.a_scaling, **kw)

    def qkv_lora(l):
        slora_hip.dispatch_bgmv_qkv_lora(bufs.y[l][0], bufs.y[l][1], bufs.y[l][2], bufs.delta[0], bufs.delta[1],
                                         bufs.delta[2], bufs.x_in[l], w.key_buffer[l], w.value_buffer[l], *t,
                                         w.a_scaling, **kw)

    def o_lora(l):
        slora_hip.dispatch_bgmv_lora(bufs.y[l][3], bufs.delta[0], bufs.x_att[l], w.key_buffer[l], w.value_buffer[l], *t,
                                     3, w.a_scaling, **kw)

    def over_layers(fn, *a):
        def sweep():
            for l in range(L):
                fn(l, *a)
        return sweep

    def all_proj(fn):
        def sweep():
            for l in range(L):
                for p in range(4):
                    fn(l, p)
        return sweep

    nv = next((n for n in (8, 10, 12, 16) if w.hidden <= 512 * n), 8)  # the instantiation the library picks
    nv_e = nv if planned else 8   # the stateless expand keeps the 4096-element pass
    sk, ek = f"bgmv_shrink_kernel<{ty}, {pl}, {nv}>", f"bgmv_expand_kernel<{ty}, %d, {pl}, {nv_e}>"
    if one_launch:
        lk = f"bgmv_lora_kernel<{ty}, %d, {nv}>"
        families = {
            "qkv_lora": (over_layers(qkv_lora), lk % 3, L, w.qkv_shrink_bytes() + w.qkv_expand_bytes()),
            "o_lora": (over_layers(o_lora), lk % 1, L, w.shrink_bytes() + w.expand_bytes(w.h_out[3])),
        }
    elif fused:
        families = {
            "qkv_shrink": (over_layers(qkv_shrink), sk, L, w.qkv_shrink_bytes()),
            "o_shrink": (over_layers(shrink, 3), sk, L, w.shrink_bytes()),
            "qkv_expand": (over_layers(qkv_expand), ek % 3, L, w.qkv_expand_bytes()),
            "o_expand": (over_layers(expand, 3), ek % 1, L, w.expand_bytes(w.h_out[3])),
        }
    else:
        families = {
            "shrink": (all_proj(shrink), sk, 4 * L, w.shrink_bytes()),
            "expand": (all_proj(expand), ek % 1, 4 * L, sum(w.expand_bytes(h) for h in w.h_out) / 4),
        }

    def step():
        if planned and not keep_plan:
            slora_hip.rebuild_plan(plan, *t, w.n_pages)
        else:
            # a new batch every step: calls that pass no plan may reuse one only within the step
            slora_hip.clear_plan_cache()
        for l in range(L):
            if one_launch:
                qkv_lora(l)
                o_lora(l)
                continue
            if fused:
                qkv_shrink(l)
                qkv_expand(l)
            else:
                # call order of lora_unordered_batch_infer.py:254-318
                for p in range(3):
                    shrink(l, p)
                    expand(l, p)
            # o projection, lora_unordered_batch_infer.py:428-448
            shrink(l, 3)
            expand(l, 3)

    return step, families


def graphed(fn, torch):
    """Capture fn once on a side stream and return a replay callable."""
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        fn()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    return g.replay


def time_region(fn, reps, warmup, torch):
    """HIP events on the stream the kernels are enqueued on; returns ms per rep."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def check_layer0(w, bufs, torch):
    """Layer 0, all four projections, every token, against the oracle (the
    adapter pages of layer 0 are copied to the host for it)."""
    import numpy as np
    import slora_hip
    from oracle import lora_oracle as O
    dt = "f16" if w.dtype == torch.float16 else "bf16"
    used = np.unique(w.a_loc_np)
    remap = np.full(w.n_pages, -1, dtype=np.int64)
    remap[used] = np.arange(used.size)
    idx = torch.from_numpy(used).to(w.key_buffer[0].device)
    key = w.key_buffer[0][idx].reshape(used.size, -1).float().cpu().numpy()
    val = w.value_buffer[0][idx].reshape(used.size, -1).float().cpu().numpy()
    loc = remap[w.a_loc_np]
    t = (w.a_start, w.a_len, w.a_loc, w.req_bins)
    for p in range(4):
        x = bufs.x_in[0] if p < 3 else bufs.x_att[0]
        delta = torch.zeros_like(bufs.delta[0])
        y = torch.zeros_like(bufs.y[0][p])
        slora_hip.dispatch_bgmv(delta, x, w.key_buffer[0], *t, p, w.a_scaling)
        slora_hip.dispatch_bgmv(y, delta, w.value_buffer[0], *t, p, w.a_scaling)
        torch.cuda.synchronize()
        d_gpu = delta.float().cpu().numpy()
        d_ref = O.ref_bgmv_shrink(np.zeros_like(d_gpu), x.float().cpu().numpy(), key, w.a_start_np, w.a_len_np, loc,
                                  w.bins_np, p, dt)
        np.testing.assert_allclose(d_gpu, d_ref, rtol=1e-2, atol=1e-3)
        y_ref = O.ref_bgmv_expand(np.zeros((w.batch, w.h_out[p]), np.float32), d_gpu, val, w.a_start_np, w.a_len_np,
                                  loc, w.bins_np, p, w.a_scaling.float().cpu().numpy(), dt)
        np.testing.assert_allclose(y.float().cpu().numpy(), y_ref, rtol=1e-2, atol=1e-3)


def cpu_baseline(w, bufs, torch, reps_arg):
    """The reference's bmm path (gather, zero-padded bmm, scatter-add) in torch
    float32 on this box's host cores, on ONE layer of the same workload."""
    import numpy as np
    from oracle import lora_oracle as O
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(os.cpu_count() or 1, 16)
    u = w.distinct_adapters()
    dev = w.key_buffer[0].device
    A, B, scal = [], [], []
    for a in u:
        r = int(w.ranks[a])
        loc = w.a_loc_np[w.a_start_np[a]: w.a_start_np[a] + 4 * r]
        idx = torch.from_numpy(loc).to(dev)
        kp = w.key_buffer[0][idx].reshape(4 * r, -1).float().cpu().numpy()
        vp = w.value_buffer[0][idx].reshape(4 * r, -1).float().cpu().numpy()
        a_p, b_p = O.unpack_from_pool(kp, vp, np.arange(4 * r), w.hidden, w.h_out)
        A.append(a_p)
        B.append(b_p)
        scal.append(float(w.scales_np[a]))
    remap = {int(a): i for i, a in enumerate(u)}
    bins = np.array([remap[int(b)] for b in w.bins_np])
    layer = O.BmmCpuLayer(A, B, scal, bins, threads=threads)
    x_in = bufs.x_in[0].float().cpu()
    x_att = bufs.x_att[0].float().cpu()
    ys = [torch.zeros((w.batch, h), dtype=torch.float32) for h in w.h_out]
    layer.decode(x_in, x_att, ys)  # warm-up
    t0 = time.perf_counter()
    layer.decode(x_in, x_att, ys)
    one = time.perf_counter() - t0
    reps = reps_arg or max(3, min(30, int(15.0 / max(one, 1e-3))))
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        layer.decode(x_in, x_att, ys)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return {
        "value": round(w.batch / (med * w.n_layers), 1),
        "unit": "tokens/s",
        "cores": threads,
        "kind": "port",
        "sample": f"1 of {w.n_layers} layers (q/k/v/o gather + padded torch.bmm o bmm + scatter-add, fp32, "
                  f"{u.size} adapters in batch), median of {reps} reps = {med * 1e3:.1f} ms/layer; "
                  f"step time extrapolated x{w.n_layers}",
        "gbps_algorithmic": round(w.layer_bytes() / med / 1e9, 2),
    }


def cpu_baseline_c1(torch):
    """Configuration 1 exactly: the reference's bmm path on the host cores, float32, hidden 4096,
    8 adapters of rank 8, 32 tokens with adapter ids uniform in [0, 8), x ~ N(0,1),
    A ~ N(0, 1/4096), B ~ N(0, 1/8), scaling 2.0, one layer of q/k/v/o."""
    import numpy as np
    from oracle import lora_oracle as O
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(os.cpu_count() or 1, 16)
    rng = np.random.default_rng(1)
    H, r, n_ad, batch = 4096, 8, 8, 32
    A = [[(rng.standard_normal((H, r)) / np.sqrt(H)).astype(np.float32) for _ in range(4)] for _ in range(n_ad)]
    B = [[(rng.standard_normal((r, H)) / np.sqrt(r)).astype(np.float32) for _ in range(4)] for _ in range(n_ad)]
    bins = rng.integers(0, n_ad, size=batch)
    layer = O.BmmCpuLayer(A, B, [2.0] * n_ad, bins, threads=threads)
    x_in = torch.from_numpy(rng.standard_normal((batch, H)).astype(np.float32))
    x_att = torch.from_numpy(rng.standard_normal((batch, H)).astype(np.float32))
    ys = [torch.zeros((batch, H), dtype=torch.float32) for _ in range(4)]
    for _ in range(5):
        layer.decode(x_in, x_att, ys)
    times = []
    for _ in range(30):
        t0 = time.perf_counter()
        layer.decode(x_in, x_att, ys)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    # algorithmic bytes of the layer with 4-byte elements: distinct adapters' A and B, x, delta, y read + written
    u = np.unique(bins).size
    nbytes = 4 * (u * r * H * 4 + batch * H * 4 + batch * r * 4) + 4 * (u * r * H * 4 + batch * r * 4 + 2 * batch * H * 4)
    return {"value": round(batch / med, 1), "unit": "tokens/s per layer", "cores": threads, "kind": "port",
            "sample": f"one layer of q/k/v/o, fp32, {n_ad} adapters of rank {r}, batch {batch}, median of 30 reps = "
                      f"{med * 1e3:.3f} ms/layer (5 warm-up)",
            "gbps_algorithmic": round(nbytes / med / 1e9, 2)}


MFMA_PEAK_TFLOPS = 2500.0


def measure_dropin_direct(w, bufs, torch, args):
    """What an unmodified caller of the reference's engine gets: its call pattern (8
    stateless-looking dispatch_bgmv calls per layer, new index tensor every step), issued as
    plain Python calls into the extension, no graph, no plan argument -- the library keeps
    the plan of the step by itself.  Wall clock around K steps (the launches are asynchronous,
    so this is the larger of host issue time and device time), and the host cost of one call
    measured on a one-token batch whose kernels the device finishes faster than they are
    issued."""
    import slora_hip
    t = (w.a_start, w.a_len, w.a_loc)
    L = w.n_layers

    def step():
        bins = w.req_bins.clone()  # the engine builds req_bins anew for every step (lora_unordered_batch_infer.py:24)
        for l in range(L):
            for p in range(3):
                slora_hip.dispatch_bgmv(bufs.delta[p], bufs.x_in[l], w.key_buffer[l], *t, bins, p, w.a_scaling)
                slora_hip.dispatch_bgmv(bufs.y[l][p], bufs.delta[p], w.value_buffer[l], *t, bins, p, w.a_scaling)
            slora_hip.dispatch_bgmv(bufs.delta[0], bufs.x_att[l], w.key_buffer[l], *t, bins, 3, w.a_scaling)
            slora_hip.dispatch_bgmv(bufs.y[l][3], bufs.delta[0], w.value_buffer[l], *t, bins, 3, w.a_scaling)

    def wall_ms(fn, n, warm):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / n

    ms = wall_ms(step, max(5, args.steps // 2), 3)
    # host cost of a call: one token, so the device is never the bottleneck
    one = torch.zeros(1, dtype=torch.int64, device=w.req_bins.device)
    x1, d1 = bufs.x_in[0][:1], bufs.delta[0][:1]

    def calls():
        for _ in range(1000):
            slora_hip.dispatch_bgmv(d1, x1, w.key_buffer[0], *t, one, 0, w.a_scaling)

    host_us = wall_ms(calls, 3, 1)  # ms per 1000 calls = us per call

    # the same step through the engine class: one object per step (as model_rpc.py:234 builds it),
    # q/k/v in one shrink and one expand launch, o as two calls
    from types import SimpleNamespace
    dirs = [f"adapter-{i}" for i in range(len(w.ranks))]
    ia = SimpleNamespace(a_start=w.a_start, a_len=w.a_len, a_loc=w.a_loc, a_scaling=w.a_scaling, adapter_dirs=dirs,
                         idx_map={d: i for i, d in enumerate(dirs)},
                         mem_manager=SimpleNamespace(key_buffer=w.key_buffer, value_buffer=w.value_buffer))
    reqs = [SimpleNamespace(lora_dir=dirs[a], r=int(w.ranks[a])) for a in w.bins_np]
    b_start = torch.zeros(w.batch, dtype=torch.int32, device=w.req_bins.device)
    b_len = torch.full((w.batch,), 100, dtype=torch.int32, device=w.req_bins.device)

    def engine_step():
        eng = slora_hip.LoraUnorderedBatchInfer(ia, reqs, fused=True)
        eng.begin_step(b_start, b_len, is_prefill=False, max_b_seq_len=100)
        for l in range(L):
            eng.lora_get_qkv(l, bufs.x_in[l], bufs.y[l][0], bufs.y[l][1], bufs.y[l][2])
            eng.lora_get_o(l, bufs.x_att[l], bufs.y[l][3])

    ms_eng = wall_ms(engine_step, max(5, args.steps // 2), 3)
    return {"engine-fused-direct": {
        "what": "LoraUnorderedBatchInfer(fused=True) built anew every step: q/k/v in one shrink and one expand "
                "launch per layer, direct launches from Python, plan built and reused by the library",
        "ms_per_step": round(ms_eng, 4), "tokens_per_s": round(w.batch / (ms_eng * 1e-3), 1),
        "launches_per_step": 4 * L + 2},
        "dropin-direct-autoplan": {
        "what": "reference call pattern (8 dispatch_bgmv per layer, new req_bins per step), direct launches from "
                "Python through the extension, plan built and reused by the library",
        "ms_per_step": round(ms, 4), "tokens_per_s": round(w.batch / (ms * 1e-3), 1), "launches_per_step": 8 * L + 2,
        "host_us_per_call": round(host_us, 2)}}


def measure_other_shapes(w, bufs, torch):
    """The decode step at the S4 and S6 shapes (a few layers each), each in a child process of
    its own once this process has given its pools back: what the same kernels reach when a
    launch moves hundreds of megabytes instead of tens."""
    import subprocess
    free_workload(w, bufs, torch)
    res = {}
    for wl, layers in (("s4", 8), ("s6", 8)):
        cmd = [sys.executable, os.path.abspath(__file__), "--workload", wl, "--layers", str(layers), "--steps", "10",
               "--warmup", "3", "--no-cpu-baseline", "--no-extras"]
        try:
            proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True, timeout=300)
            d = json.loads([l for l in proc.stdout.splitlines() if l.startswith("{")][-1])
            res[wl] = {"workload": d["config"]["workload"], "layers": d["config"]["layers"],
                       "ms_per_step": d["ms_per_step"], "tokens_per_s": d["value"], "step_hbm": d["step_hbm"],
                       "pool_GB": round(2 * d["config"]["layers"] * d["config"]["pool_pages_per_layer"] *
                                        d["config"]["page_bytes"] / 1e9, 1),
                       "kernels": {k: {"us_per_launch": v["us_per_launch"], "frac": v["frac"],
                                       "kernel_over_ceiling": v.get("read_only_ceiling", {}).get("kernel_over_ceiling")}
                                   for k, v in d["kernels"].items()}}
        except Exception as e:  # the headline line is printed whatever happens here
            res[wl] = {"error": f"{type(e).__name__}: {e}"}
    return res


def free_workload(w, bufs, torch):
    """Give the decode pools back before another workload is built."""
    w.key_buffer.clear()
    w.value_buffer.clear()
    for name in ("x_in", "x_att", "y", "delta"):
        getattr(bufs, name).clear()
    torch.cuda.empty_cache()


def measure_prefill(args, torch, device, w=None, seg=None):
    """q/k/v/o segmented shrink and expand over a prefill batch, per layer (C3 unless a pool
    workload and its requests are passed).  Returns the JSON object of the prefill workload."""
    import slora_hip
    import workloads
    L = min(args.layers, 4)
    if w is None:
        w, seg = workloads.c3_prefill(device, n_layers=L)
    T, H, R = seg.n_tokens, w.hidden, w.max_rank
    g = torch.Generator(device=device)
    g.manual_seed(7)
    x = [torch.randn((T, H), generator=g, device=device, dtype=torch.float32).to(w.dtype) for _ in range(L)]
    y = [torch.zeros((T, H), device=device, dtype=w.dtype) for _ in range(L)]
    d = torch.zeros((T, R), device=device, dtype=w.dtype)
    ty = "F16" if w.dtype == torch.float16 else "BF16"
    ks = 1 if R <= 32 else (2 if R <= 64 else 4)
    d3 = [torch.zeros((T, R), device=device, dtype=w.dtype) for _ in range(3)]
    y3 = [[torch.zeros((T, H), device=device, dtype=w.dtype) for _ in range(3)] for _ in range(L)]  # q, k, v outputs
    t = (w.a_loc, w.a_start, w.a_len, seg.b_start_loc, seg.b_seq_len, seg.b_indicies)

    def plan():  # once per prefill step, as the automatic cache does for a caller that passes none
        return slora_hip.make_prefill_plan(w.a_start, w.a_len, seg.b_start_loc, seg.b_seq_len, seg.b_indicies, T, R,
                                           seg.max_len)

    def shrink_sweep():
        pl = plan()
        for l in range(L):
            for p in range(4):
                slora_hip.lora_get_qkvo_fwd_shrink(x[l], w.key_buffer[l].view(-1, H), d, *t, H, p, R, seg.max_len,
                                                   plan=pl)

    def qkv_shrink_sweep():  # 4 launches per layer keep the per-launch arithmetic below the same
        pl = plan()
        for l in range(L):
            for _ in range(4):
                slora_hip.lora_get_qkvo_fwd_shrink_qkv(x[l], w.key_buffer[l].view(-1, H), *d3, *t, H, R, seg.max_len,
                                                       plan=pl)

    def expand_sweep():
        for l in range(L):
            for p in range(4):
                slora_hip.lora_get_qkvo_fwd_expand(d, w.value_buffer[l].view(-1, H), y[l], w.a_scaling, *t, H, p, R,
                                                   seg.max_len)

    def qkv_expand_sweep():
        for l in range(L):
            for _ in range(4):
                slora_hip.lora_get_qkvo_fwd_expand_qkv(*d3, w.value_buffer[l].view(-1, H), *y3[l], w.a_scaling, *t, H, H,
                                                       R, seg.max_len)

    def step_fused():  # q, k and v in one shrink launch (x read once) and one expand launch: 4 launches per layer
        pl = plan()
        for l in range(L):
            key, val = w.key_buffer[l].view(-1, H), w.value_buffer[l].view(-1, H)
            slora_hip.lora_get_qkvo_fwd_shrink_qkv(x[l], key, *d3, *t, H, R, seg.max_len, plan=pl)
            slora_hip.lora_get_qkvo_fwd_expand_qkv(*d3, val, *y3[l], w.a_scaling, *t, H, H, R, seg.max_len)
            slora_hip.lora_get_qkvo_fwd_shrink(x[l], key, d, *t, H, 3, R, seg.max_len, plan=pl)
            slora_hip.lora_get_qkvo_fwd_expand(d, val, y[l], w.a_scaling, *t, H, 3, R, seg.max_len)

    def step():
        pl = plan()
        for l in range(L):
            for p in range(4):
                slora_hip.lora_get_qkvo_fwd_shrink(x[l], w.key_buffer[l].view(-1, H), d, *t, H, p, R, seg.max_len,
                                                   plan=pl)
                slora_hip.lora_get_qkvo_fwd_expand(d, w.value_buffer[l].view(-1, H), y[l], w.a_scaling, *t, H, p, R,
                                                   seg.max_len)

    use_graph = args.launch == "graph"
    wrap = (lambda f: graphed(f, torch)) if use_graph else (lambda f: f)
    reps = max(5, args.steps)
    ms_step = time_region(wrap(step), reps, args.warmup, torch)
    ms_step_fused = time_region(wrap(step_fused), reps, args.warmup, torch)
    kernels = {}
    flops1 = seg.flops(w, H)
    ring = "true" if T > 4096 and H % 64 == 0 else "false"   # the instantiation that streams through LDS
    for label, sweep, kname, nbytes, flops in (
            ("shrink", shrink_sweep, f"sgmm_shrink_planned_kernel<{ty}, 1, {'true' if T <= 4096 else 'false'}, {ring}>",
             seg.shrink_bytes(w), flops1),
            ("qkv_shrink", qkv_shrink_sweep, f"sgmm_shrink_planned_kernel<{ty}, 3, false, {ring}>",
             3 * seg.shrink_bytes(w) - 2 * T * H * 2, 3 * flops1),
            ("expand", expand_sweep, f"sgmm_expand_walk_kernel<{ty}, {ks}, 1>", seg.expand_bytes(w, H), flops1),
            ("qkv_expand", qkv_expand_sweep, f"sgmm_expand_walk_kernel<{ty}, {ks}, 3>", 3 * seg.expand_bytes(w, H),
             3 * flops1)):
        us = time_region(wrap(sweep), reps, 3, torch) * 1e3 / (4 * L)
        kernels[label] = {"kernel": kname, "launches_per_step": 4 * L, "us_per_launch": round(us, 3),
                          "bytes_per_launch": nbytes, "GBps": round(nbytes / us / 1e3, 1),
                          "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                          "TFLOPs": round(flops / us / 1e6, 1),
                          "frac_mfma": round(flops / us / 1e6 / MFMA_PEAK_TFLOPS, 4),
                          "traffic": TRAFFIC_BYTES.get(("c3", kname))}
    # Floors of the access patterns, from the two plain page kernels (one wavefront per 8 KiB row, nothing but
    # the accesses): the shrink reads x and the weight rows of the adapters in the batch; the expand reads and
    # writes y (its delta and B^T reads, 5 % of its bytes, are not in the floor).
    import numpy as np
    from slora_hip.infer_adapter import page_checksums, page_xor
    rows = torch.arange(T, dtype=torch.int64, device=device)
    u = np.unique(seg.ids_np)
    a_pages = torch.from_numpy(w.a_loc_np[np.concatenate(
        [w.a_start_np[a] + 3 * w.ranks[a] + np.arange(int(w.ranks[a])) for a in u])]).to(device)

    def read_sweep():
        for l in range(L):
            for _ in range(4):
                page_checksums(x[l], rows)
                page_checksums(w.key_buffer[l], a_pages)

    def rmw_sweep():
        for l in range(L):
            for _ in range(4):
                page_xor(y[l], rows, 0)

    us_read = time_region(wrap(read_sweep), reps, 3, torch) * 1e3 / (4 * L)
    us_rmw = time_region(wrap(rmw_sweep), reps, 3, torch) * 1e3 / (4 * L)
    nb_read = T * H * 2 + int(a_pages.numel()) * w.page_elems * 2
    kernels["shrink"]["read_only_ceiling"] = {
        "what": "x rows and one projection's weight rows, loads only (two launches)", "us": round(us_read, 3),
        "bytes": nb_read, "GBps": round(nb_read / us_read / 1e3, 1),
        "kernel_over_ceiling": round(kernels["shrink"]["us_per_launch"] / us_read, 3)}
    kernels["qkv_shrink"]["read_only_ceiling"] = {
        "what": "the same floor: the fused launch reads x once", "us": round(us_read, 3),
        "kernel_over_ceiling": round(kernels["qkv_shrink"]["us_per_launch"] / us_read, 3)}
    kernels["expand"]["rmw_ceiling"] = {
        "what": "y rows read and written in place, nothing else", "us": round(us_rmw, 3), "bytes": 2 * T * H * 2,
        "GBps": round(2 * T * H * 2 / us_rmw / 1e3, 1),
        "kernel_over_ceiling": round(kernels["expand"]["us_per_launch"] / us_rmw, 3)}
    kernels["qkv_expand"]["rmw_ceiling"] = {
        "what": "three times the single projection's floor", "us": round(3 * us_rmw, 3),
        "kernel_over_ceiling": round(kernels["qkv_expand"]["us_per_launch"] / (3 * us_rmw), 3)}
    dom = max((k for n, k in kernels.items() if not n.startswith("qkv_")), key=lambda k: k["us_per_launch"])
    out = {
        "metric": "LoRA prefill tokens/s + achieved HBM GB/s (% peak), C3 segmented shrink/expand",
        "value": round(T / (ms_step * 1e-3 / L), 1),
        "unit": "tokens/s per layer",
        "n_gpus": 1, "steps": reps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16" if w.dtype == torch.float16 else "bf16", "data": "synthetic",
        "config": {"workload": w.name, "layers": L, "tokens": T, "requests": int(seg.lens_np.size),
                   "launch": args.launch, "launches_per_step": 8 * L + 1},
        "ms_per_step_qkv_fused": round(ms_step_fused, 4),
        "roofline": {"kernel": dom["kernel"], "bound": "hbm", "achieved": dom["GBps"], "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": dom["frac"], "traffic": TRAFFIC_BYTES.get(("c3", dom["kernel"])),
                     "algorithmic_bytes_per_launch": dom["bytes_per_launch"], "us_per_launch": dom["us_per_launch"]},
        "kernels": kernels,
    }
    return out


def main_load(args, torch, device):
    """Loading rank-64 adapters into the pools of 32 layers: for every adapter one
    call scatters its 256 rows of 8 KiB into the key and value buffer of every
    layer (64 buffers), as InferAdapter.load_lora_A/B do with 64 index_puts."""
    import numpy as np
    from slora_hip.infer_adapter import load_rows_into_pool
    L, H, r, n_pages, n_adapters = min(args.layers, 32), 4096, 64, 16384, 8
    bufs = [torch.zeros((n_pages, 32, H // 32), dtype=torch.float16, device=device) for _ in range(2 * L)]
    rows = [[torch.randn((4 * r, 32, H // 32), device=device, dtype=torch.float32).to(torch.float16)
             for _ in range(2 * L)] for _ in range(n_adapters)]
    perm = np.random.default_rng(0).permutation(n_pages)
    locs = [torch.from_numpy(perm[i * 4 * r:(i + 1) * 4 * r].astype(np.int64)).to(device) for i in range(n_adapters)]

    def step():
        for a in range(n_adapters):
            load_rows_into_pool(bufs, rows[a], locs[a])

    def torch_step():
        for a in range(n_adapters):
            for b in range(2 * L):
                bufs[b][locs[a]] = rows[a][b]

    use_graph = args.launch == "graph"
    ms = time_region(graphed(step, torch) if use_graph else step, max(5, args.steps), args.warmup, torch)
    ms_torch = time_region(graphed(torch_step, torch) if use_graph else torch_step, max(5, args.steps), args.warmup,
                           torch)
    # the allocator call that precedes a load: 256 pages out of a 65536-page map (and back)
    from slora_hip.infer_adapter import PageAllocator
    pa = PageAllocator(65536, device)
    pa.alloc(30000)  # a used prefix, as after some uptime
    state = pa.mem_state.clone()
    cum = torch.empty(65536, dtype=torch.int32, device=device)
    idx = torch.arange(65536, dtype=torch.long, device=device)

    def alloc_free():
        pa.free(pa.alloc(4 * r))

    def torch_alloc_free():  # mem_allocator.py:34-38, 196
        torch.cumsum(state, dim=0, dtype=torch.int32, out=cum)
        sel = idx[torch.logical_and(cum <= 4 * r, state == 1)]
        state[sel] = 0
        state[sel] = 1

    def host_us(fn, n=200):
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e6

    alloc_us, torch_alloc_us = host_us(alloc_free), host_us(torch_alloc_free)

    # merging one rank-64 adapter into the four [H, H] base matrices of a layer and taking it out again
    from slora_hip.infer_adapter import merge_adapter, unmerge_adapter
    a_start = torch.zeros(1, dtype=torch.int64, device=device)
    a_len = torch.full((1,), 4 * r, dtype=torch.int64, device=device)
    a_scal = torch.full((1,), 0.25, dtype=torch.float16, device=device)
    n_w = 4
    weights = [[torch.randn((H, H), device=device, dtype=torch.float32).to(torch.float16) for _ in range(4)]
               for _ in range(n_w)]

    def merge_unmerge():
        for l in range(n_w):
            merge_adapter(weights[l], bufs[l], bufs[L + l], a_start, a_len, locs[0], a_scal, 0)
            unmerge_adapter(weights[l], bufs[l], bufs[L + l], a_start, a_len, locs[0], a_scal, 0)

    merge_ms = time_region(merge_unmerge, 5, 2, torch) / (2 * n_w)
    merge_bytes = 4 * (2 * H * H * 2 + 2 * r * H * 2)
    nbytes = 2 * (4 * r) * H * 2 * 2 * L  # read + write per adapter
    us = ms * 1e3 / n_adapters
    gbs = nbytes / us / 1e3
    out = {
        "metric": "adapter load into the unified pool, GB/s moved (read + write)",
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": max(5, args.steps), "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "config": {"workload": f"{n_adapters} adapters of rank {r}, hidden {H}, {L} layers, key + value buffers",
                   "launch": args.launch, "launches_per_step": n_adapters},
        "roofline": {"kernel": "pool_scatter_kernel", "bound": "hbm", "achieved": round(gbs, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "algorithmic_bytes_per_launch": nbytes, "us_per_launch": round(us, 3)},
        "torch_index_put": {"us_per_adapter": round(ms_torch * 1e3 / n_adapters, 3),
                            "launches_per_adapter": 2 * L},
        "merge_adapter": {"what": "rank-64 adapter into q, k, v, o [4096, 4096] of one layer (4 gathers + 4 launches)",
                          "us_per_layer": round(merge_ms * 1e3, 1), "bytes_per_layer": merge_bytes,
                          "GBps": round(merge_bytes / merge_ms / 1e6, 1),
                          "frac": round(merge_bytes / merge_ms / 1e6 / HBM_PEAK_GBS, 4)},
        "allocator": {"what": "alloc(256) + free on a 65536-page map, wall time per pair incl. Python",
                      "us": round(alloc_us, 1), "torch_ops_us": round(torch_alloc_us, 1)},
    }
    print(json.dumps(out), flush=True)


def main_streaming(args, torch, device):
    """What plain reads of pool pages reach on this chip, with the library's own checksum kernel
    (one wavefront per 8 KiB page, loads only; four pages per workgroup, consecutive workgroups
    on consecutive XCDs): launches of several sizes over scattered pages (the fit t = t0 + bytes /
    rate is the ceiling the decode launches are held against), one pool against one pool per
    launch, and pages that are read twice -- by the same workgroup, by another workgroup of the
    same XCD, by a workgroup of another XCD."""
    import numpy as np
    from slora_hip.infer_adapter import page_checksums
    L, n_pages, page_elems = min(args.layers, 32), 65536, 4096
    pools = [torch.zeros((n_pages, page_elems), dtype=torch.float16, device=device) for _ in range(L)]
    rng = np.random.default_rng(0)
    use_graph = args.launch == "graph"

    def dev(a):
        return torch.from_numpy(np.ascontiguousarray(a).astype(np.int64)).to(device)

    def timed(lists, pool_of):
        def sweep():
            for l in range(L):
                page_checksums(pools[pool_of(l)], lists[l % len(lists)])
        fn = graphed(sweep, torch) if use_graph else sweep
        return time_region(fn, max(5, args.steps // 2), 3, torch) * 1e3 / L

    def repeated(b, times, apart):
        # blocks of `apart` entries, each block `times` times in a row: the copies of a page are `apart` entries apart
        blocks = b[: len(b) // apart * apart].reshape(-1, apart)
        return np.repeat(blocks[:, None, :], times, axis=1).reshape(-1)

    page_bytes = page_elems * 2
    sizes = {}
    for n in (3072, 7944, 9728, 18432):   # 25, 65, 80, 151 MB per launch
        lists = [dev(rng.permutation(n_pages)[:n]) for _ in range(4)]
        us = timed(lists, lambda l: l)
        sizes[n] = us
    ns = np.array(sorted(sizes)); ts = np.array([sizes[n] for n in ns])
    slope, t0 = np.polyfit(ns * page_bytes, ts, 1)      # us per byte, us
    K = 7944
    base = [rng.permutation(n_pages)[:K] for _ in range(4)]
    uniq = [dev(b) for b in base]
    rows = {
        "one pool per launch (%d pools in turn)" % L: (K, timed(uniq, lambda l: l)),
        "one pool for every launch": (K, timed(uniq, lambda l: 0)),
        "the same pages in every launch (65 MB, warm in the 256 MB Infinity Cache)": (K, timed(uniq[:1], lambda l: 0)),
        "the same pages in every second launch": (K, timed(uniq[:2], lambda l: 0)),
        "each page twice, same workgroup": (2 * K, timed([dev(repeated(b, 2, 1)) for b in base], lambda l: l)),
        "each page twice, next workgroup of the same XCD": (2 * (K // 32 * 32),
                                                            timed([dev(repeated(b, 2, 32)) for b in base], lambda l: l)),
        "each page twice, next workgroup (another XCD)": (2 * K, timed([dev(repeated(b, 2, 4)) for b in base], lambda l: l)),
        "twice as many different pages": (2 * K, timed([dev(rng.permutation(n_pages)[:2 * K]) for _ in range(4)],
                                                       lambda l: l)),
    }
    rate = 1.0 / slope / 1e3   # GB/s
    out = {
        "metric": "read-only streaming of scattered pool pages, asymptotic GB/s",
        "value": round(rate, 1), "unit": "GB/s", "n_gpus": 1, "steps": max(5, args.steps // 2), "warmup": 3,
        "ms_per_step": round(sizes[7944] * L * 1e-3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": f"page checksums over {L} pools of {n_pages} pages of {page_bytes} bytes",
                   "launch": args.launch},
        "roofline": {"kernel": "page_xor_kernel", "bound": "hbm", "achieved": round(rate, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(rate / HBM_PEAK_GBS, 4), "traffic": None},
        "launch_sizes": {"us_per_launch_by_pages": {str(n): round(sizes[n], 3) for n in ns},
                         "fit": {"fixed_us": round(float(t0), 3), "GBps": round(rate, 1)}},
        "reads_of_%d_pages" % K: {k: {"page_reads": n, "us_per_launch": round(us, 3),
                                      "GBps_of_page_reads": round(n * page_bytes / us / 1e3, 1)}
                                  for k, (n, us) in rows.items()},
    }
    print(json.dumps(out), flush=True)


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the LoRA path has no cross-GPU part); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    import slora_hip
    import workloads
    slora_hip.load_library()
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.calibrate_copy:
        src = torch.ones(128 * 1024 * 1024, dtype=torch.float16, device=device)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if args.workload == "c3":
        print(json.dumps(measure_prefill(args, torch, device)), flush=True)
        return
    if args.workload == "load":
        main_load(args, torch, device)
        return
    if args.workload == "streaming":
        main_streaming(args, torch, device)
        return
    if args.workload == "s2":
        w = workloads.s2_decode(device, n_layers=args.layers, batch=args.batch, placement=args.placement)
    elif args.workload == "s4":
        w = workloads.s4_decode(device, n_layers=args.layers, batch=args.batch if args.batch != 256 else 512,
                                placement=args.placement)
    else:
        w = workloads.s6_decode(device, n_layers=min(args.layers, 8), batch=args.batch if args.batch != 256 else 1024,
                                placement=args.placement)
    bufs = StepBuffers(w, device)
    step, families = make_step(w, bufs, args.mode, args.keep_plan)
    fused = args.mode.endswith("fused") or args.mode == "planned-lora"
    if args.check:
        check_layer0(w, bufs, torch)

    use_graph = args.launch == "graph"
    run_step = graphed(step, torch) if use_graph else step

    def time_steps(fn):
        """exactly K steps between two synchronisations; ms per step"""
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        ev_ms = e0.elapsed_time(e1) / args.steps
        return max(ev_ms, wall_ms) if args.launch == "direct" else ev_ms

    ms_per_step = time_steps(run_step)

    def step_percentiles(fn, reps=100):
        """every step between its own pair of events: spread of the step time (not part of `value`)"""
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
        for a, b in evs:
            a.record()
            fn()
            b.record()
        torch.cuda.synchronize()
        ts = sorted(a.elapsed_time(b) for a, b in evs)
        return {"reps": reps, "p10": round(ts[reps // 10], 4), "median": round(ts[reps // 2], 4),
                "p90": round(ts[reps * 9 // 10], 4)}

    spread = step_percentiles(run_step) if use_graph else None
    other_modes = {}
    if args.all_modes:
        for m in ("dropin", "fused", "planned", "planned-fused", "planned-lora"):
            if m == args.mode:
                continue
            st, _ = make_step(w, bufs, m)
            fn = graphed(st, torch) if use_graph else st
            ms = time_steps(fn)
            other_modes[m] = {"ms_per_step": round(ms, 4), "tokens_per_s": round(w.batch / (ms * 1e-3), 1),
                              "launches_per_step": w.n_layers * (2 if m == "planned-lora" else 4 if m.endswith("fused") else 8)}

    # ---- launch duration of every kind of launch in the step: a sweep of that kind over
    # all layers, HIP events on the stream the kernels run on (back-to-back launches, so
    # the figure includes the gap between two launches)
    reps = max(5, args.steps // 2)
    kernels = {}
    for label, (sweep, kname, n_launch, nbytes) in families.items():
        fn = graphed(sweep, torch) if use_graph else sweep
        us = time_region(fn, reps, 3, torch) * 1e3 / n_launch
        gbs = nbytes / (us * 1e-6) / 1e9
        kernels[label] = {"kernel": kname, "launches_per_step": n_launch, "us_per_launch": round(us, 3),
                          "bytes_per_launch": int(nbytes), "GBps": round(gbs, 1),
                          "frac": round(gbs / HBM_PEAK_GBS, 4)}
    dom = max(kernels.values(), key=lambda k: k["us_per_launch"] * k["launches_per_step"])
    if fused:
        # streaming ceiling of each kind of launch: a checksum kernel (one wavefront per page, loads only)
        # over exactly the weight pages that launch reads -- no activations, no outputs, no dependent lookups
        import numpy as np
        from slora_hip.infer_adapter import page_checksums
        u = w.distinct_adapters()

        def pages_of(projs, expand):
            # A side: one page per rank row; B side: the r * h_out elements of B^T from the slot's first page on
            def n_pages(a, p):
                return -(-int(w.ranks[a]) * w.h_out[p] // w.page_elems) if expand else int(w.ranks[a])
            idx = [w.a_start_np[a] + p * w.ranks[a] + np.arange(n_pages(a, p)) for p in projs for a in u]
            return torch.from_numpy(w.a_loc_np[np.concatenate(idx)]).to(device)

        one_launch = args.mode == "planned-lora"
        kinds = ((("qkv_lora", (0, 1, 2)), ("o_lora", (3,))) if one_launch else
                 (("qkv_shrink", (0, 1, 2)), ("o_shrink", (3,)), ("qkv_expand", (0, 1, 2)), ("o_expand", (3,))))
        for label, projs in kinds:
            # a launch that does both halves reads the A pages and then the B pages: two checksum launches
            sides = ([(w.key_buffer, False), (w.value_buffer, True)] if one_launch else
                     [(w.value_buffer, True)] if label.endswith("expand") else [(w.key_buffer, False)])
            locs = [(side, pages_of(projs, expand)) for side, expand in sides]

            def sweep(locs=locs):
                for l in range(w.n_layers):
                    for side, loc in locs:
                        page_checksums(side[l], loc)

            fn = graphed(sweep, torch) if use_graph else sweep
            us = time_region(fn, reps, 3, torch) * 1e3 / w.n_layers
            nb = sum(int(loc.numel()) for _, loc in locs) * w.page_elems * 2
            kernels[label]["read_only_ceiling"] = {"us": round(us, 3), "page_bytes": nb, "launches": len(locs),
                                                   "GBps": round(nb / us / 1e3, 1),
                                                   "kernel_over_ceiling": round(kernels[label]["us_per_launch"] / us, 3)}

    streaming = None
    if fused:
        # what a plain read reaches on this chip when a launch is large: the same checksum kernel over
        # 16384 neighbouring pages of every layer's pool (as many bytes as a 134 MB launch would move)
        n_seq = min(16384, w.n_pages)
        seq = torch.arange(n_seq, dtype=torch.int64, device=device)

        def seq_sweep():
            for l in range(w.n_layers):
                page_checksums(w.key_buffer[l], seq)

        fn = graphed(seq_sweep, torch) if use_graph else seq_sweep
        us = time_region(fn, reps, 3, torch) * 1e3 / w.n_layers
        nb = n_seq * w.page_elems * 2
        streaming = {"contiguous_read": {"what": f"{n_seq} neighbouring pages per launch, one wavefront per page, loads only",
                                         "bytes": nb, "us": round(us, 3), "GBps": round(nb / us / 1e3, 1),
                                         "frac_of_peak": round(nb / us / 1e3 / HBM_PEAK_GBS, 4)}}
        # the step if every launch ran at its read-only ceiling
        ceil_us = sum(k["read_only_ceiling"]["us"] * k["launches_per_step"] for k in kernels.values())
        streaming["step_at_read_only_ceilings"] = {
            "ms": round(ceil_us * 1e-3, 4),
            "frac_of_peak": round(w.step_bytes(fused) / (ceil_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}

    step_gbs = w.step_bytes(fused) / (ms_per_step * 1e-3) / 1e9
    out = {
        "metric": METRIC,
        "value": round(w.batch / (ms_per_step * 1e-3), 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "step_ms_spread": spread,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16" if w.dtype == torch.float16 else "bf16",
        "data": "synthetic",
        "config": {
            "workload": w.name,
            "layers": w.n_layers,
            "batch": w.batch,
            "distinct_adapters_in_batch": int(w.distinct_adapters().size),
            "pool_pages_per_layer": w.n_pages, "page_bytes": w.page_elems * 2, "placement": args.placement,
            "mode": args.mode,
            "launch": args.launch,
            "launches_per_step": w.n_layers * (2 if args.mode == "planned-lora" else 4 if fused else 8) +
                                 (1 if args.mode.startswith("planned") else 0),
        },
        "step_hbm": {
            "algorithmic_bytes_per_step": w.step_bytes(fused),
            "achieved_GBps": round(step_gbs, 1),
            "frac_of_peak": round(step_gbs / HBM_PEAK_GBS, 4),
        },
        "roofline": {
            "kernel": dom["kernel"],
            "bound": "hbm",
            "achieved": dom["GBps"],
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": dom["frac"],
            "traffic": TRAFFIC_BYTES.get((args.workload, w.batch, args.mode, dom["kernel"])),
            "algorithmic_bytes_per_launch": dom["bytes_per_launch"],
            "us_per_launch": dom["us_per_launch"],
        },
        "kernels": kernels,
    }
    if streaming is not None:
        out["streaming"] = streaming
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w, bufs, torch, args.cpu_reps)
        if args.workload == "s2":
            out["cpu_baseline"]["c1"] = cpu_baseline_c1(torch)
    if args.workload == "s4" and not args.no_extras:
        # the prefill half of the mixed S4 step, over the same pool: 4 requests of 256 tokens
        pf = measure_prefill(argparse.Namespace(layers=min(w.n_layers, 4), steps=10, warmup=3, launch="graph"), torch,
                             device, w=w, seg=workloads.c4_prefill_segments(w, device))
        n = pf["config"]["layers"]
        out["prefill_part"] = {"what": "4 prefill requests of 256 tokens in the same step, same pool",
                               "ms_per_layer": round(pf["ms_per_step"] / n, 4),
                               "ms_per_layer_qkv_fused": round(pf["ms_per_step_qkv_fused"] / n, 4),
                               "decode_ms_per_layer": round(ms_per_step / w.n_layers, 4), "kernels": pf["kernels"]}
    if args.workload == "s2" and not args.no_extras:
        other_modes.update(measure_dropin_direct(w, bufs, torch, args))
        free_workload(w, bufs, torch)
        c3 = measure_prefill(argparse.Namespace(layers=2, steps=10, warmup=3, launch="graph"), torch, device)
        out["prefill_c3"] = {"tokens_per_s_per_layer": c3["value"], "ms_per_layer": round(c3["ms_per_step"] / 2, 4),
                             "ms_per_layer_qkv_fused": round(c3["ms_per_step_qkv_fused"] / 2, 4),
                             "tokens": c3["config"]["tokens"], "dtype": "bf16", "kernels": c3["kernels"]}
    if other_modes:
        out["modes"] = other_modes
    if args.workload == "s2" and not args.no_extras:
        out["other_shapes"] = measure_other_shapes(w, bufs, torch)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
