"""Shrink and expand in one launch (dispatch_bgmv_lora / dispatch_bgmv_qkv_lora) against the two
stateless calls: bitwise, for single projections and q/k/v, over several launches on one plan
(the hand-over counters are never reset), with and without an item count."""
import numpy as np
import pytest
import torch

from lora_cases import make_case
from test_bgmv_gpu import GpuCase

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("hidden,ranks,batch,h_out,rank_cap", [
    (1024, [64, 8, 32, 16], 70, [1024, 256, 256, 1024], 64),
    (4096, [64, 32, 16, 8, 8, 16], 256, None, 64),
    (512, [16, 8, 64, 32], 1500, None, 64),
    (256, [4, 12, 8, 24], 30, None, 24),       # element-wise expand path
    (512, [64, 8, 128], 40, None, 32),          # ranks above rank_cap keep using a_loc
    (5120, [64, 16, 32], 33, None, 64),         # a page of one and a quarter 4096-element passes
    (8192, [64, 8], 20, [8192, 1024, 1024, 8192], 64),
])
def test_one_launch_lora_equals_the_two_calls(gpu, dtype, hidden, ranks, batch, h_out, rank_cap):
    import slora_hip
    from slora_hip import dispatch_bgmv, dispatch_bgmv_lora, dispatch_bgmv_qkv_lora
    bins = None
    if batch == 1500:
        bins = np.random.default_rng(3).choice(4, size=batch, p=[0.85, 0.05, 0.05, 0.05])
    c = make_case(300 + hidden + batch, hidden, ranks, batch, dtype=dtype, h_out=h_out, zipf_alpha=1.0, bins=bins)
    g = GpuCase(c, gpu)
    R = max(max(ranks), 8)
    R = (R + 7) // 8 * 8
    t = (g.a_start, g.a_len, g.a_loc, g.bins)
    y0 = [torch.randn((batch, c.h_out[p]), dtype=g.tdt, device=gpu) for p in range(4)]
    d_s = [torch.zeros((batch, R), dtype=g.tdt, device=gpu) for _ in range(4)]
    y_s = [v.clone() for v in y0]
    for p in range(4):
        dispatch_bgmv(d_s[p], g.x, g.key, *t, p, g.scales, plan=False)
        dispatch_bgmv(y_s[p], d_s[p], g.value, *t, p, g.scales, plan=False)
    for readback in (True, False):
        plan = slora_hip.make_plan(*t, rank_cap, c.n_pages, readback=readback)
        for rep in range(3):   # the counters behind the plan keep counting
            print(f"one-launch lora {dtype} hidden {hidden} batch {batch} readback {readback} rep {rep}", flush=True)
            for p in range(4):
                d = torch.zeros((batch, R), dtype=g.tdt, device=gpu)
                y = y0[p].clone()
                dispatch_bgmv_lora(y, d, g.x, g.key, g.value, *t, p, g.scales, plan=plan)
                assert torch.equal(d, d_s[p]), (p, rep)
                assert torch.equal(y, y_s[p]), (p, rep)
            d3 = [torch.zeros((batch, R), dtype=g.tdt, device=gpu) for _ in range(3)]
            y3 = [v.clone() for v in y0[:3]]
            dispatch_bgmv_qkv_lora(*y3, *d3, g.x, g.key, g.value, *t, g.scales, plan=plan)
            for p in range(3):
                assert torch.equal(d3[p], d_s[p]) and torch.equal(y3[p], y_s[p]), (p, rep)
        # no hand-over was abandoned
        words = plan.buf.cpu().numpy()
        assert words[0] == 0x534c5033
    # without a plan the same entry point issues the two stateless launches
    d = torch.zeros((batch, R), dtype=g.tdt, device=gpu)
    y = y0[3].clone()
    dispatch_bgmv_lora(y, d, g.x, g.key, g.value, *t, 3, g.scales, plan=False)
    assert torch.equal(d, d_s[3]) and torch.equal(y, y_s[3])
