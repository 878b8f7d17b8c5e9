"""The LoRA half of the batch engine (slora_hip.LoraUnorderedBatchInfer) on the GPU: a
small multi-layer "model" whose base projections are random matrices, adapters loaded
through InferAdapter into a MemoryAllocator pool, decode and prefill steps.  Checked
against the bmm semantics of the oracle (rtol 1e-2 / atol 1e-3 scaled to the size of
the outputs, see ``close``) and, bit for bit, the fused issue order against the
reference's 8 calls per layer."""
import numpy as np
import pytest
import torch

from oracle import lora_oracle as O
from test_pool_gpu import _Adapter, _np_mats

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-3


def close(got, want):
    """rtol 1e-2, atol 1e-3 per unit of the outputs' scale: the outputs are sums of a base
    projection of order 1..4 and a delta, rounded to a 16-bit type several times on the way."""
    scale = max(1.0, float(np.abs(want).max()))
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL * scale)


class _Model:
    """Pool, adapters and tables of a tiny model: hidden H, L layers, k/v width KV."""

    def __init__(self, gpu, dtype, H, KV, L, ranks, heads=4, pool=1400, seed=0):
        from slora_hip.infer_adapter import InferAdapter, MemoryAllocator
        self.H, self.KV, self.L, self.dtype = H, KV, L, dtype
        self.tdt = torch.float16 if dtype == "f16" else torch.bfloat16
        rng = np.random.default_rng(seed)
        self.mm = MemoryAllocator(pool, 0, self.tdt, heads, H // heads, L, device=gpu)
        for b in self.mm.key_buffer + self.mm.value_buffer:
            b.zero_()
        hole = self.mm.alloc(37)                     # KV pages in use between the adapters' pages
        self.mm.free(hole[::3].contiguous())
        self.ia = InferAdapter.init(self.mm, device=gpu)
        self.h_out = [H, KV, KV, H]
        self.mats, self.adapters = {}, {}
        for name, r in ranks.items():
            A, B = _np_mats(rng, H, self.h_out, r, L, dtype)
            self.mats[name] = (A, B)
            self.adapters[name] = _Adapter(
                name, r, 16.0, [[torch.from_numpy(a).to(gpu, self.tdt) for a in A[l]] for l in range(L)],
                [[torch.from_numpy(b).to(gpu, self.tdt) for b in B[l]] for l in range(L)])
        self.ia.load_adapters(list(self.adapters.values()))
        self.names = list(ranks)
        self.scal = np.array([16.0 / ranks[n] for n in self.names], np.float32)

    def ref(self, layer, p, y0, x, bins):
        A = [self.mats[n][0][layer][p] for n in self.names]
        B = [self.mats[n][1][layer][p] for n in self.names]
        return O.ref_bmm(y0, x, A, B, self.scal, bins, self.dtype)


def _run_layers(m, eng, gpu, x_np, base_np, kv_rows=None):
    """All layers of one step.  base_np[l][p]: the base model's projection outputs.  With
    kv_rows (a contiguous range of pool pages, the decode slots of
    transformer_layer_infer_template.py:39-41) cache_k / cache_v are those rows of the
    layer's own key / value buffers.  Returns the outputs per layer and projection."""
    outs = []
    for l in range(m.L):
        x = torch.from_numpy(x_np[l][0]).to(gpu, m.tdt)
        xo = torch.from_numpy(x_np[l][1]).to(gpu, m.tdt)
        q = torch.from_numpy(base_np[l][0]).to(gpu, m.tdt)
        if kv_rows is None:
            ck = torch.from_numpy(base_np[l][1]).to(gpu, m.tdt)
            cv = torch.from_numpy(base_np[l][2]).to(gpu, m.tdt)
        else:
            ck = m.mm.key_buffer[l][kv_rows[0]: kv_rows[1]].view(-1, m.KV)
            cv = m.mm.value_buffer[l][kv_rows[0]: kv_rows[1]].view(-1, m.KV)
            ck.copy_(torch.from_numpy(base_np[l][1]).to(gpu, m.tdt))
            cv.copy_(torch.from_numpy(base_np[l][2]).to(gpu, m.tdt))
        o = torch.from_numpy(base_np[l][3]).to(gpu, m.tdt)
        eng.lora_get_qkv(l, x, q, ck, cv)
        eng.lora_get_o(l, xo, o)
        torch.cuda.synchronize()
        outs.append([t.float().cpu().numpy().copy() for t in (q, ck, cv, o)])
    return outs


def _inputs(m, rng, n_tok):
    x = [[O.round_to(rng.standard_normal((n_tok, m.H)).astype(np.float32), m.dtype) for _ in range(2)]
         for _ in range(m.L)]
    base = [[O.round_to(rng.standard_normal((n_tok, m.h_out[p])).astype(np.float32), m.dtype) for p in range(4)]
            for _ in range(m.L)]
    return x, base


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_decode_step_fused_and_reference_order(gpu, dtype):
    """A decode step over 3 layers: 23 requests on 5 adapters of ranks 8..64; k and v are
    written into contiguous decode slots of the pool itself (for v the output and the weight
    pages are one buffer).  Fused and reference call order agree bit for bit; both match bmm."""
    from slora_hip import LoraUnorderedBatchInfer
    ranks = {"a": 8, "b": 64, "c": 16, "d": 32, "e": 8}
    m = _Model(gpu, dtype, 256, 256, 3, ranks)
    rng = np.random.default_rng(11)
    req = [m.names[i] for i in rng.integers(0, len(ranks), size=23)]
    bins = np.array([m.names.index(n) for n in req])
    got = m.mm.alloc_contiguous(len(req))
    assert got is not None
    kv_rows = (int(got[1]), int(got[2]))
    b_seq_len = torch.from_numpy(rng.integers(5, 90, size=len(req)).astype(np.int32)).to(gpu)
    b_start = torch.zeros(len(req), dtype=torch.int32, device=gpu)
    x, base = _inputs(m, rng, len(req))
    res = {}
    for fused in (True, False):
        eng = LoraUnorderedBatchInfer(m.ia, [m.adapters[n] for n in req], fused=fused)
        assert eng.max_lora_dim == 64 and eng.req_bins.cpu().tolist() == bins.tolist()
        eng.begin_step(b_start, b_seq_len, is_prefill=False)
        assert not eng.use_segmented and len(eng.delta) == 3 and eng.delta[0].shape == (len(req), 64)
        res[fused] = _run_layers(m, eng, gpu, x, base, kv_rows=kv_rows)
    for l in range(m.L):
        for p in range(4):
            assert np.array_equal(res[True][l][p], res[False][l][p]), (l, p)
            xin = x[l][1] if p == 3 else x[l][0]
            close(res[True][l][p], m.ref(l, p, base[l][p], xin, bins))
    m.mm.free(got[0])


@pytest.mark.parametrize("lens,segmented", [
    ([210, 40, 3, 250, 64], True),      # a long request, rank 64 present, 5 requests: segmented kernels
    ([150, 40, 199], False),            # no request reaches 200 tokens: per-token BGMV
    ([300], False),                     # a single request: BGMV (lora_unordered_batch_infer.py:334)
])
def test_prefill_step_kernel_choice_and_results(gpu, lens, segmented):
    from slora_hip import LoraUnorderedBatchInfer
    ranks = {"a": 64, "b": 8, "c": 32}
    m = _Model(gpu, "f16", 512, 128, 2, ranks, heads=4)
    rng = np.random.default_rng(sum(lens))
    req = [m.names[i] for i in rng.integers(0, len(ranks), size=len(lens))]
    if "a" not in req:
        req[0] = "a"
    lens_np = np.asarray(lens, np.int32)
    bins = np.repeat([m.names.index(n) for n in req], lens_np)
    b_seq_len = torch.from_numpy(lens_np).to(gpu)
    start = np.zeros(len(lens), np.int32)
    start[1:] = np.cumsum(lens_np)[:-1]
    b_start = torch.from_numpy(start).to(gpu)
    x, base = _inputs(m, rng, int(lens_np.sum()))
    res = {}
    for fused in (True, False):
        eng = LoraUnorderedBatchInfer(m.ia, [m.adapters[n] for n in req], fused=fused)
        if fused:     # reads max(b_seq_len) and the token count back, as the reference does
            eng.begin_step(b_start, b_seq_len, is_prefill=True)
        else:         # or is told both
            eng.begin_step(b_start, b_seq_len, is_prefill=True, max_b_seq_len=int(lens_np.max()),
                           total_token_num=int(lens_np.sum()))
        assert eng.use_segmented == segmented and eng.max_b_seq_len == int(lens_np.max())
        assert eng.batch_req_bins.cpu().tolist() == bins.tolist()
        res[fused] = _run_layers(m, eng, gpu, x, base)
    for l in range(m.L):
        for p in range(4):
            assert np.array_equal(res[True][l][p], res[False][l][p]), (l, p)
            xin = x[l][1] if p == 3 else x[l][0]
            close(res[True][l][p], m.ref(l, p, base[l][p], xin, bins))


def test_engine_takes_buffers_from_the_adapter_table_itself(gpu):
    """The reference's NaiveInferAdapter keeps key_buffer / value_buffer on itself
    (lora_unordered_batch_infer.py:28-30); such an object works as well."""
    from types import SimpleNamespace
    from slora_hip import LoraUnorderedBatchInfer
    m = _Model(gpu, "f16", 256, 256, 1, {"a": 8, "b": 16})
    naive = SimpleNamespace(a_loc=m.ia.a_loc, a_start=m.ia.a_start, a_len=m.ia.a_len, a_scaling=m.ia.a_scaling,
                            adapter_dirs=m.ia.adapter_dirs, key_buffer=m.mm.key_buffer, value_buffer=m.mm.value_buffer)
    req = ["b", "a", "a", "b", "b"]
    bins = np.array([m.names.index(n) for n in req])
    eng = LoraUnorderedBatchInfer(naive, [m.adapters[n] for n in req])
    assert eng.req_bins.cpu().tolist() == bins.tolist()      # found by searching adapter_dirs, as the reference does
    eng.begin_step(torch.zeros(5, dtype=torch.int32, device=gpu), torch.full((5,), 9, dtype=torch.int32, device=gpu),
                   is_prefill=False, max_b_seq_len=9)
    rng = np.random.default_rng(2)
    x, base = _inputs(m, rng, 5)
    out = _run_layers(m, eng, gpu, x, base)
    for p in range(4):
        close(out[0][p], m.ref(0, p, base[0][p], x[0][1] if p == 3 else x[0][0], bins))


def test_engine_rejects_requests_without_adapter(gpu):
    from slora_hip import LoraUnorderedBatchInfer
    m = _Model(gpu, "f16", 256, 256, 1, {"a": 8})
    with pytest.raises(ValueError, match="without an adapter"):
        LoraUnorderedBatchInfer(m.ia, [m.adapters["a"], None])
