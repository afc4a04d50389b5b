"""One decode step of the paged int4 cache in one launch (qr_kv_quant_append_batch_decode_f16_i4): the pages must hold
what quantise-and-append stores (bit for bit), the output must be the attention over that cache (oracle, rtol / atol
1e-3) and agree with the two-launch form."""
import numpy as np
import pytest
import torch

from oracle import quarot_oracle as o
from quarot_amd import _lib
from quarot_amd.transformers import kv_cache as kv
from test_gpu_paged_kv import ATOL, F16, RTOL, bits, close, gpu, paged_case, synth_kv

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("hadamard", [True, False])
@pytest.mark.parametrize("page_size,lens,heads", [(16, [1, 16, 17, 100, 700], 5), (64, [64, 1000, 129], 3), (5, [11, 1, 64], 4),
                                                  (16, [4100, 33], 8), (2048, [2048, 2047], 2)])
def test_append_and_attention_in_one_launch(page_size, lens, heads, hadamard):
    rng = np.random.default_rng(page_size + len(lens) + heads)
    layer = 1
    data, param, indptr, indices, last = paged_case(rng, heads, page_size, lens)
    B = len(lens)
    k, v = synth_kv(rng, B, heads), synth_kv(rng, B, heads)
    # special vectors: an infinity, a NaN, all zeros, a constant, the fp16 extremes
    k[0, 0, 5] = np.inf
    v[0, 1, 7] = np.nan
    k[1, 0, :] = 0
    v[1, 0, :] = F16(3.25)
    if B > 2:
        k[2, 1, 3], k[2, 1, 4] = 65504, -65504
        v[2, 0, :] = F16(1e-7)
    q = (rng.standard_normal((B, heads, 128)) * 2).astype(F16)
    tabs = (gpu(indptr), gpu(indices), gpu(last))
    # two launches
    gd2, gp2 = gpu(data), gpu(param)
    kv.quantize_append_kv_i4(gd2, gp2, *tabs, gpu(k), gpu(v), None, layer, hadamard=hadamard)
    two = torch.full((B, heads, 128), float("nan"), dtype=torch.float16, device="cuda:0")
    kv.batch_decode_i4(two, gpu(q), gd2, gp2, *tabs, layer, q_hadamard=True)
    want = o.paged_batch_decode(o.kv_hadamard(q), gd2.cpu().numpy(), gp2.cpu().numpy(), indptr, indices, last, layer)
    for hint in (0, max(lens)):
        gd1, gp1 = gpu(data), gpu(param)
        one = torch.full_like(two, float("nan"))
        kv.batch_decode_i4(one, gpu(q), gd1, gp1, *tabs, layer, max_seq_len=hint, q_hadamard=True, append=(gpu(k), gpu(v), hadamard))
        assert torch.equal(gd1, gd2), (page_size, hint)
        assert torch.equal(gp1.view(torch.int16), gp2.view(torch.int16))
        g1, g2 = one.cpu().numpy(), two.cpu().numpy()
        finite = np.isfinite(want)
        assert np.array_equal(np.isnan(g1), np.isnan(g2))
        assert close(g1[finite], want[finite]) and close(g1[finite], g2[finite])
    # without the query's Hadamard, through the C entry point
    L = _lib.lib()
    gd1, gp1 = gpu(data), gpu(param)
    gq, gk, gv = gpu(o.kv_hadamard(q)), gpu(k), gpu(v)
    one = torch.full_like(two, float("nan"))
    rc = L.qr_kv_quant_append_batch_decode_f16_i4(one.data_ptr(), gq.data_ptr(), 0, gk.data_ptr(), gv.data_ptr(), 1 if hadamard else 0,
                                                  gd1.data_ptr(), gp1.data_ptr(), tabs[0].data_ptr(), tabs[1].data_ptr(), tabs[2].data_ptr(),
                                                  gd1.shape[0], 2, layer, heads, page_size, 128, B, 0, None, 0,
                                                  torch.cuda.current_stream().cuda_stream)
    assert rc == 0 and torch.equal(gd1, gd2)
    finite = np.isfinite(want)
    assert close(one.cpu().numpy()[finite], want[finite])
    assert L.qr_kv_quant_append_batch_decode_f16_i4(one.data_ptr(), gq.data_ptr(), 0, None, gv.data_ptr(), 1, gd1.data_ptr(), gp1.data_ptr(),
                                                    tabs[0].data_ptr(), tabs[1].data_ptr(), tabs[2].data_ptr(), gd1.shape[0], 2, layer, heads,
                                                    page_size, 128, B, 0, None, 0, None) == -1
    assert L.qr_kv_quant_append_batch_decode_f16_i4(one.data_ptr(), gq.data_ptr(), 2, gk.data_ptr(), gv.data_ptr(), 1, gd1.data_ptr(),
                                                    gp1.data_ptr(), tabs[0].data_ptr(), tabs[1].data_ptr(), tabs[2].data_ptr(), gd1.shape[0],
                                                    2, layer, heads, page_size, 128, B, 0, None, 0, None) == -5


def test_cache_class_holds_the_token_for_the_attention_call_and_never_shows_a_stale_cache():
    """update() of a decode step hands the token to the attention call; reading the pages, asking for the tables or
    updating again before that call stores it first; a second call of the returned callable is plain attention."""
    dev = torch.device("cuda:0")
    B, P, S, H = 3, 16, 70, 4
    g = torch.Generator(device=dev).manual_seed(1)
    rnd = lambda *shape: torch.randn(*shape, generator=g, device=dev).half()
    k0, v0 = rnd(B, S, H, 128), rnd(B, S, H, 128)
    steps = [(rnd(B, 1, H, 128), rnd(B, 1, H, 128), rnd(B, 1, H, 128)) for _ in range(4)]

    def fresh():
        c = kv.MultiLayerPagedKVCache4Bit(B, P, S + 8, dev, 1, H, 128)
        c.pages.zero_()                                      # (the pool is uninitialised memory: make untouched slots comparable)
        c.scales.zero_()
        c.update(k0, v0, 0, {})
        return c

    # reference: every step as two launches (the token stored before the attention call)
    ref, outs = fresh(), []
    for k1, v1, q1 in steps:
        f = ref.update(k1, v1, 0, {})
        ref.pages                                            # (looking at the pages stores the held token)
        assert not ref._pending
        outs.append(f(q1))
    # one launch per step
    c = fresh()
    for i, (k1, v1, q1) in enumerate(steps):
        f = c.update(k1, v1, 0, {})
        assert 0 in c._pending
        y = f(q1)
        assert not c._pending
        assert close(y.cpu().numpy(), outs[i].cpu().numpy())
        y2 = f(q1)                                            # again: plain attention over the same cache
        assert close(y2.cpu().numpy(), outs[i].cpu().numpy())
    assert torch.equal(c.pages, ref.pages) and torch.equal(c.scales.view(torch.int16), ref.scales.view(torch.int16))
    # the callable never called: the next update stores the token first
    c2 = fresh()
    for k1, v1, q1 in steps:
        c2.update(k1, v1, 0, {})
    assert torch.equal(c2.pages, ref.pages) and torch.equal(c2.scales.view(torch.int16), ref.scales.view(torch.int16))
    # asking for the tables stores it as well
    c3 = fresh()
    c3.update(*steps[0][:2], 0, {})
    specs = c3.get_cache_specs_for_flash_infer(None)
    assert not c3._pending
    c4 = fresh()
    c4.update(*steps[0][:2], 0, {})(steps[0][2])
    assert torch.equal(specs["kv_data"], c4.pages)


@pytest.mark.parametrize("page_size", [16, 5])
@pytest.mark.parametrize("B,heads", [(40, 32), (12, 24)])
def test_append_and_attention_with_many_sequence_head_pairs(B, heads, page_size):
    """Batches with 288 and 1280 (sequence, head) pairs: the entry point then forms workgroups of eight and of four
    waves; pages and outputs as in the test above."""
    rng = np.random.default_rng(B + heads + page_size)
    lens = [int(v) for v in rng.integers(1, 90, B)]
    data, param, indptr, indices, last = paged_case(rng, heads, page_size, lens, layers=1)
    k, v = synth_kv(rng, B, heads), synth_kv(rng, B, heads)
    q = (rng.standard_normal((B, heads, 128)) * 2).astype(F16)
    tabs = (gpu(indptr), gpu(indices), gpu(last))
    gd2, gp2 = gpu(data), gpu(param)
    kv.quantize_append_kv_i4(gd2, gp2, *tabs, gpu(k), gpu(v), None, 0, hadamard=True)
    two = torch.empty((B, heads, 128), dtype=torch.float16, device="cuda:0")
    kv.batch_decode_i4(two, gpu(q), gd2, gp2, *tabs, 0, q_hadamard=True)
    want = o.paged_batch_decode(o.kv_hadamard(q), gd2.cpu().numpy(), gp2.cpu().numpy(), indptr, indices, last, 0)
    gd1, gp1 = gpu(data), gpu(param)
    one = torch.full_like(two, float("nan"))
    kv.batch_decode_i4(one, gpu(q), gd1, gp1, *tabs, 0, q_hadamard=True, append=(gpu(k), gpu(v), True))
    assert torch.equal(gd1, gd2) and torch.equal(gp1.view(torch.int16), gp2.view(torch.int16))
    assert close(one.cpu().numpy(), want) and close(one.cpu().numpy(), two.cpu().numpy())


def test_one_launch_decode_step_replays_from_a_hip_graph_and_rejects_wrong_shapes():
    """The step's one launch captured into a HIP graph: replays with fresh keys, values and queries copied into the
    static buffers, eager work and synchronisation in between, store the same pages and give the same outputs as the
    eager two-launch step.  The Python mirror refuses new-token tensors of the wrong shape, dtype or layout."""
    rng = np.random.default_rng(21)
    heads, P, lens = 8, 16, [300, 17, 64]
    B = len(lens)
    data, param, indptr, indices, last = paged_case(rng, heads, P, lens, layers=1)
    tabs = (gpu(indptr), gpu(indices), gpu(last))
    gd1, gp1 = gpu(data), gpu(param)
    sk, sv, sq = (torch.zeros((B, heads, 128), dtype=torch.float16, device="cuda:0") for _ in range(3))
    out = torch.empty_like(sq)
    step = lambda: kv.batch_decode_i4(out, sq, gd1, gp1, *tabs, 0, q_hadamard=True, append=(sk, sv, True))
    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for i in range(4):
        k, v = gpu(synth_kv(rng, B, heads)), gpu(synth_kv(rng, B, heads))
        q = gpu((rng.standard_normal((B, heads, 128)) * 2).astype(F16))
        gd2, gp2 = gpu(data), gpu(param)
        kv.quantize_append_kv_i4(gd2, gp2, *tabs, k, v, None, 0, hadamard=True)          # eager work between the replays
        two = torch.empty_like(out)
        kv.batch_decode_i4(two, q, gd2, gp2, *tabs, 0, q_hadamard=True)
        torch.cuda.synchronize()
        sk.copy_(k); sv.copy_(v); sq.copy_(q)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(gd1, gd2) and torch.equal(gp1.view(torch.int16), gp2.view(torch.int16)), f"replay {i}"
        assert close(out.cpu().numpy(), two.cpu().numpy()), f"replay {i}"
    q = gpu(rng.standard_normal((B, heads, 128)).astype(F16))
    good = gpu(synth_kv(rng, B, heads))
    for bad in (good[:, :, :64], good.float(), good[:2].contiguous(), good.view(B, heads * 128), good.transpose(0, 1)):
        with pytest.raises(RuntimeError):
            kv.batch_decode_i4(out, q, gd1, gp1, *tabs, 0, q_hadamard=True, append=(bad, good, True))
        with pytest.raises(RuntimeError):
            kv.batch_decode_i4(out, q, gd1, gp1, *tabs, 0, q_hadamard=True, append=(good, bad, True))
