"""The paged cache with fp16 pages (the reference's disable_quant mode: quarot/transformers/kv_cache.py:134-151,
quarot/kernels/bindings.cpp:247-374): append bit for bit against the oracle's page arithmetic, decode attention
against the oracle within rtol / atol 1e-3, and the cache class driven as the model code drives it."""
import numpy as np
import pytest
import torch

from oracle import quarot_oracle as o
from quarot_amd import _lib
from quarot_amd.transformers import kv_cache as kv
from test_gpu_paged_kv import ATOL, F16, RTOL, bits, close, gpu, paged_case, synth_kv

pytestmark = pytest.mark.gpu


def f16_case(rng, heads, page_size, lens, layers=2):
    """paged_case's page tables around a pool of fp16 pages full of random finite halves."""
    _, param, indptr, indices, last = paged_case(rng, heads, page_size, lens, layers=layers)
    pool = param.shape[0]
    data = rng.standard_normal((pool, layers, 2, heads, page_size, 128)).astype(F16)
    return data, param, indptr, indices, last


@pytest.mark.parametrize("page_size,lens,add", [(16, [40, 16, 1, 33], [40, 16, 1, 20]), (4, [6, 1, 9, 4], [3, 1, 9, 2]),
                                                (1, [3, 5], [3, 2]), (100, [250, 100, 99], [250, 7, 99])])
def test_append_of_fp16_vectors_prefill_and_single_token(page_size, lens, add):
    rng = np.random.default_rng(page_size)
    heads, layer = 3, 1
    data, param, indptr, indices, last = f16_case(rng, heads, page_size, lens)
    tokens = sum(add)
    k, v = synth_kv(rng, tokens, heads), synth_kv(rng, tokens, heads)
    kp = rng.standard_normal((tokens, heads, 2)).astype(F16)
    vp = rng.standard_normal((tokens, heads, 2)).astype(F16)
    app = np.concatenate([[0], np.cumsum(add)]).astype(np.int32)
    gd, gp = gpu(data), gpu(param)
    kv.init_kv_f16(gd, gp, gpu(indptr), gpu(indices), gpu(last), gpu(k), gpu(v), gpu(kp), gpu(vp), gpu(app), layer)
    wd, wp = data.copy(), param.copy()
    o.paged_append(wd, wp, indptr, indices, last, k, v, kp, vp, layer, app)
    assert np.array_equal(bits(gd.cpu().numpy()), bits(wd)) and np.array_equal(bits(gp.cpu().numpy()), bits(wp))
    # one more token per sequence (the tables already count it)
    B = len(lens)
    k1, v1 = synth_kv(rng, B, heads), synth_kv(rng, B, heads)
    p1 = rng.standard_normal((B, heads, 2)).astype(F16)
    kv.append_kv_f16(gd, gp, gpu(indptr), gpu(indices), gpu(last), gpu(k1), gpu(v1), gpu(p1), gpu(p1), layer)
    o.paged_append(wd, wp, indptr, indices, last, k1, v1, p1, p1, layer)
    assert np.array_equal(bits(gd.cpu().numpy()), bits(wd)) and np.array_equal(bits(gp.cpu().numpy()), bits(wp))


@pytest.mark.parametrize("page_size,lens,heads", [(16, [1, 16, 17, 100, 700], 5), (64, [64, 1000, 129], 3), (5, [11, 1, 64], 4),
                                                  (16, [4100, 33], 8), (2048, [2048, 2047], 2), (16, [300] * 40, 16)])
def test_decode_attention_over_fp16_pages_against_the_oracle(page_size, lens, heads):
    rng = np.random.default_rng(page_size + len(lens))
    layer = 1
    data, param, indptr, indices, last = f16_case(rng, heads, page_size, lens)
    # unused entries of the sequences' last pages and the spare pages hold NaNs: they must not reach a result
    used = np.zeros(data.shape[0], bool)
    used[indices] = True
    data[~used] = np.nan
    for b, n in enumerate(lens):
        pg = int(indices[int(indptr[b + 1]) - 1])
        data[pg, :, :, :, int(last[b]):, :] = np.nan
    B = len(lens)
    q = (rng.standard_normal((B, heads, 128)) * 2).astype(F16)
    got = torch.full((B, heads, 128), float("nan"), dtype=torch.float16, device="cuda:0")
    kv.batch_decode_f16(got, gpu(q), gpu(data), gpu(param), gpu(indptr), gpu(indices), gpu(last), layer)
    want = o.paged_batch_decode_f16(q, data, indptr, indices, last, layer)
    assert np.isfinite(want).all()
    assert close(got.cpu().numpy(), want)


def test_decode_attention_over_fp16_pages_of_a_sequence_without_pages_and_bad_page_numbers():
    rng = np.random.default_rng(3)
    heads, P = 2, 16
    data, param, indptr, indices, last = f16_case(rng, heads, P, [20, 7, 40])
    # the middle sequence loses its pages: a NaN row, nothing read
    per = np.diff(indptr)
    indptr2 = np.array([0, per[0], per[0], per[0] + per[2]], np.int32)
    indices2 = np.concatenate([indices[:per[0]], indices[per[0] + per[1]:]]).astype(np.int32)
    q = rng.standard_normal((3, heads, 128)).astype(F16)
    got = torch.zeros((3, heads, 128), dtype=torch.float16, device="cuda:0")
    kv.batch_decode_f16(got, gpu(q), gpu(data), gpu(param), gpu(indptr2), gpu(indices2), gpu(last), 0)
    g = got.cpu().numpy()
    assert np.isnan(g[1]).all()
    want = o.paged_batch_decode_f16(q[[0, 2]], data, np.array([0, per[0], per[0] + per[2]], np.int32), indices2, last[[0, 2]], 0)
    assert close(g[[0, 2]], want)
    # a page number outside the pool: its positions are skipped (the int4 kernel's rule), the others still count
    bad = indices.copy()
    bad[int(indptr[2]) + 1] = data.shape[0] + 5
    kv.batch_decode_f16(got, gpu(q), gpu(data), gpu(param), gpu(indptr), gpu(bad), gpu(last), 0)
    keep = np.r_[0:P, 2 * P:40]
    pages = indices[int(indptr[2]) + keep // P]
    kf = data[pages, 0, 0, :, keep % P, :].astype(np.float64)
    vf = data[pages, 0, 1, :, keep % P, :].astype(np.float64)
    lg = np.einsum("hd,shd->hs", q[2].astype(np.float64), kf) / np.sqrt(128.0)
    w = np.exp(lg - lg.max(axis=1, keepdims=True))
    w /= w.sum(axis=1, keepdims=True)
    assert close(got.cpu().numpy()[2], np.einsum("hs,shd->hd", w, vf))


def test_argument_errors_of_the_fp16_page_functions():
    rng = np.random.default_rng(5)
    heads, P = 2, 16
    data, param, indptr, indices, last = f16_case(rng, heads, P, [20, 7])
    gd, gp, tabs = gpu(data), gpu(param), (gpu(indptr), gpu(indices), gpu(last))
    q = gpu(rng.standard_normal((2, heads, 128)).astype(F16))
    out = torch.empty_like(q)
    with pytest.raises(RuntimeError, match="kv_data must be fp16"):
        kv.batch_decode_f16(out, q, gd.view(torch.uint8), gp, *tabs, 0)
    with pytest.raises(RuntimeError, match="kv_data must be uint8"):
        kv.batch_decode_i4(out, q, gd, gp, *tabs, 0)
    with pytest.raises(RuntimeError, match="q must be"):
        kv.batch_decode_f16(out[:, :1].contiguous(), q[:, :1].contiguous(), gd, gp, *tabs, 0)
    with pytest.raises(RuntimeError, match="layer_idx"):
        kv.batch_decode_f16(out, q, gd, gp, *tabs, 2)
    k = gpu(synth_kv(rng, 2, heads))
    prm = torch.zeros((2, heads, 2), dtype=torch.float16, device="cuda:0")
    with pytest.raises(RuntimeError, match="k and v must be fp16"):
        kv.append_kv_f16(gd, gp, *tabs, k.view(torch.uint8), k.view(torch.uint8), prm, prm, 0)
    with pytest.raises(RuntimeError, match="one token per sequence"):
        kv.append_kv_f16(gd, gp, *tabs, k[:1], k[:1], prm[:1], prm[:1], 0)
    L = _lib.lib()
    st = torch.cuda.current_stream().cuda_stream
    args = (gd.data_ptr(), gp.data_ptr(), tabs[0].data_ptr(), tabs[1].data_ptr(), tabs[2].data_ptr())
    assert L.qr_batch_decode_f16(out.data_ptr(), q.data_ptr(), *args, gd.shape[0], 2, 0, heads, P, 64, 2, st) == _lib.QR_E_UNSUPPORTED
    assert L.qr_batch_decode_f16(None, q.data_ptr(), *args, gd.shape[0], 2, 0, heads, P, 128, 2, st) == _lib.QR_E_NULL
    assert L.qr_batch_decode_f16(out.data_ptr(), q.data_ptr(), *args, gd.shape[0], 2, 2, heads, P, 128, 2, st) == _lib.QR_E_SHAPE
    assert L.qr_batch_decode_f16(out.data_ptr(), q.data_ptr(), *args, gd.shape[0], 2, 0, heads, P, 128, 0, st) == 0
    assert L.qr_kv_append_f16(*args, gd.shape[0], k.data_ptr(), k.data_ptr(), prm.data_ptr(), prm.data_ptr(), None, 3, 2, 0, heads, P,
                              128, 2, st) == _lib.QR_E_SHAPE


@pytest.mark.parametrize("hadamard_dtype", [torch.float16, None, torch.float32])
def test_cache_class_with_fp16_pages_prefill_then_decode_steps(hadamard_dtype):
    """MultiLayerPagedKVCache4Bit(disable_quant=True) as the model code drives it: the prompt through update(), then
    decode steps whose update() returns the attention callable; against the oracle's page arithmetic (bit for bit:
    the pages hold the kernel's own transformed keys and the values as they came) and its attention."""
    rng = np.random.default_rng(23)
    B, H, P, L, prompt = 3, 4, 16, 2, 37
    cache = kv.MultiLayerPagedKVCache4Bit(batch_size=B, page_size=P, max_seq_len=64, device="cuda:0", n_layers=L, num_heads=H,
                                          head_dim=128, disable_quant=True, hadamard_dtype=hadamard_dtype)
    assert cache.pages.shape == (4 * B, L, 2, H, P, 128) and cache.pages.dtype == torch.float16
    cache.pages.zero_(); cache.scales.zero_()
    data, param = np.zeros(cache.pages.shape, F16), np.zeros(cache.scales.shape, F16)

    def had(x):
        return x if hadamard_dtype is None else kv.matmul_had_cuda(gpu(x), hadamard_dtype).cpu().numpy()

    def oracle_store(k, v, layer, length, added):
        pc = -(-length // P)
        indptr = (np.arange(B + 1) * pc).astype(np.int32)
        indices = (np.arange(pc)[None, :] * B + np.arange(B)[:, None]).reshape(-1).astype(np.int32)
        last = np.full(B, length - (pc - 1) * P, np.int32)
        kk, vv = had(k).reshape(-1, H, 128), v.reshape(-1, H, 128)
        prm = np.zeros((kk.shape[0], H, 2), F16)
        prm[..., 0] = 1
        app = (np.arange(B + 1) * added).astype(np.int32)
        o.paged_append(data, param, indptr, indices, last, kk, vv, prm, prm, layer, app if added > 1 else None)
        return indptr, indices, last

    kpr, vpr = synth_kv(rng, B * prompt, H).reshape(B, prompt, H, 128), synth_kv(rng, B * prompt, H).reshape(B, prompt, H, 128)
    for layer in range(L):
        rk, rv = cache.update(gpu(kpr), gpu(vpr), layer, {})
        assert torch.equal(rk, gpu(kpr)) and torch.equal(rv, gpu(vpr))
        oracle_store(kpr, vpr, layer, prompt, prompt)
    assert np.array_equal(bits(cache.pages.cpu().numpy()), bits(data)) and np.array_equal(bits(cache.scales.cpu().numpy()), bits(param))
    for step in range(2):
        k1, v1 = synth_kv(rng, B, H).reshape(B, 1, H, 128), synth_kv(rng, B, H).reshape(B, 1, H, 128)
        qs = (rng.standard_normal((B, 1, H, 128)) * 2).astype(F16)
        for layer in range(L):
            fn = cache.update(gpu(k1), gpu(v1), layer, {})
            assert callable(fn)
            tabs = oracle_store(k1, v1, layer, prompt + step + 1, 1)
            attn = fn(gpu(qs))
            assert attn.shape == (B, 1, H, 128) and attn.dtype == torch.float16
            want = o.paged_batch_decode_f16(had(qs.reshape(B, H, 128)), data, *tabs, layer)
            assert close(attn.cpu().numpy().reshape(B, H, 128), want)
        assert np.array_equal(bits(cache.pages.cpu().numpy()), bits(data))
    assert cache.get_seq_length() == prompt + 2


def test_cache_class_with_fp16_pages_and_a_padded_prompt():
    """A left-padded prompt (attention_mask): only the rows the mask keeps enter the cache (kv_cache.py:206-220)."""
    rng = np.random.default_rng(29)
    B, H, P, S = 2, 2, 16, 24
    mask = np.ones((B, S), np.int64)
    mask[0, :5] = 0
    mask[1, :3] = 0                                          # 19 and 21 tokens: two pages each
    cache = kv.MultiLayerPagedKVCache4Bit(batch_size=B, page_size=P, max_seq_len=48, device="cuda:0", n_layers=1, num_heads=H,
                                          head_dim=128, disable_quant=True, hadamard_dtype=None)
    cache.pages.zero_()
    k, v = synth_kv(rng, B * S, H).reshape(B, S, H, 128), synth_kv(rng, B * S, H).reshape(B, S, H, 128)
    cache.update(gpu(k), gpu(v), 0, {"attention_mask": gpu(mask)})
    pages = cache.pages.cpu().numpy()
    for b, n in enumerate(mask.sum(axis=1)):
        kept = k[b, S - n:]
        for pos in range(n):
            assert np.array_equal(bits(pages[(pos // P) * B + b, 0, 0, :, pos % P, :]), bits(kept[pos]))
            assert np.array_equal(bits(pages[(pos // P) * B + b, 0, 1, :, pos % P, :]), bits(v[b, S - n + pos]))
