"""Paged int4 KV cache on the GPU through the C ABI's Python mirror: append (bit-exact data movement),
quantise-and-append (codes, scales and zeros bit-exact against the oracle quantiser, placed as the
oracle's append places them) and single-query attention over the cache (fp32 arithmetic: within
rtol 1e-3 / atol 1e-3 of the oracle's float64 softmax over the dequantised cache)."""
import numpy as np
import pytest
import torch

from oracle import quarot_oracle as o
from quarot_amd import _lib
from quarot_amd.transformers import kv_cache as kv

pytestmark = pytest.mark.gpu
F16, F32 = np.float16, np.float32
RTOL = ATOL = 1e-3


def gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


def bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


def close(got, want, rtol=RTOL, atol=ATOL):
    g, w = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return np.all(np.abs(g - w) <= atol + rtol * np.abs(w))


def paged_case(rng, heads, page_size, lens, layers=2, spare_pages=3):
    """Cache arrays full of random bytes (so untouched places can be verified) and the page tables of
    sequences with `lens` tokens, their pages scattered over the pool."""
    per = [max(1, -(-n // page_size)) for n in lens]
    total = sum(per) + spare_pages
    order = rng.permutation(total)
    indptr = np.concatenate([[0], np.cumsum(per)]).astype(np.int32)
    indices = order[: sum(per)].astype(np.int32)
    last = np.array([n - (p - 1) * page_size for n, p in zip(lens, per)], np.int32)
    data = rng.integers(0, 256, (total, layers, 2, heads, page_size, 64), dtype=np.uint8)
    param = (rng.standard_normal((total, layers, 2, heads, page_size, 2)) * np.array([0.05, 0.5])).astype(F16)
    param[..., 0] = np.abs(param[..., 0]) + F16(0.01)
    return data, param, indptr, indices, last


def synth_kv(rng, tokens, heads):
    x = rng.standard_normal((tokens, heads, 128))
    x[rng.random(x.shape) < 0.005] *= 15
    return x.astype(F16)


@pytest.mark.parametrize("page_size,lens,add", [(16, [40, 16, 1, 33], [40, 16, 1, 20]), (4, [6, 1, 9, 4], [3, 1, 9, 2]),
                                                (1, [3, 5], [3, 2]), (100, [250, 100, 99], [250, 7, 99]), (64, [64] * 5, [64] * 5)])
def test_append_of_quantised_vectors_prefill_and_single_token(page_size, lens, add):
    rng = np.random.default_rng(page_size + len(lens))
    heads, layer = 3, 1
    data, param, indptr, indices, last = paged_case(rng, heads, page_size, lens)
    app = np.concatenate([[0], np.cumsum(add)]).astype(np.int32)
    T = int(app[-1])
    k, v = rng.integers(0, 256, (T, heads, 64), dtype=np.uint8), rng.integers(0, 256, (T, heads, 64), dtype=np.uint8)
    kp, vp = rng.standard_normal((T, heads, 2)).astype(F16), rng.standard_normal((T, heads, 2)).astype(F16)
    gd, gp = gpu(data), gpu(param)
    tabs = dict(kv_indptr=gpu(indptr), kv_indices=gpu(indices), last_page_offset=gpu(last))
    assert kv.init_kv_i4(gd, gp, **tabs, k=gpu(k), v=gpu(v), k_param=gpu(kp), v_param=gpu(vp), seqlen_indptr=gpu(app),
                         layer_idx=layer) is None
    o.paged_append(data, param, indptr, indices, last, k, v, kp, vp, layer, app)
    assert np.array_equal(gd.cpu().numpy(), data) and np.array_equal(bits(gp.cpu().numpy()), bits(param))
    # one more token per sequence: the page tables must already count it
    lens2 = [n + 1 for n in lens]
    per = [max(1, -(-n // page_size)) for n in lens2]
    if per == [int(indptr[i + 1] - indptr[i]) for i in range(len(lens))]:       # still inside the pages it owns
        last2 = np.array([n - (p - 1) * page_size for n, p in zip(lens2, per)], np.int32)
        B = len(lens)
        k1, v1 = rng.integers(0, 256, (B, heads, 64), dtype=np.uint8), rng.integers(0, 256, (B, heads, 64), dtype=np.uint8)
        kp1, vp1 = rng.standard_normal((B, heads, 2)).astype(F16), rng.standard_normal((B, heads, 2)).astype(F16)
        kv.append_kv_i4(gd, gp, gpu(indptr), gpu(indices), gpu(last2), gpu(k1), gpu(v1), gpu(kp1), gpu(vp1), layer)
        o.paged_append(data, param, indptr, indices, last2, k1, v1, kp1, vp1, layer, None)
        assert np.array_equal(gd.cpu().numpy(), data) and np.array_equal(bits(gp.cpu().numpy()), bits(param))


@pytest.mark.parametrize("hadamard", [True, False])
@pytest.mark.parametrize("page_size,lens,add", [(16, [40, 16, 1, 33], [40, 16, 1, 20]), (5, [11, 5, 7], [11, 2, 7]),
                                                (128, [300, 128], [300, 128])])
def test_quantise_and_append_places_the_oracle_quantisers_codes(page_size, lens, add, hadamard):
    """fp16 K / V -> pages in two launches: the cache must equal what the oracle's quantiser (applied to the
    kernel's own Hadamard output for K, as everywhere) and the oracle's append produce, every byte."""
    rng = np.random.default_rng(page_size)
    heads, layer = 4, 0
    data, param, indptr, indices, last = paged_case(rng, heads, page_size, lens)
    app = np.concatenate([[0], np.cumsum(add)]).astype(np.int32)
    T = int(app[-1])
    k, v = synth_kv(rng, T, heads), synth_kv(rng, T, heads)
    gd, gp = gpu(data), gpu(param)
    kv.quantize_append_kv_i4(gd, gp, gpu(indptr), gpu(indices), gpu(last), gpu(k), gpu(v), gpu(app), layer, hadamard=hadamard)
    kin = kv.matmul_had_cuda(gpu(k), torch.float16).cpu().numpy() if hadamard else k
    if hadamard:
        assert close(kin, o.kv_hadamard(k))
    kq, ks, kz = o.kv_asym_quant(kin)
    vq, vs, vz = o.kv_asym_quant(v)
    o.paged_append(data, param, indptr, indices, last, kq, vq, np.concatenate([ks, kz], -1), np.concatenate([vs, vz], -1), layer, app)
    assert np.array_equal(gd.cpu().numpy(), data) and np.array_equal(bits(gp.cpu().numpy()), bits(param))
    # and the staged calls of the reference's update() give the same cache
    gd2, gp2 = gpu(data * 0), gpu(param * 0)
    gd3, gp3 = gd2.clone(), gp2.clone()
    q1, s1, z1 = kv.asym_quantize_and_pack_i4(gpu(k), hadamard=hadamard)
    q2, s2, z2 = kv.asym_quantize_and_pack_i4(gpu(v))
    kv.init_kv_i4(gd2, gp2, gpu(indptr), gpu(indices), gpu(last), q1, q2, torch.cat([s1, z1], -1), torch.cat([s2, z2], -1), gpu(app), layer)
    kv.quantize_append_kv_i4(gd3, gp3, gpu(indptr), gpu(indices), gpu(last), gpu(k), gpu(v), gpu(app), layer, hadamard=hadamard)
    assert torch.equal(gd2, gd3) and torch.equal(gp2, gp3)


@pytest.mark.parametrize("hadamard", [True, False])
def test_quantise_and_append_with_infinities_and_nans_equals_the_separate_quantisers(hadamard):
    """A vector that holds an infinity or a NaN: the one-launch quantise-and-append must store what the separate
    quantiser (itself pinned against the oracle on such vectors) followed by the append stores -- in particular an
    untransformed vector keeps the non-finite value in its own element (scale inf, zero = -min for an infinity)."""
    rng = np.random.default_rng(77)
    heads, layer, page_size, lens = 4, 1, 16, [40, 9, 23]
    data, param, indptr, indices, last = paged_case(rng, heads, page_size, lens)
    app = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(app[-1])
    k, v = synth_kv(rng, T, heads), synth_kv(rng, T, heads)
    for t, (a, b) in enumerate([(np.inf, None), (-np.inf, None), (np.nan, None), (np.inf, -np.inf), (np.inf, np.nan), (65504, -65504)]):
        for x in (k, v):
            x[3 + 5 * t, t % heads, 7 * t] = a
            if b is not None:
                x[3 + 5 * t, t % heads, 127 - t] = b
    gd2, gp2 = gpu(data), gpu(param)
    gd3, gp3 = gd2.clone(), gp2.clone()
    q1, s1, z1 = kv.asym_quantize_and_pack_i4(gpu(k), hadamard=hadamard)
    q2, s2, z2 = kv.asym_quantize_and_pack_i4(gpu(v))
    vq, vs, vz = o.kv_asym_quant(v)                         # the untransformed side against the oracle as well
    assert np.array_equal(q2.cpu().numpy(), vq)
    assert np.array_equal(bits(s2.cpu().numpy()), bits(vs)) and np.array_equal(bits(z2.cpu().numpy()), bits(vz))
    kv.init_kv_i4(gd2, gp2, gpu(indptr), gpu(indices), gpu(last), q1, q2, torch.cat([s1, z1], -1), torch.cat([s2, z2], -1), gpu(app), layer)
    kv.quantize_append_kv_i4(gd3, gp3, gpu(indptr), gpu(indices), gpu(last), gpu(k), gpu(v), gpu(app), layer, hadamard=hadamard)
    assert torch.equal(gd2, gd3)
    assert torch.equal(gp2.view(torch.int16), gp3.view(torch.int16))          # (bit patterns: NaN parameters compare unequal as floats)


@pytest.mark.parametrize("page_size,lens", [(16, [1, 16, 17, 100, 700]), (64, [64, 1000, 129]), (5, [11, 1, 64]), (100, [250, 99, 1]),
                                            (2048, [2048, 2047])])
def test_decode_attention_against_the_oracle(page_size, lens):
    rng = np.random.default_rng(page_size + 1)
    heads, layer = 5, 1
    data, param, indptr, indices, last = paged_case(rng, heads, page_size, lens)
    q = rng.standard_normal((len(lens), heads, 128)).astype(F16)
    want = o.paged_batch_decode(q, data, param, indptr, indices, last, layer)
    out = torch.full((len(lens), heads, 128), float("nan"), dtype=torch.float16, device="cuda:0")
    args = (gpu(data), gpu(param), gpu(indptr), gpu(indices), gpu(last))
    assert kv.batch_decode_i4(out, gpu(q), *args, layer) is None
    assert close(out.cpu().numpy(), want)
    # split along the sequence (needs the length hint), same tolerance
    out2 = torch.full_like(out, float("nan"))
    kv.batch_decode_i4(out2, gpu(q), *args, layer, max_seq_len=max(lens))
    assert close(out2.cpu().numpy(), want)
    # a sequence of one token returns its value vector, dequantised
    if 1 in lens:
        b = lens.index(1)
        _, _, vc, vp = o.paged_gather(data, param, indptr, indices, last, layer, b)
        assert close(out[b].cpu().numpy(), o.paged_dequant(vc, vp)[0])


def test_decode_attention_of_a_sequence_without_pages_reads_nothing():
    """A sequence whose page list is empty (it is the LAST one, so its slice of kv_indices starts at the list's end)
    gets the empty softmax, 0 / 0 = NaN, as in the reference's kernel; the other sequences are unaffected.  With the
    split along the sequence as well.  A cache without any page is refused before the launch."""
    rng = np.random.default_rng(3)
    heads, layer, page_size, lens = 3, 0, 16, [40, 7]
    data, param, indptr, indices, last = paged_case(rng, heads, page_size, lens, layers=1)
    q = rng.standard_normal((3, heads, 128)).astype(F16)
    want = o.paged_batch_decode(q[:2], data, param, indptr, indices, last, layer)
    indptr3 = np.concatenate([indptr, indptr[-1:]]).astype(np.int32)        # third sequence: no pages
    last3 = np.concatenate([last, [0]]).astype(np.int32)
    used = gpu(indices[: indptr[-1]])                                       # the list ends where the empty slice starts
    for hint in (None, 40):
        out = torch.zeros((3, heads, 128), dtype=torch.float16, device="cuda:0")
        kw = {} if hint is None else {"max_seq_len": hint}
        kv.batch_decode_i4(out, gpu(q), gpu(data), gpu(param), gpu(indptr3), used, gpu(last3), layer, **kw)
        got = out.cpu().numpy()
        assert close(got[:2], want) and np.isnan(got[2]).all()
    L, st = _lib.lib(), torch.cuda.current_stream().cuda_stream
    out = torch.zeros((3, heads, 128), dtype=torch.float16, device="cuda:0")
    gq, gd, gp, gi, gl = gpu(q), gpu(data), gpu(param), gpu(indptr3), gpu(last3)
    rc = L.qr_batch_decode_i4(out.data_ptr(), gq.data_ptr(), gd.data_ptr(), gp.data_ptr(), gi.data_ptr(), used.data_ptr(),
                              gl.data_ptr(), 0, 1, 0, heads, page_size, 128, 3, 0, None, 0, st)
    assert rc == -2, rc                                                     # QR_E_SHAPE: sequences but no page pool


@pytest.mark.parametrize("page_size,lens", [(16, [1, 33, 700, 4100]), (5, [11, 64])])
def test_decode_attention_with_the_querys_hadamard_inside(page_size, lens):
    """q_hadamard=True: the kernel transforms the raw query itself.  Against the oracle on the oracle's own
    transform of q (kv_hadamard: float64 sums, 1 / sqrt(128), fp16), and against the two-launch form
    (matmul_had_cuda, then batch_decode_i4) -- with and without the split along the sequence, and through
    the C entry point."""
    rng = np.random.default_rng(page_size + 9)
    heads, layer = 6, 0
    data, param, indptr, indices, last = paged_case(rng, heads, page_size, lens, layers=1)
    q = (rng.standard_normal((len(lens), heads, 128)) * 2).astype(F16)
    q[0, 0, :] = 0
    q[1, 2, 5] = 40.0
    qh = o.kv_hadamard(q)
    want = o.paged_batch_decode(qh, data, param, indptr, indices, last, layer)
    args = (gpu(data), gpu(param), gpu(indptr), gpu(indices), gpu(last))
    two = torch.empty((len(lens), heads, 128), dtype=torch.float16, device="cuda:0")
    kv.batch_decode_i4(two, kv.matmul_had_cuda(gpu(q), torch.float16), *args, layer)
    for hint in (0, max(lens)):
        out = torch.full_like(two, float("nan"))
        kv.batch_decode_i4(out, gpu(q), *args, layer, max_seq_len=hint, q_hadamard=True)
        assert close(out.cpu().numpy(), want)
        assert close(out.cpu().numpy(), two.cpu().numpy())
    L = _lib.lib()
    out = torch.full_like(two, float("nan"))
    gq = gpu(q)
    rc = L.qr_batch_decode_qhad_i4(out.data_ptr(), gq.data_ptr(), args[0].data_ptr(), args[1].data_ptr(), args[2].data_ptr(),
                                   args[3].data_ptr(), args[4].data_ptr(), args[0].shape[0], 1, 0, heads, page_size, 128, len(lens), 0,
                                   None, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0 and close(out.cpu().numpy(), want)
    assert L.qr_batch_decode_qhad_i4(None, gq.data_ptr(), args[0].data_ptr(), args[1].data_ptr(), args[2].data_ptr(), args[3].data_ptr(),
                                     args[4].data_ptr(), args[0].shape[0], 1, 0, heads, page_size, 128, len(lens), 0, None, 0, None) == -1


def test_decode_attention_real_quantised_cache_and_split_workspace():
    """A cache filled by the quantiser from N(0,1) keys and values with outliers (config 5's statistics),
    page size 16, 2 sequences x 8 heads x 1500 tokens: few workgroups, so the entry point splits the
    sequence; the C entry point is called with and without workspace."""
    rng = np.random.default_rng(3)
    heads, P, lens = 8, 16, [1500, 1203]
    data, param, indptr, indices, last = paged_case(rng, heads, P, lens, layers=1)
    app = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    k, v = synth_kv(rng, sum(lens), heads), synth_kv(rng, sum(lens), heads)
    gd, gp = gpu(data), gpu(param)
    tabs = (gpu(indptr), gpu(indices), gpu(last))
    kv.quantize_append_kv_i4(gd, gp, *tabs, gpu(k), gpu(v), gpu(app), 0, hadamard=True)
    q = kv.matmul_had_cuda(gpu(rng.standard_normal((2, heads, 128)).astype(F16)), torch.float16)
    want = o.paged_batch_decode(q.cpu().numpy(), gd.cpu().numpy(), gp.cpu().numpy(), indptr, indices, last, 0)
    L = _lib.lib()
    ws_bytes = L.qr_batch_decode_workspace_bytes(2, heads, 1500)
    assert ws_bytes > 0 and L.qr_batch_decode_workspace_bytes(2, heads, 0) == 0
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda:0")
    st = torch.cuda.current_stream().cuda_stream
    outs = []
    for wptr, wbytes in ((ws.data_ptr(), ws_bytes), (None, 0), (ws.data_ptr(), ws_bytes - 8)):
        out = torch.full((2, heads, 128), float("nan"), dtype=torch.float16, device="cuda:0")
        rc = L.qr_batch_decode_i4(out.data_ptr(), q.data_ptr(), gd.data_ptr(), gp.data_ptr(), tabs[0].data_ptr(), tabs[1].data_ptr(),
                                  tabs[2].data_ptr(), gd.shape[0], 1, 0, heads, P, 128, 2, 1500, wptr, wbytes, st)
        assert rc == 0
        outs.append(out.cpu().numpy())
        assert close(outs[-1], want)
    assert np.array_equal(outs[1], outs[2])                              # too small a workspace = no workspace
    # attention over dequantised values tracks attention over the original fp16 values (what the cache is for)
    kh = kv.matmul_had_cuda(gpu(k), torch.float16).float()
    for b in range(2):
        ks, vs = kh[app[b]:app[b + 1]], gpu(v)[app[b]:app[b + 1]].float()
        w = torch.softmax(torch.einsum("hd,shd->hs", q[b].float(), ks) / np.sqrt(128.0), dim=1)
        ref = torch.einsum("hs,shd->hd", w, vs).cpu().numpy()
        err = outs[0][b].astype(F32) - ref                               # int4 noise of values with x15 outliers
        assert np.linalg.norm(err) < 0.35 * np.linalg.norm(ref)


def test_page_numbers_outside_the_pool_are_skipped():
    """The index arrays live on the device and cannot be validated by the host: a page number outside
    [0, num_pages) must be skipped (its tokens count as absent), never dereferenced."""
    rng = np.random.default_rng(9)
    heads, P, lens = 2, 16, [48, 32]
    data, param, indptr, indices, last = paged_case(rng, heads, P, lens, layers=1)
    q = rng.standard_normal((2, heads, 128)).astype(F16)
    bad = indices.copy()
    bad[indptr[0] + 2] = data.shape[0]                                   # sequence 0's last page: one past the pool
    out = torch.empty((2, heads, 128), dtype=torch.float16, device="cuda:0")
    kv.batch_decode_i4(out, gpu(q), gpu(data), gpu(param), gpu(indptr), gpu(bad), gpu(last), 0)
    ind0 = np.concatenate([indptr[:1], indptr[1:] - 1]).astype(np.int32)    # the same cache with sequence 0 cut to 2 pages
    idx0 = np.delete(indices, indptr[0] + 2)
    want = o.paged_batch_decode(q, data, param, ind0, idx0, np.array([16, last[1]], np.int32), 0)
    assert close(out.cpu().numpy(), want)
    gd, gp = gpu(data), gpu(param)
    k = rng.integers(0, 256, (2, heads, 64), dtype=np.uint8)
    kp = rng.standard_normal((2, heads, 2)).astype(F16)
    kv.append_kv_i4(gd, gp, gpu(indptr), gpu(bad), gpu(last), gpu(k), gpu(k), gpu(kp), gpu(kp), 0)
    o.paged_append(data, param, indptr[1:] - indptr[1], indices[indptr[1]:], last[1:], k[1:], k[1:], kp[1:], kp[1:], 0, None)
    assert np.array_equal(gd.cpu().numpy(), data)                         # only sequence 1's token was written


def test_argument_errors_of_the_python_mirror_and_the_c_entry_points():
    rng = np.random.default_rng(1)
    data, param, indptr, indices, last = paged_case(rng, 2, 16, [20, 5], layers=1)
    gd, gp, gi, gx, gl = gpu(data), gpu(param), gpu(indptr), gpu(indices), gpu(last)
    q = gpu(rng.standard_normal((2, 2, 128)).astype(F16))
    out = torch.empty_like(q)
    with pytest.raises(RuntimeError, match="uint8"):
        kv.batch_decode_i4(out, q, gd.to(torch.float16), gp, gi, gx, gl, 0)
    with pytest.raises(RuntimeError, match="head_dim"):
        kv.batch_decode_i4(out, q, gd[..., :32].contiguous(), gp, gi, gx, gl, 0)
    with pytest.raises(RuntimeError, match="layer_idx"):
        kv.batch_decode_i4(out, q, gd, gp, gi, gx, gl, 1)
    with pytest.raises(RuntimeError, match="contiguous"):
        kv.batch_decode_i4(out, q.transpose(0, 1), gd, gp, gi, gx, gl, 0)
    with pytest.raises(RuntimeError, match="batch_size"):
        kv.batch_decode_i4(out, q, gd, gp, gi[:2], gx, gl, 0)
    with pytest.raises(RuntimeError, match="one token per sequence"):
        kv.append_kv_i4(gd, gp, gi, gx, gl, gd.new_zeros(3, 2, 64), gd.new_zeros(3, 2, 64), gp.new_zeros(3, 2, 2), gp.new_zeros(3, 2, 2), 0)
    L = _lib.lib()
    st = torch.cuda.current_stream().cuda_stream
    a = (gd.data_ptr(), gp.data_ptr(), gi.data_ptr(), gx.data_ptr(), gl.data_ptr())
    assert L.qr_batch_decode_i4(out.data_ptr(), q.data_ptr(), *a, gd.shape[0], 1, 0, 2, 16, 64, 2, 0, None, 0, st) == -3   # head_dim
    assert L.qr_batch_decode_i4(out.data_ptr(), q.data_ptr(), *a, gd.shape[0], 1, 2, 2, 16, 128, 2, 0, None, 0, st) == -2  # layer
    assert L.qr_batch_decode_i4(None, q.data_ptr(), *a, gd.shape[0], 1, 0, 2, 16, 128, 2, 0, None, 0, st) == -1
    assert L.qr_batch_decode_i4(out.data_ptr(), q.data_ptr(), *a, gd.shape[0], 1, 0, 2, 16, 128, 0, 0, None, 0, st) == 0    # empty batch
    assert L.qr_kv_append_i4(*a, gd.shape[0], gd.data_ptr(), gd.data_ptr(), gp.data_ptr(), gp.data_ptr(), None, 3, 1, 0, 2, 16, 128, 2, st) == -2
    assert L.qr_kv_quant_append_f16_i4(q.data_ptr(), q.data_ptr(), 2, None, 7, *a, gd.shape[0], 1, 0, 2, 16, 128, 2, st) == -5


@pytest.mark.parametrize("hadamard_dtype", [torch.float16, None, torch.float32])
def test_cache_class_prefill_then_decode_steps(hadamard_dtype):
    """MultiLayerPagedKVCache4Bit driven as the model code drives it (e2e/quantized_llama/modeling_llama.py:
    60-81): the prompt through update() (fp16 states come back for the prefill's own attention), then two
    decode steps whose update() returns the attention callable.  Checked against the oracle pipeline:
    Hadamard (kernel's own output) -> oracle quantiser -> oracle append -> oracle attention."""
    rng = np.random.default_rng(17)
    B, H, P, L, prompt = 3, 4, 16, 2, 37
    cache = kv.MultiLayerPagedKVCache4Bit(batch_size=B, page_size=P, max_seq_len=64, device="cuda:0", n_layers=L, num_heads=H,
                                          head_dim=128, hadamard_dtype=hadamard_dtype)
    assert cache.pages.shape == (4 * B, L, 2, H, P, 64) and cache.scales.shape == (4 * B, L, 2, H, P, 2)
    cache.pages.zero_(); cache.scales.zero_()
    data, param = np.zeros(cache.pages.shape, np.uint8), np.zeros(cache.scales.shape, F16)

    def had(x):                     # the kernel's own transform, in the dtype the cache was told to use
        if hadamard_dtype is None:
            return x
        return kv.matmul_had_cuda(gpu(x), hadamard_dtype).cpu().numpy()

    def oracle_store(k, v, layer, length, added):
        spec_len = np.full(B, length, np.int64)
        pc = -(-length // P)
        indptr = (np.arange(B + 1) * pc).astype(np.int32)
        indices = (np.arange(pc)[None, :] * B + np.arange(B)[:, None]).reshape(-1).astype(np.int32)
        last = np.full(B, length - (pc - 1) * P, np.int32)
        kq, ks, kz = o.kv_asym_quant(had(k).reshape(-1, H, 128))
        vq, vs, vz = o.kv_asym_quant(v.reshape(-1, H, 128))
        app = (np.arange(B + 1) * added).astype(np.int32)
        o.paged_append(data, param, indptr, indices, last, kq, vq, np.concatenate([ks, kz], -1), np.concatenate([vs, vz], -1), layer,
                       app if added > 1 else None)
        return indptr, indices, last

    kpr, vpr = synth_kv(rng, B * prompt, H).reshape(B, prompt, H, 128), synth_kv(rng, B * prompt, H).reshape(B, prompt, H, 128)
    for layer in range(L):
        ret = cache.update(gpu(kpr), gpu(vpr), layer, {})
        assert isinstance(ret, tuple) and torch.equal(ret[0], gpu(kpr)) and torch.equal(ret[1], gpu(vpr))
        oracle_store(kpr, vpr, layer, prompt, prompt)
    assert cache.get_seq_length() == prompt and cache.seen_tokens == prompt
    assert np.array_equal(cache.pages.cpu().numpy(), data) and np.array_equal(bits(cache.scales.cpu().numpy()), bits(param))
    for step in range(2):
        k1, v1 = synth_kv(rng, B, H).reshape(B, 1, H, 128), synth_kv(rng, B, H).reshape(B, 1, H, 128)
        qs = rng.standard_normal((B, 1, H, 128)).astype(F16)
        for layer in range(L):
            fn = cache.update(gpu(k1), gpu(v1), layer, {})
            assert callable(fn)
            tabs = oracle_store(k1, v1, layer, prompt + step + 1, 1)
            attn = fn(gpu(qs))
            assert attn.shape == (B, 1, H, 128) and attn.dtype == torch.float16
            want = o.paged_batch_decode(had(qs.reshape(B, H, 128)), data, param, *tabs, layer)
            assert close(attn.cpu().numpy().reshape(B, H, 128), want)
        assert np.array_equal(cache.pages.cpu().numpy(), data)
    assert cache.get_seq_length() == prompt + 2 and cache.to_legacy_cache() is cache and cache.get_max_length() is None


def test_cache_class_padded_prompt_and_the_reference_benchmarks_fake_prefill():
    """A left-padded prompt (attention_mask): only the rows the mask keeps enter the cache
    (kv_cache.py:206-220).  And the way benchmarks/qattention_benchmark.py:53-57 drives the cache: no
    prefill, length set by hand, one page per sequence."""
    rng = np.random.default_rng(23)
    B, H, P, T = 2, 2, 32, 20
    cache = kv.MultiLayerPagedKVCache4Bit(B, P, 32, "cuda:0", 1, H, 128)
    cache.pages.zero_(); cache.scales.zero_()
    mask = torch.ones(B, T, dtype=torch.int64)
    mask[0, :4] = 0
    mask[1, :4] = 0                                                      # equal page counts are required by the class
    k, v = synth_kv(rng, B * T, H).reshape(B, T, H, 128), synth_kv(rng, B * T, H).reshape(B, T, H, 128)
    cache.update(gpu(k), gpu(v), 0, {"attention_mask": mask.to("cuda:0")})
    kh = kv.matmul_had_cuda(gpu(k), torch.float16).cpu().numpy()
    kq, ks, kz = o.kv_asym_quant(kh[:, 4:].reshape(-1, H, 128))
    vq, vs, vz = o.kv_asym_quant(v[:, 4:].reshape(-1, H, 128))
    data, param = np.zeros(cache.pages.shape, np.uint8), np.zeros(cache.scales.shape, F16)
    indptr, indices, last = np.array([0, 1, 2], np.int32), np.array([0, 1], np.int32), np.array([16, 16], np.int32)
    o.paged_append(data, param, indptr, indices, last, kq, vq, np.concatenate([ks, kz], -1), np.concatenate([vs, vz], -1), 0,
                   np.array([0, 16, 32], np.int32))
    assert np.array_equal(cache.pages.cpu().numpy(), data) and np.array_equal(bits(cache.scales.cpu().numpy()), bits(param))
    # qattention_benchmark.py:39-57
    seq_len = 96
    cache = kv.MultiLayerPagedKVCache4Bit(batch_size=B, page_size=seq_len, max_seq_len=seq_len, device=torch.device("cuda:0"),
                                          n_layers=1, num_heads=H, head_dim=128, disable_quant=False, hadamard_dtype=torch.float16)
    cache.pages.copy_(gpu(rng.integers(0, 256, tuple(cache.pages.shape), dtype=np.uint8)))
    cache.scales.copy_(gpu((np.abs(rng.standard_normal(tuple(cache.scales.shape))) * 0.05 + 0.01).astype(F16)))
    query_states = torch.rand((B, 1, H, 128), device="cuda:0", dtype=torch.float16)
    key_states, value_states = torch.rand_like(query_states), torch.rand_like(query_states)
    cache._needs_init = [False] * len(cache._needs_init)
    cache.length = seq_len - 1
    forward_func = cache.update(key_states, value_states, layer_idx=0, cache_kwargs={})
    attn_out = forward_func(query_states)
    qh = kv.matmul_had_cuda(query_states.view(B, H, 128), torch.float16).cpu().numpy()
    want = o.paged_batch_decode(qh, cache.pages.cpu().numpy(), cache.scales.cpu().numpy(), np.array([0, 1, 2], np.int32),
                                np.array([0, 1], np.int32), np.array([seq_len, seq_len], np.int32), 0)
    assert close(attn_out.cpu().numpy().reshape(B, H, 128), want)


def test_cache_class_long_sequence_small_batch_keeps_one_scratch_buffer():
    """One sequence of 1500+ tokens, 8 heads: decode attention is split along the sequence, and the partial states go
    through the scratch buffer that the cache keeps (one allocation, reused by every step and layer).  Three decode
    steps of two layers each against the oracle on the cache's own pages."""
    B, H, P, S0, L = 1, 8, 16, 1500, 2
    g = torch.Generator().manual_seed(12)
    cache = kv.MultiLayerPagedKVCache4Bit(B, P, S0 + 8, "cuda:0", L, H, 128)
    assert kv._decode_workspace_bytes(B, H, S0 + 8, 0) > 0                 # this shape does split
    for layer in range(L):
        k = torch.randn(B, S0, H, 128, generator=g).half().cuda()
        v = torch.randn(B, S0, H, 128, generator=g).half().cuda()
        cache.update(k, v, layer, {})
    seen = set()
    for step in range(3):
        for layer in range(L):
            k1 = torch.randn(B, 1, H, 128, generator=g).half().cuda()
            v1 = torch.randn(B, 1, H, 128, generator=g).half().cuda()
            q1 = torch.randn(B, 1, H, 128, generator=g).half().cuda()
            out = cache.update(k1, v1, layer, {})(q1)
            seen.add(cache._decode_ws.data_ptr())
            specs = cache.get_cache_specs_for_flash_infer(None)
            qh = kv.matmul_had_cuda(q1.view(B, H, 128), torch.float16).cpu().numpy()
            want = o.paged_batch_decode(qh, cache.pages.cpu().numpy(), cache.scales.cpu().numpy(),
                                        *[specs[n].cpu().numpy() for n in ("kv_indptr", "kv_indices", "last_page_offset")], layer)
            assert out.shape == (B, 1, H, 128) and close(out.cpu().numpy().reshape(B, H, 128), want)
    assert len(seen) == 1 and cache.length == S0 + 3


def test_decode_attention_at_config5_size():
    """The cache of config 5 (32 sequences x 4096 tokens x 8 KV heads x 128) in pages of 16: filled by the
    fused quantise-and-append, read by decode attention; sampled (sequence, head) pairs against the oracle,
    every output against the property that it is a convex combination of the sequence's V vectors."""
    B, S, H, P = 32, 4096, 8, 16
    g = torch.Generator().manual_seed(4)
    k = torch.randn(B, S, H, 128, generator=g)
    mask = torch.rand(k.shape, generator=torch.Generator().manual_seed(5)) < 0.005
    k[mask] *= 15
    v = torch.randn(B, S, H, 128, generator=torch.Generator().manual_seed(6))
    v[mask] *= 15
    k, v = k.half().cuda(), v.half().cuda()
    cache = kv.MultiLayerPagedKVCache4Bit(B, P, S, "cuda:0", 1, H, 128)
    cache.update(k, v, 0, {})
    q = torch.randn(B, 1, H, 128, generator=torch.Generator().manual_seed(7)).half().cuda()
    specs = cache.get_cache_specs_for_flash_infer(None)
    qh = kv.matmul_had_cuda(q.view(B, H, 128), torch.float16)
    out = torch.empty_like(qh)
    kv.batch_decode_i4(out, qh, **specs, layer_idx=0)
    tabs = [specs[n].cpu().numpy() for n in ("kv_indptr", "kv_indices", "last_page_offset")]
    pages, scales = cache.pages.cpu().numpy(), cache.scales.cpu().numpy()
    for b in (0, 13, 31):
        one = (tabs[0][b:b + 2] - tabs[0][b], tabs[1][tabs[0][b]:tabs[0][b + 1]], tabs[2][b:b + 1])
        want = o.paged_batch_decode(qh[b:b + 1].cpu().numpy(), pages, scales, *one, 0)
        assert close(out[b:b + 1].cpu().numpy(), want)
    vd = kv.unpack_i4_and_asym_dequantize(*kv.asym_quantize_and_pack_i4(v)).float()      # [B, S, H, 128]
    lo, hi = vd.amin(dim=1), vd.amax(dim=1)
    assert bool(((out.float() >= lo - 2e-2) & (out.float() <= hi + 2e-2)).all())
