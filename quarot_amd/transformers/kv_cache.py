"""KV-cache path (mirror of quarot/transformers/kv_cache.py) on HIP kernels: the asymmetric int4
quantiser and its inverse, the paged int4 cache (append, quantise-and-append, single-query attention over
the cache) and the cache class the model code drives; and the same cache with fp16 pages (the reference's
disable_quant mode: init_kv_f16 / append_kv_f16 / batch_decode_f16)."""
import functools
import math
import weakref

import torch


from .. import _lib
from ..functional.hadamard import hadamard_transform


def _vectors(x, name):
    if x.dtype != torch.float16:
        raise RuntimeError(f"{name}: expected an fp16 tensor, got {x.dtype}")
    if not x.is_cuda:
        raise RuntimeError(f"{name}: expected a GPU tensor, got {x.device}")
    xc = x.contiguous()
    dim = xc.shape[-1]
    return xc, dim, (xc.numel() // dim if dim else 0)


def asym_quantize_and_pack_i4(x: torch.Tensor, hadamard: bool = False):
    """Per last-axis vector: scale = (max - min).clamp(1e-5) / 15, zero = -min,
    q = clamp(round((x + zero) / scale), 0, 15), packed low nibble first.
    Returns (q uint8 [..., D/2], scale fp16 [..., 1], zero fp16 [..., 1]) (kv_cache.py:10-22).
    hadamard=True first applies matmul_had_cuda(x, fp16) in the same kernel (kv_cache.py:188-189)."""
    xc, dim, vecs = _vectors(x, "asym_quantize_and_pack_i4")
    lead = xc.shape[:-1]
    q = torch.empty((*lead, dim // 2), dtype=torch.uint8, device=xc.device)
    scale = torch.empty((*lead, 1), dtype=torch.float16, device=xc.device)
    zero = torch.empty((*lead, 1), dtype=torch.float16, device=xc.device)
    with _lib.on_device(xc.device):
        _lib.check(_lib.lib().qr_kv_quant_f16_i4(xc.data_ptr(), vecs, dim, 1 if hadamard else 0, q.data_ptr(),
                                                 scale.data_ptr(), zero.data_ptr(), _lib.stream_ptr(xc.device)))
    return q, scale, zero


def unpack_i4_and_asym_dequantize(q, scale, zero):
    """q * scale - zero in fp16 after unpacking (kv_cache.py:24-28)."""
    assert q.dtype == torch.uint8
    if not q.is_cuda:
        raise RuntimeError("unpack_i4_and_asym_dequantize: expected GPU tensors")
    qc, sc, zc = q.contiguous(), scale.contiguous(), zero.contiguous()
    if sc.dtype != torch.float16 or zc.dtype != torch.float16:
        raise RuntimeError("unpack_i4_and_asym_dequantize: scale and zero must be fp16")
    half_dim = qc.shape[-1]
    vecs = qc.numel() // half_dim if half_dim else 0
    if sc.numel() != vecs or zc.numel() != vecs:
        raise RuntimeError("unpack_i4_and_asym_dequantize: one scale and zero per vector expected")
    y = torch.empty((*qc.shape[:-1], half_dim * 2), dtype=torch.float16, device=qc.device)
    with _lib.on_device(qc.device):
        _lib.check(_lib.lib().qr_kv_dequant_i4_f16(qc.data_ptr(), sc.data_ptr(), zc.data_ptr(), vecs, half_dim * 2,
                                                   y.data_ptr(), _lib.stream_ptr(qc.device)))
    return y


def matmul_had_cuda(X, dtype):
    """FWHT over the last axis scaled by 1/sqrt(n), computed in `dtype`, returned in X's dtype
    (kv_cache.py:30-33)."""
    n = X.shape[-1]
    out = hadamard_transform(X.to(dtype).contiguous(), scale=1 / math.sqrt(n))
    return out.to(X.dtype).view(X.shape)


# ---------------------------------------------------------------------------------------------------
# paged int4 cache: kv_data uint8 [pages, layers, 2, heads, page_size, head_dim / 2],
# kv_param fp16 [pages, layers, 2, heads, page_size, 2] = {scale, zero}

_CHECKED = None     # the five cache tensors validated last (weak references), their element counts, their dimensions


def _cache_args(fn, kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, layer_idx, f16=False):
    """The checks of quarot/kernels/bindings.cpp:118-374 (CHECK_INPUT / CHECK_DIM / CHECK_EQ) as RuntimeError; f16: the
    cache with fp16 pages (the *_f16 bindings).
    A decode step passes the same five tensor objects to the append and to the attention of every layer: the
    objects validated last (same identity, same element counts) are not walked through again."""
    global _CHECKED
    seen = _CHECKED
    if seen is not None:
        refs, counts, dims = seen
        if (refs[0]() is kv_data and refs[1]() is kv_param and refs[2]() is kv_indptr and refs[3]() is kv_indices
                and refs[4]() is last_page_offset and kv_data.dtype == (torch.float16 if f16 else torch.uint8)
                and counts == (kv_data.numel(), kv_param.numel(), kv_indptr.numel(), kv_indices.numel(), last_page_offset.numel())):
            if not (0 <= int(layer_idx) < dims[1]):
                raise RuntimeError(f"{fn}: layer_idx out of range")
            return dims
    for name, t in (("kv_data", kv_data), ("kv_param", kv_param), ("kv_indptr", kv_indptr), ("kv_indicies", kv_indices),
                    ("last_page_offset", last_page_offset)):
        if not (t.is_cuda):
            raise RuntimeError(f"{fn}: {name} must be a CUDA tensor")
        if not (t.is_contiguous()):
            raise RuntimeError(f"{fn}: {name} must be contiguous")
    if not (kv_data.dim() == 6):
        raise RuntimeError(f"{fn}: kv_data must be a 6D tensor")
    if not (kv_param.dim() == 6):
        raise RuntimeError(f"{fn}: kv_param must be a 6D tensor")
    if not (kv_indptr.dim() == 1 and kv_indices.dim() == 1 and last_page_offset.dim() == 1):
        raise RuntimeError(f"{fn}: kv_indptr, kv_indicies and last_page_offset must be 1D tensors")
    if not (kv_data.dtype == (torch.float16 if f16 else torch.uint8)):
        raise RuntimeError(f"{fn}: kv_data must be {'fp16' if f16 else 'uint8'}")
    if not (kv_param.dtype == torch.float16):
        raise RuntimeError(f"{fn}: kv_param must be fp16")
    for name, t in (("kv_indptr", kv_indptr), ("kv_indicies", kv_indices), ("last_page_offset", last_page_offset)):
        if not (t.dtype == torch.int32):
            raise RuntimeError(f"{fn}: {name} must be int32")
    pages, layers, two, heads, page_size, half_dim = kv_data.shape
    if not (two == 2 and tuple(kv_param.shape) == (pages, layers, 2, heads, page_size, 2)):
        raise RuntimeError(f"{fn}: kv_param must be [pages, layers, 2, heads, page_size, 2]")
    head_dim = half_dim if f16 else half_dim * 2           # (the last axis holds halves or packed pairs of codes)
    if not (head_dim == 128):
        raise RuntimeError(f"{fn}: CHECK_EQ(head_dim, 128) failed. {head_dim} vs 128")
    if not (0 <= int(layer_idx) < layers):
        raise RuntimeError(f"{fn}: layer_idx out of range")
    dims = (pages, layers, heads, page_size, head_dim)
    five = (kv_data, kv_param, kv_indptr, kv_indices, last_page_offset)
    _CHECKED = (tuple(weakref.ref(t) for t in five), tuple(t.numel() for t in five), dims)
    return dims


def _append(fn, kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, k_param, v_param, seqlen_indptr, layer_idx,
            f16=False):
    pages, layers, heads, page_size, head_dim = _cache_args(fn, kv_data, kv_param, kv_indptr, kv_indices, last_page_offset,
                                                            layer_idx, f16)
    batch = last_page_offset.shape[0]
    if not (kv_indptr.shape[0] == batch + 1):
        raise RuntimeError(f"{fn}: CHECK_EQ(kv_indptr.size(0), batch_size + 1) failed")
    for name, t in (("k", k), ("v", v), ("k_param", k_param), ("v_param", v_param)):
        if not (t.is_cuda and t.is_contiguous() and t.dim() == 3):
            raise RuntimeError(f"{fn}: {name} must be a contiguous 3D CUDA tensor")
    if f16:
        if not (k.shape == v.shape and k.dtype == v.dtype == torch.float16 and tuple(k.shape[1:]) == (heads, head_dim)):
            raise RuntimeError(f"{fn}: k and v must be fp16 [tokens, heads, head_dim]")
    elif not (k.shape == v.shape and k.dtype == v.dtype == torch.uint8 and tuple(k.shape[1:]) == (heads, head_dim // 2)):
        raise RuntimeError(f"{fn}: k and v must be uint8 [tokens, heads, head_dim / 2]")
    tokens = k.shape[0]
    for name, t in (("k_param", k_param), ("v_param", v_param)):
        if not (t.dtype == torch.float16 and tuple(t.shape) == (tokens, heads, 2)):
            raise RuntimeError(f"{fn}: {name} must be fp16 [tokens, heads, 2]")
    if seqlen_indptr is None:
        if not (tokens == batch):
            raise RuntimeError(f"{fn}: one token per sequence expected")
    else:
        if not (seqlen_indptr.is_cuda and seqlen_indptr.is_contiguous() and seqlen_indptr.dtype == torch.int32 and tuple(seqlen_indptr.shape) == (batch + 1,)):
            raise RuntimeError(f"{fn}: seqlen_indptr must be int32 [batch_size + 1]")
    dev = kv_data.device
    with _lib.on_device(dev):
        entry = _lib.lib().qr_kv_append_f16 if f16 else _lib.lib().qr_kv_append_i4
        _lib.check(entry(
            kv_data.data_ptr(), kv_param.data_ptr(), kv_indptr.data_ptr(), kv_indices.data_ptr(), last_page_offset.data_ptr(),
            pages, k.data_ptr(), v.data_ptr(), k_param.data_ptr(), v_param.data_ptr(),
            None if seqlen_indptr is None else seqlen_indptr.data_ptr(), tokens, layers, int(layer_idx), heads, page_size,
            head_dim, batch, _lib.stream_ptr(dev)))


def init_kv_i4(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, k_param, v_param, seqlen_indptr, layer_idx):
    """Write the quantised K / V vectors of a prompt into their pages (kv_cache.py:36-46 ->
    bindings.cpp:155-198): the tokens seqlen_indptr[b] .. seqlen_indptr[b + 1] - 1 of sequence b become the
    last positions of that sequence.  Returns None, like the reference's binding."""
    _append("init_kv_i4", kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, k_param, v_param, seqlen_indptr,
            layer_idx)


def append_kv_i4(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, k_param, v_param, layer_idx):
    """Write one new quantised K / V vector per sequence at its last position (kv_cache.py:49-58 ->
    bindings.cpp:200-245)."""
    _append("append_kv_i4", kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, k_param, v_param, None, layer_idx)


def init_kv_f16(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, k_param, v_param, seqlen_indptr, layer_idx):
    """init_kv_i4 for the cache with fp16 pages (kv_cache.py:69-79 -> bindings.cpp:287-330): k, v fp16
    [tokens, heads, 128], kv_data fp16 [pages, layers, 2, heads, page_size, 128]."""
    _append("init_kv_f16", kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, k_param, v_param, seqlen_indptr,
            layer_idx, f16=True)


def append_kv_f16(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, k_param, v_param, layer_idx):
    """append_kv_i4 for the cache with fp16 pages (kv_cache.py:82-91 -> bindings.cpp:332-374)."""
    _append("append_kv_f16", kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, k_param, v_param, None, layer_idx,
            f16=True)


def batch_decode_f16(o, q, kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, layer_idx):
    """o[b, h] = softmax(q[b, h] . K^T / sqrt(128)) . V over the fp16 pages of sequence b (kv_cache.py:93-101 ->
    bindings.cpp:247-285).  Writes into `o` and returns None, like the reference's binding."""
    fn = "batch_decode_f16"
    pages, layers, heads, page_size, head_dim = _cache_args(fn, kv_data, kv_param, kv_indptr, kv_indices, last_page_offset,
                                                            layer_idx, f16=True)
    for name, t in (("o", o), ("q", q)):
        if not (t.is_cuda and t.is_contiguous() and t.dim() == 3 and t.dtype == torch.float16):
            raise RuntimeError(f"{fn}: {name} must be a contiguous 3D fp16 CUDA tensor")
    if not (o.shape == q.shape):
        raise RuntimeError(f"{fn}: o.size() != q.size()")
    batch = o.shape[0]
    if not (tuple(q.shape[1:]) == (heads, head_dim)):
        raise RuntimeError(f"{fn}: q must be [batch_size, {heads}, {head_dim}]")
    if not (kv_indptr.shape[0] == batch + 1):
        raise RuntimeError(f"{fn}: CHECK_EQ(kv_indptr.size(0), batch_size + 1) failed")
    if not (last_page_offset.shape[0] == batch):
        raise RuntimeError(f"{fn}: CHECK_EQ(last_page_offset.size(0), batch_size) failed")
    dev = kv_data.device
    with _lib.on_device(dev):
        _lib.check(_lib.lib().qr_batch_decode_f16(
            o.data_ptr(), q.data_ptr(), kv_data.data_ptr(), kv_param.data_ptr(), kv_indptr.data_ptr(), kv_indices.data_ptr(),
            last_page_offset.data_ptr(), pages, layers, int(layer_idx), heads, page_size, head_dim, batch, _lib.stream_ptr(dev)))


def quantize_append_kv_i4(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, seqlen_indptr, layer_idx,
                          hadamard=True):
    """fp16 K and V [tokens, heads, 128] -> (Hadamard over the head dimension of K) -> asymmetric int4 ->
    straight into the pages: matmul_had_cuda + asym_quantize_and_pack_i4 (twice) + the two torch.cat +
    init_kv_i4 / append_kv_i4 of MultiLayerPagedKVCache4Bit.update (kv_cache.py:174-251) as one launch,
    with the same codes, scales and zeros.  seqlen_indptr None: one token per sequence."""
    fn = "quantize_append_kv_i4"
    pages, layers, heads, page_size, head_dim = _cache_args(fn, kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, layer_idx)
    batch = last_page_offset.shape[0]
    if not (kv_indptr.shape[0] == batch + 1):
        raise RuntimeError(f"{fn}: CHECK_EQ(kv_indptr.size(0), batch_size + 1) failed")
    for name, t in (("k", k), ("v", v)):
        if not (t.is_cuda and t.is_contiguous() and t.dtype == torch.float16 and t.dim() == 3 and tuple(t.shape[1:]) == (heads, head_dim)):
            raise RuntimeError(f"{fn}: {name} must be a contiguous fp16 [tokens, heads, 128] CUDA tensor")
    if not (k.shape == v.shape):
        raise RuntimeError(f"{fn}: k and v differ in shape")
    tokens = k.shape[0]
    if seqlen_indptr is None:
        if not (tokens == batch):
            raise RuntimeError(f"{fn}: one token per sequence expected")
    else:
        if not (seqlen_indptr.is_cuda and seqlen_indptr.is_contiguous() and seqlen_indptr.dtype == torch.int32 and tuple(seqlen_indptr.shape) == (batch + 1,)):
            raise RuntimeError(f"{fn}: seqlen_indptr must be int32 [batch_size + 1]")
    dev = kv_data.device
    with _lib.on_device(dev):
        _lib.check(_lib.lib().qr_kv_quant_append_f16_i4(
            k.data_ptr(), v.data_ptr(), tokens, None if seqlen_indptr is None else seqlen_indptr.data_ptr(), 1 if hadamard else 0,
            kv_data.data_ptr(), kv_param.data_ptr(), kv_indptr.data_ptr(), kv_indices.data_ptr(), last_page_offset.data_ptr(),
            pages, layers, int(layer_idx), heads, page_size, head_dim, batch, _lib.stream_ptr(dev)))


@functools.lru_cache(maxsize=1024)
def _decode_workspace_bytes(batch, heads, max_seq_len, device_index=None):
    # (the split plan depends on the current device's compute-unit count: called with the device current, and
    # the device index is part of the cache key)
    return _lib.lib().qr_batch_decode_workspace_bytes(batch, heads, max_seq_len)


def batch_decode_i4(o, q, kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, layer_idx, max_seq_len=0,
                    q_hadamard=False, workspace=None, append=None):
    """o[b, h] = softmax(q[b, h] . K^T / sqrt(128)) . V over the int4 cache of sequence b, dequantised in
    registers as float(code) * scale - zero (kv_cache.py:60-67 -> bindings.cpp:118-153).  Writes into `o`
    and returns None, like the reference's binding.  max_seq_len (optional, an upper bound of the
    sequence lengths) lets a small batch be split along the sequence.  q_hadamard: `q` is the
    untransformed query and the kernel applies matmul_had_cuda(q, torch.float16) itself (one launch
    instead of two).  workspace: a uint8 tensor on the cache's device to hold the partial states of a split along
    the sequence; one is allocated per call when it is missing or too small.  append = (k, v, hadamard): the fp16
    key and value [batch_size, heads, 128] of the step's new token, which the page tables already count as every
    sequence's last position: the kernel quantises them as quantize_append_kv_i4 would (same codes, scales and zeros,
    written to the same page slots) and attends to them along with the cache -- append and attention in one launch."""
    fn = "batch_decode_i4"
    pages, layers, heads, page_size, head_dim = _cache_args(fn, kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, layer_idx)
    for name, t in (("o", o), ("q", q)):
        if not (t.is_cuda and t.is_contiguous()):
            raise RuntimeError(f"{fn}: {name} must be a contiguous CUDA tensor")
        if not (t.dim() == 3):
            raise RuntimeError(f"{fn}: {name} must be a 3D tensor")
        if not (t.dtype == torch.float16):
            raise RuntimeError(f"{fn}: {name} must be fp16")
    if not (o.shape == q.shape):
        raise RuntimeError(f"{fn}: o.size() != q.size()")
    batch = o.shape[0]
    if not (tuple(q.shape[1:]) == (heads, head_dim)):
        raise RuntimeError(f"{fn}: q must be [batch_size, {heads}, {head_dim}]")
    if not (kv_indptr.shape[0] == batch + 1):
        raise RuntimeError(f"{fn}: CHECK_EQ(kv_indptr.size(0), batch_size + 1) failed")
    if not (last_page_offset.shape[0] == batch):
        raise RuntimeError(f"{fn}: CHECK_EQ(last_page_offset.size(0), batch_size) failed")
    if append is not None:
        for name, t in (("k", append[0]), ("v", append[1])):
            if not (t.is_cuda and t.is_contiguous() and t.dtype == torch.float16 and tuple(t.shape) == (batch, heads, head_dim)):
                raise RuntimeError(f"{fn}: append {name} must be a contiguous fp16 [batch_size, {heads}, {head_dim}] CUDA tensor")
    dev = kv_data.device
    with _lib.on_device(dev):
        ws_bytes = _decode_workspace_bytes(batch, heads, int(max_seq_len), dev.index) if max_seq_len else 0
        ws = None
        if ws_bytes:
            fits = (workspace is not None and workspace.device == dev and workspace.dtype == torch.uint8
                    and workspace.is_contiguous() and workspace.numel() >= ws_bytes)
            ws = workspace if fits else torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
        if append is not None:
            _lib.check(_lib.lib().qr_kv_quant_append_batch_decode_f16_i4(
                o.data_ptr(), q.data_ptr(), 1 if q_hadamard else 0, append[0].data_ptr(), append[1].data_ptr(),
                1 if append[2] else 0, kv_data.data_ptr(), kv_param.data_ptr(), kv_indptr.data_ptr(), kv_indices.data_ptr(),
                last_page_offset.data_ptr(), pages, layers, int(layer_idx), heads, page_size, head_dim, batch, int(max_seq_len),
                None if ws is None else ws.data_ptr(), ws_bytes, _lib.stream_ptr(dev)))
            return
        entry = _lib.lib().qr_batch_decode_qhad_i4 if q_hadamard else _lib.lib().qr_batch_decode_i4
        _lib.check(entry(
            o.data_ptr(), q.data_ptr(), kv_data.data_ptr(), kv_param.data_ptr(), kv_indptr.data_ptr(), kv_indices.data_ptr(),
            last_page_offset.data_ptr(), pages, layers, int(layer_idx), heads, page_size, head_dim, batch, int(max_seq_len),
            None if ws is None else ws.data_ptr(), ws_bytes, _lib.stream_ptr(dev)))


class _AttentionStub(object):
    """What MultiLayerPagedKVCache4Bit.update hands back for a decode step (kv_cache.py:104-129): called
    with the query states it runs attention over the cache."""

    def __init__(self, cache_page_size, device, n_layers, disable_quant, hadamard_dtype):
        self.cache_page_size = cache_page_size
        self.n_layers = n_layers
        self.disable_quant = disable_quant
        self.hadamard_dtype = hadamard_dtype

    def forward(self, q, num_kv_heads, attention_kwargs, layer_idx, max_seq_len=0, workspace=None, take_pending=None):
        batch_size, q_len, num_qo_heads, head_dim = q.shape
        assert q_len == 1
        q = q.view(batch_size, num_qo_heads, head_dim)
        if self.disable_quant:                   # fp16 pages (kv_cache.py:116-119)
            if self.hadamard_dtype is not None:
                q = matmul_had_cuda(q, dtype=self.hadamard_dtype)
            attn_output = torch.empty_like(q)
            batch_decode_f16(attn_output, q.contiguous(), **attention_kwargs, layer_idx=layer_idx)
            return attn_output.unsqueeze(1)
        fused = self.hadamard_dtype == torch.float16 and q.dtype == torch.float16 and q.is_contiguous()
        if self.hadamard_dtype is not None and not fused:
            q = matmul_had_cuda(q, dtype=self.hadamard_dtype)
        attn_output = torch.empty_like(q)
        # the step's new token, if the cache still holds it back for this call (see MultiLayerPagedKVCache4Bit.update)
        append = take_pending() if take_pending is not None else None
        batch_decode_i4(attn_output, q, **attention_kwargs, layer_idx=layer_idx, max_seq_len=max_seq_len, q_hadamard=fused,
                        workspace=workspace, append=append)
        return attn_output.unsqueeze(1)


class MultiLayerPagedKVCache4Bit:
    """Paged int4 KV cache of all layers with the interface of kv_cache.py:132-289: `update` quantises
    and stores the new keys and values (the first call per layer takes the whole prompt and returns the
    fp16 states for the prefill's own attention; later calls take one token per sequence and return a
    callable that runs decode attention over the cache).  Keys pass through the Hadamard transform over
    the head dimension before quantisation, queries before attention (hadamard_dtype, None to skip).
    The reference derives the class from transformers' Cache for the methods that base supplied in the
    version it pins (get_usable_length); they are defined here instead, so the class does not depend on the
    installed transformers version."""

    def __init__(self, batch_size, page_size, max_seq_len, device, n_layers, num_heads, head_dim, disable_quant=False,
                 hadamard_dtype=torch.float16):
        self.page_size = page_size
        self.batch_size = batch_size
        max_page_cnt = self.page_cnt_from_length(max_seq_len)
        self.disable_quant = disable_quant       # fp16 pages instead of int4 codes (kv_cache.py:134-151)
        self._pages = torch.empty((max_page_cnt * batch_size, n_layers, 2, num_heads, page_size,
                                   head_dim if disable_quant else head_dim // 2),
                                  dtype=torch.float16 if disable_quant else torch.uint8, device=device)
        self._scales = torch.empty((max_page_cnt * batch_size, n_layers, 2, num_heads, page_size, 2), dtype=torch.float16,
                                   device=device)
        self._pending = {}      # layer -> (token, k, v, specs, hadamard): a decode step's new token, held for the attention call
        self.max_seq_len = max_seq_len
        self._needs_init = [True] * n_layers
        self.length = 0
        self.device = device
        self.hadamard_dtype = hadamard_dtype
        self._stub = _AttentionStub(self.page_size, device, n_layers, disable_quant=self.disable_quant,
                                    hadamard_dtype=self.hadamard_dtype)

    def page_cnt_from_length(self, length):
        return (length + self.page_size - 1) // self.page_size

    # A decode step's new token is quantised and stored by the attention launch that follows update() (one launch per
    # step instead of two).  Whoever looks at the cache before that call -- the page tensors, the tables, the next
    # update -- first gets the token stored by the quantise-and-append kernel, so the cache never shows a state the
    # reference's would not.  The key and value tensors handed to update() are read by that later launch: they must
    # keep their contents until the returned callable has run (the reference reads them inside update()).
    @property
    def pages(self):
        self._flush()
        return self._pages

    @property
    def scales(self):
        self._flush()
        return self._scales

    def _flush(self, layer_idx=None):
        for layer in ([layer_idx] if layer_idx is not None else list(self._pending)):
            held = self._pending.pop(layer, None)
            if held is not None:
                _, k, v, specs, hadamard = held
                quantize_append_kv_i4(**specs, k=k, v=v, seqlen_indptr=None, layer_idx=layer, hadamard=hadamard)

    def _take_pending(self, layer_idx, token):
        held = self._pending.get(layer_idx)
        if held is None or held[0] is not token:
            return None                          # stored meanwhile (or this callable was used before): plain attention
        del self._pending[layer_idx]
        return held[1], held[2], held[4]

    def _decode_workspace(self, num_heads):
        """Scratch for decode attention split along the sequence, kept with the cache (every layer of every decode
        step would otherwise allocate its own): sized for the longer of the current and the maximum length."""
        key = (self.length, num_heads)
        if getattr(self, "_decode_ws_key", None) == key:
            return self._decode_ws
        dev = self._pages.device
        with _lib.on_device(dev):
            need = max((_decode_workspace_bytes(self.batch_size, num_heads, int(n), dev.index)
                        for n in (self.length, self.max_seq_len) if n), default=0)
        ws = getattr(self, "_decode_ws", None)
        if need and (ws is None or ws.numel() < need):
            ws = torch.empty((need,), dtype=torch.uint8, device=dev)
        self._decode_ws, self._decode_ws_key = ws, key
        return ws

    def _ensure_page_cnt_per_batch(self, expected_page_cnt_per_batch):
        if expected_page_cnt_per_batch * self.batch_size <= self._pages.shape[0]:
            return
        raise NotImplementedError

    @property
    def seen_tokens(self):
        return self.length

    def update(self, key_states, value_states, layer_idx, cache_kwargs=None):
        b_sz, added_length, num_heads, head_dim = key_states.shape
        assert b_sz == self.batch_size
        cache_kwargs = cache_kwargs or {}
        if self._pending:
            self._flush()
        if layer_idx == 0:
            new_length = self.length + added_length
            self._ensure_page_cnt_per_batch(self.page_cnt_from_length(new_length))
            self.length = new_length
        attention_mask = cache_kwargs.get("attention_mask")
        first = self._needs_init[layer_idx]
        specs = self.get_cache_specs_for_flash_infer(attention_mask)
        if self.disable_quant:
            return self._update_f16(key_states, value_states, layer_idx, attention_mask, first, specs)
        k_in, fused_had = key_states, self.hadamard_dtype is not None
        if self.hadamard_dtype is not None and self.hadamard_dtype != torch.float16:
            k_in, fused_had = matmul_had_cuda(key_states, dtype=self.hadamard_dtype), False   # e.g. the fp32 transform
        if first:
            self._needs_init[layer_idx] = False
            if attention_mask is not None:
                # padded prompt: quantise every row, keep the rows the mask selects (kv_cache.py:206-220)
                kq, ks, kz = asym_quantize_and_pack_i4(k_in, hadamard=fused_had)
                vq, vs, vz = asym_quantize_and_pack_i4(value_states)
                keep = torch.nonzero(attention_mask.flatten(), as_tuple=False).flatten()
                rows = self.batch_size * added_length
                pick = lambda t, w: t.reshape(rows, num_heads, w).index_select(0, keep).contiguous()
                seqlens = torch.nn.functional.pad(torch.cumsum(attention_mask.sum(dim=-1, dtype=torch.int32), dim=0,
                                                               dtype=torch.int32), (1, 0))
                init_kv_i4(**specs, k=pick(kq, head_dim // 2), v=pick(vq, head_dim // 2),
                           k_param=pick(torch.cat([ks, kz], dim=-1), 2), v_param=pick(torch.cat([vs, vz], dim=-1), 2),
                           seqlen_indptr=seqlens, layer_idx=layer_idx)
            else:
                seqlens = torch.arange(self.batch_size + 1, device=self.device, dtype=torch.int32) * added_length
                quantize_append_kv_i4(**specs, k=k_in.reshape(-1, num_heads, head_dim).contiguous(),
                                      v=value_states.reshape(-1, num_heads, head_dim).contiguous(), seqlen_indptr=seqlens,
                                      layer_idx=layer_idx, hadamard=fused_had)
            return key_states, value_states
        assert added_length == 1
        k3 = k_in.reshape(self.batch_size, num_heads, head_dim).contiguous()
        v3 = value_states.reshape(self.batch_size, num_heads, head_dim).contiguous()
        if k3.dtype == torch.float16 and v3.dtype == torch.float16 and head_dim == 128:
            # held for the attention call, which quantises and stores the token itself
            token = object()
            self._pending[layer_idx] = (token, k3, v3, specs, fused_had)
            take = functools.partial(self._take_pending, layer_idx, token)
        else:
            quantize_append_kv_i4(**specs, k=k3, v=v3, seqlen_indptr=None, layer_idx=layer_idx, hadamard=fused_had)
            take = None
        return functools.partial(self._stub.forward, num_kv_heads=num_heads, attention_kwargs=specs, layer_idx=layer_idx,
                                 max_seq_len=self.length, workspace=self._decode_workspace(num_heads), take_pending=take)

    def _update_f16(self, key_states, value_states, layer_idx, attention_mask, first, specs):
        """update() with fp16 pages (kv_cache.py:187-251 with disable_quant): the transformed keys and the values are
        stored as they are, with parameters {1, 0} beside them."""
        b_sz, added_length, num_heads, head_dim = key_states.shape
        k = key_states if self.hadamard_dtype is None else matmul_had_cuda(key_states, dtype=self.hadamard_dtype)
        rows = self.batch_size * added_length
        k = k.reshape(rows, num_heads, head_dim).contiguous()
        v = value_states.reshape(rows, num_heads, head_dim).contiguous()
        param = torch.zeros((rows, num_heads, 2), dtype=torch.float16, device=k.device)
        param[..., 0] = 1
        if first:
            self._needs_init[layer_idx] = False
            if attention_mask is not None:
                keep = torch.nonzero(attention_mask.flatten(), as_tuple=False).flatten()
                k, v, param = k.index_select(0, keep), v.index_select(0, keep), param.index_select(0, keep)
                seqlens = torch.nn.functional.pad(torch.cumsum(attention_mask.sum(dim=-1, dtype=torch.int32), dim=0,
                                                               dtype=torch.int32), (1, 0))
            else:
                seqlens = torch.arange(self.batch_size + 1, device=self.device, dtype=torch.int32) * added_length
            init_kv_f16(**specs, k=k, v=v, k_param=param, v_param=param, seqlen_indptr=seqlens, layer_idx=layer_idx)
            return key_states, value_states
        assert added_length == 1
        append_kv_f16(**specs, k=k, v=v, k_param=param, v_param=param, layer_idx=layer_idx)
        return functools.partial(self._stub.forward, num_kv_heads=num_heads, attention_kwargs=specs, layer_idx=layer_idx)

    def get_cache_specs_for_flash_infer(self, attention_mask):
        """Page tables of the current state (kv_cache.py:253-275): page i of sequence b is page number
        i * batch_size + b; every sequence must span the same number of pages."""
        if self._pending:
            self._flush()
        if attention_mask is None:
            # every sequence holds self.length tokens: the tables depend on that number alone and are built
            # once per length (every layer of a decode step asks for them), with host arithmetic
            cached = getattr(self, "_specs", None)
            if cached is not None and cached[0] == self.length:
                return cached[1]
            page_cnt = self.page_cnt_from_length(self.length)
            ptr = self.length % self.page_size
            ptr = self.page_size if (self.length != 0 and ptr == 0) else ptr
            arange = functools.partial(torch.arange, device=self.device, dtype=torch.int32)
            specs = {
                "kv_data": self._pages,
                "kv_indptr": arange(0, self.batch_size + 1) * page_cnt,
                "kv_indices": (arange(page_cnt).unsqueeze(0) * self.batch_size + arange(self.batch_size).unsqueeze(1)).reshape(-1),
                "last_page_offset": torch.full((self.batch_size,), ptr, dtype=torch.int32, device=self.device),
                "kv_param": self._scales,
            }
            self._specs = (self.length, specs)
            return specs
        seqlens_in_batch = attention_mask.sum(dim=-1, dtype=torch.int32)
        page_cnt = self.page_cnt_from_length(seqlens_in_batch)
        if (page_cnt[0] != page_cnt).any():
            raise NotImplementedError("Current implementation does not support the case where batches have different number of pages")
        page_cnt = page_cnt[0]
        page_ptr = seqlens_in_batch % self.page_size
        page_ptr = torch.where((seqlens_in_batch != 0) & (page_ptr == 0), self.page_size, page_ptr).to(torch.int32).contiguous()
        arange = functools.partial(torch.arange, device=self.device, dtype=torch.int32)
        return {
            "kv_data": self._pages,
            "kv_indptr": (arange(0, self.batch_size + 1) * page_cnt).to(torch.int32),
            "kv_indices": ((arange(int(page_cnt)) * self.batch_size).unsqueeze(0) + arange(self.batch_size).unsqueeze(1)).reshape(-1).contiguous(),
            "last_page_offset": page_ptr,
            "kv_param": self._scales,
        }

    def get_seq_length(self, layer_idx=0):
        return self.length

    def get_max_length(self):
        return None

    def get_usable_length(self, new_seq_length, layer_idx=0):
        """transformers' Cache.get_usable_length for a cache without a maximum length: everything seen so far
        (called by e2e/quantized_llama/modeling_llama.py:54)."""
        return self.get_seq_length(layer_idx)

    def to_legacy_cache(self):
        return self
