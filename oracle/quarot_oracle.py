"""CPU oracle for QuaRot's quantized-linear hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, in numpy, what the reference computes on the path
OnlineHadamard -> Quantizer -> Linear4bit (and the KV-cache asymmetric int4 round trip).
It exists so that the HIP kernels can be checked; nothing in the shipped package imports it.
Only tests, the smoke check and the benchmark's CPU-baseline leg may call it.

Every function cites the reference lines it follows (paths relative to the reference root).
All half-precision arithmetic is done the way IEEE-754 binary16 hardware does it: one
correctly rounded operation at a time.  numpy evaluates float16 +,-,*,/ in float32 and rounds
the result, which is the correctly rounded answer for a single operation (24 >= 2*11 + 2).

How each function is pinned (see tests/test_oracle.py):
  get_hadK             known answers for every Llama width named by the reference's comments
  tables               SHA-256 of the bit-packed matrices + H.H^T = K.I
  matmul_hadU          float64 closed form X @ kron(hadK, scipy.linalg.hadamard(m)).T / sqrt(n),
                       unit vectors, orthonormality, inverse by the transposed factor
  hadamard_staged      same closed form (it only adds the intermediate roundings)
  quantizer_scales     exact rational rounding (fractions) over every finite fp16 amax
  sym_quant_codes      exact rational arithmetic on random pairs and on constructed ties
  pack_i4 / unpack_i4  all 256 byte values, nibble order
  int4_matmul          int64 brute force, closed-form all-7 x all-(-8) = -56.K, one-hot rows
  sym_dequant          exact rational rounding of each of the three operations
  kv_asym_*            range/extreme-code invariants and exact rational spot checks
  heads_hadamard       float64 einsum with scipy.linalg.hadamard over the head axis, a row constant
                       across heads (only head 0 survives, times sqrt(H)), one-hot heads (sign columns)
  rmsnorm              float64 closed form x / sqrt(sum(x^2) / mean_dim + eps) rounded once,
                       constant rows, mean_dim different from the row length, sign symmetry
  paged_append/gather  an element-by-element walk over a flat buffer with the reference's offset formulas
                       (page.cuh:75-103), append -> gather round trips, untouched bytes stay untouched
  paged_dequant        exact rational arithmetic of float(nibble) * scale - zero rounded once to float32
  paged_batch_decode   torch's scaled_dot_product_attention in float64 on the gathered, dequantised cache;
                       a one-token sequence returns v_0, equal V vectors return that vector, q = 0 the mean
"""
from __future__ import annotations

import pathlib

import numpy as np

F16 = np.float16
F32 = np.float32

_ORDERS = (12, 20, 28, 36, 40, 52, 60, 108, 140, 156, 172)
# Order in which the reference tests divisibility (quarot/functional/hadamard.py:7-50):
# 40 is tried before 20, 28 before 40.
_PROBE_ORDER = (172, 156, 140, 108, 60, 52, 36, 28, 40, 20, 12)
_TABLE_FILE = pathlib.Path(__file__).resolve().parent.parent / "quarot_amd" / "functional" / "hadamard_tables.bin"
_tables = None


def hadamard_tables():
    """{K: int8 [K, K] of +-1}: the reference's tables (quarot/functional/hadamard.py:153-4193),
    read from the bit-packed data file (row-major, +1 -> bit 1)."""
    global _tables
    if _tables is None:
        raw = np.frombuffer(_TABLE_FILE.read_bytes(), dtype=np.uint8)
        out, pos = {}, 0
        for k in _ORDERS:
            nbytes = (k * k + 7) // 8
            bits = np.unpackbits(raw[pos:pos + nbytes])[:k * k]
            out[k] = (bits.astype(np.int8) * 2 - 1).reshape(k, k)
            pos += nbytes
        assert pos == raw.size
        _tables = out
    return _tables


def is_pow2(n):
    """quarot/functional/hadamard.py:146-147."""
    return n > 0 and (n & (n - 1)) == 0


def get_hadK(n, transpose=False):
    """quarot/functional/hadamard.py:5-55: first K in the probe order dividing n (cofactor must be
    a power of two, else AssertionError); K = 1 when n itself is a power of two."""
    for k in _PROBE_ORDER:
        if n % k == 0:
            assert is_pow2(n // k)
            h = hadamard_tables()[k].astype(np.float64)
            return (h.T.copy() if transpose else h), k
    assert is_pow2(n)
    return None, 1


def sylvester(m):
    """Natural-order (Sylvester) Hadamard matrix of power-of-two order m, entries +-1 (int64).
    H[i, j] = (-1)^popcount(i & j)."""
    assert is_pow2(m)
    i = np.arange(m)
    x = i[:, None] & i[None, :]
    pc = np.zeros_like(x)
    while x.any():
        pc += x & 1
        x >>= 1
    return 1 - 2 * (pc & 1)


def fwht_butterfly(x, stop_len=1):
    """The butterfly loop of matmul_hadU (quarot/functional/hadamard.py:61-70): view as
    [rows, L, 1]; while L > stop_len: pair ADJACENT entries of the L axis, (a, b) -> (a+b, a-b),
    sums to the first half-axis position, moving the pair index into the trailing axis.
    Arithmetic is done in x's dtype (each stage rounds, as in the reference).
    Returns an array of shape [rows, stop_len, n // stop_len]."""
    n = x.shape[-1]
    cur = np.array(x, copy=True).reshape(-1, n, 1)
    while cur.shape[1] > stop_len:
        r, L, t = cur.shape
        v = cur.reshape(r, L // 2, 2, t)
        nxt = np.empty_like(v)
        nxt[:, :, 0, :] = v[:, :, 0, :] + v[:, :, 1, :]
        nxt[:, :, 1, :] = v[:, :, 0, :] - v[:, :, 1, :]
        cur = nxt.reshape(r, L // 2, 2 * t)
    return cur


def matmul_hadU(x, transpose=False):
    """quarot/functional/hadamard.py:58-79 (= fake_quant/hadamard_utils.py:58-79): butterflies
    down to length K, then hadK @ (.) over the remaining axis, then / sqrt(n); in x's dtype."""
    x = np.asarray(x)
    n = x.shape[-1]
    hadk, k = get_hadK(n, transpose)
    cur = fwht_butterfly(x, stop_len=k)
    if k > 1:
        cur = np.matmul(hadk.astype(x.dtype)[None], cur)
    root = np.sqrt(F32(n))  # torch.tensor(n).sqrt() is a float32 0-dim tensor
    cur = cur.reshape(x.shape)
    if x.dtype == F16:      # fp16 tensor / float32 scalar: evaluated in float32, rounded to fp16
        return (cur.astype(F32) / root).astype(F16)
    return cur / root.astype(x.dtype)


def hadamard_closed_form(x, transpose=False):
    """float64 closed form of the same transform: X @ kron(hadK, H_m)^T / sqrt(n)."""
    x = np.asarray(x, dtype=np.float64)
    n = x.shape[-1]
    hadk, k = get_hadK(n, transpose)
    hm = sylvester(n // k).astype(np.float64)
    full = hm if k == 1 else np.kron(hadk, hm)
    return x @ full.T / np.sqrt(np.float64(n))


def had_scale(n):
    """The scale the reference hands to the FWHT kernel: 1.0 / torch.tensor(n).sqrt(), a float32
    (quarot/functional/hadamard.py:95,99)."""
    return F32(1.0) / np.sqrt(F32(n))


def fwht_natural(x64):
    """Unnormalised natural-order Walsh-Hadamard transform along the last axis, float64."""
    y = np.array(x64, dtype=np.float64, copy=True)
    m = y.shape[-1]
    h = 1
    while h < m:
        v = y.reshape(*y.shape[:-1], m // (2 * h), 2, h)
        a = v[..., 0, :] + v[..., 1, :]
        b = v[..., 0, :] - v[..., 1, :]
        y = np.stack([a, b], axis=-2).reshape(y.shape)
        h *= 2
    return y


def hadamard_staged(x, hadk, k, io_dtype):
    """matmul_hadU_cuda (quarot/functional/hadamard.py:92-101) with its intermediate roundings:
    view [..., K, n/K]; FWHT along the last axis with the float32 scale applied inside, result
    rounded to io_dtype; then hadK.to(io_dtype) @ (.) accumulated wide and rounded to io_dtype.
    Wide accumulation is float64 here (float32 in the reference's libraries)."""
    x = np.asarray(x)
    n = x.shape[-1]
    scale = np.float64(had_scale(n))
    if k == 1:
        return (fwht_natural(x.astype(np.float64)) * scale).astype(io_dtype)
    m = n // k
    t = (fwht_natural(x.astype(np.float64).reshape(*x.shape[:-1], k, m)) * scale).astype(io_dtype)
    h = np.asarray(hadk).astype(io_dtype).astype(np.float64)
    y = np.matmul(h, t.astype(np.float64)).astype(io_dtype)
    return y.reshape(x.shape)


def online_hadamard(x, force_fp32=False):
    """OnlineHadamard.forward (quarot/nn/hadamard.py:17-23): transform in fp16, or in fp32 when
    force_fp32, then cast back to x's dtype."""
    x = np.asarray(x)
    hadk, k = get_hadK(x.shape[-1])
    io = F32 if force_fp32 else x.dtype
    return hadamard_staged(x.astype(io), hadk, k, io).astype(x.dtype)


def heads_hadamard(x, num_heads):
    """The transform in front of o_proj (e2e/quantized_llama/modeling_llama.py:108-109):
    OnlineHadamard(num_heads) applied to attn_output.transpose(-1, -2), transposed back and reshaped
    to [..., hidden].  x fp16 [..., num_heads, head_dim] -> fp16 [..., num_heads * head_dim]."""
    x = np.asarray(x)
    assert x.shape[-2] == num_heads
    y = np.swapaxes(online_hadamard(np.swapaxes(x, -1, -2)), -1, -2)
    return np.ascontiguousarray(y).reshape(*x.shape[:-2], x.shape[-2] * x.shape[-1])


# ----------------------------------------------------------------------------------------------
# symmetric per-token int4 quantisation

def quantizer_scales(x, clip=1.0):
    """Quantizer.forward's scale (quarot/nn/quantization.py:10):
    (max|x| over the last axis / 7).to(fp16) * clip.  The division is one fp16 operation; the
    multiplication by the Python scalar is evaluated in float32 and rounded to fp16."""
    x = np.asarray(x, dtype=F16)
    amax = np.max(np.abs(x), axis=-1)
    s = (amax.astype(F32) / F32(7)).astype(F16)
    return (s.astype(F32) * F32(clip)).astype(F16)


def sym_quant_codes(x, scale):
    """sym_quantize_f16_i4_kernel (quarot/kernels/quant.cu:36-38): q = clamp(rn_even(x / s), -8, 7)
    with x / s one correctly rounded fp16 division; NaN (0/0) gives 0.  x [rows, cols] fp16,
    scale [rows] fp16 -> int8 [rows, cols]."""
    x = np.asarray(x, dtype=F16)
    s = np.asarray(scale, dtype=F16).reshape(-1, 1)
    with np.errstate(divide="ignore", invalid="ignore"):
        d = (x.astype(F32) / s.astype(F32)).astype(F16)
    r = np.rint(d.astype(F32))
    r = np.where(np.isnan(r), F32(0), r)
    return np.clip(r, -8, 7).astype(np.int8)


def pack_i4(q):
    """pack_i4 (quarot/functional/quantization.py:42-49) and Int4Subbyte::set
    (quarot/kernels/include/int4.h:86-98): two's-complement nibbles, even column -> low nibble.
    An odd trailing column leaves the last high nibble 0 (quarot/kernels/quant.cu:28-42)."""
    q = np.asarray(q)
    assert q.min(initial=0) >= -8 and q.max(initial=0) <= 7
    u = (q.astype(np.int16) & 0xF).astype(np.uint8)
    if u.shape[-1] % 2:
        u = np.concatenate([u, np.zeros((*u.shape[:-1], 1), np.uint8)], axis=-1)
    return (u[..., 0::2] | (u[..., 1::2] << 4)).astype(np.uint8)


def unpack_i4(p):
    """unpack_i4 (quarot/functional/quantization.py:52-74): uint8 [..., C] -> int32 [..., 2C]."""
    p = np.asarray(p, dtype=np.uint8)
    lo = (p & 0xF).astype(np.int32)
    hi = (p >> 4).astype(np.int32)
    lo -= 16 * (lo >= 8)
    hi -= 16 * (hi >= 8)
    return np.stack([lo, hi], axis=-1).reshape(*p.shape[:-1], 2 * p.shape[-1])


def quantizer(x, clip=1.0):
    """Quantizer.forward (quarot/nn/quantization.py:9-13) on a 2-D fp16 array:
    returns (packed uint8 [rows, ceil(cols/2)], scales fp16 [rows])."""
    s = quantizer_scales(x, clip)
    return pack_i4(sym_quant_codes(x, s)), s


# ----------------------------------------------------------------------------------------------
# int4 x int4 GEMM and the dequant epilogue

def rmsnorm(x, mean_dim, eps=1e-5):
    """quarot/nn/normalization.py:15-21: fp16 input is promoted to fp32, the sum of squares is
    divided by mean_dim (not necessarily the row length), x * rsqrt(var + eps) is computed in fp32
    and cast back.  The association order of the fp32 sum is the only freedom (torch's differs
    from numpy's, the kernel's from both): results agree to within one rounding of the fp32 sum,
    far below half an fp16 ulp except on exact ties."""
    xf = np.asarray(x).astype(F32)
    var = (xf * xf).sum(-1, keepdims=True, dtype=F32) / F32(mean_dim)
    r = F32(1.0) / np.sqrt(var + F32(eps), dtype=F32)
    return (xf * r).astype(np.asarray(x).dtype)


def int4_matmul(a_packed, b_packed, exact_int=False):
    """matmul_host (quarot/kernels/gemm.cu:7-46): C[M, N] int32 = unpack(A) . unpack(B)^T.
    Default path multiplies in float32 BLAS, which is exact here: every partial sum is an integer
    of magnitude <= 64.K < 2^24 (asserted).  exact_int=True uses int64 (slow; small cases)."""
    a = unpack_i4(a_packed)
    b = unpack_i4(b_packed)
    if exact_int:
        return (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.int32)
    assert 64 * a.shape[-1] < (1 << 24)
    return np.rint(a.astype(F32) @ b.astype(F32).T).astype(np.int32)


def sym_dequant(q, scale_row, scale_col, bias=None):
    """sym_dequantize_i32_f16_kernel (quarot/kernels/quant.cu:79-80): three rounded fp16
    operations, left to right: (scale_row[r] * scale_col[c]) * half(q); then the optional bias as
    a fourth rounded fp16 add (quarot/nn/linear.py:53-54).  int32 -> fp16 is round-to-nearest-even
    (values beyond 65519 become inf)."""
    q = np.asarray(q, dtype=np.int32)
    sr = np.asarray(scale_row, dtype=F16).reshape(-1, 1)
    sc = np.asarray(scale_col, dtype=F16).reshape(1, -1)
    with np.errstate(over="ignore", invalid="ignore"):
        qh = q.astype(np.float64).astype(F16)          # |q| < 2^53: a single rounding
        ss = (sr.astype(F32) * sc.astype(F32)).astype(F16)
        y = (ss.astype(F32) * qh.astype(F32)).astype(F16)
        if bias is not None:
            b = np.asarray(bias, dtype=F16).reshape(1, -1)
            y = (y.astype(F32) + b.astype(F32)).astype(F16)
    return y


def linear4bit(a_packed, scales_x, w_packed, w_scales, bias=None):
    """Linear4bit.forward (quarot/nn/linear.py:42-56)."""
    return sym_dequant(int4_matmul(a_packed, w_packed), scales_x, w_scales, bias)


def weight_codes_from_float(w, w_scales):
    """Linear4bit.from_float (quarot/nn/linear.py:74-75): (W / s).round() in W's fp16 dtype, then
    pack_i4 (which asserts the range)."""
    w = np.asarray(w, dtype=F16)
    s = np.asarray(w_scales, dtype=F16).reshape(-1, 1)
    d = (w.astype(F32) / s.astype(F32)).astype(F16)
    return pack_i4(np.rint(d.astype(F32)).astype(np.int8))


# ----------------------------------------------------------------------------------------------
# KV-cache asymmetric int4

def kv_hadamard(x, fp32=False):
    """matmul_had_cuda (quarot/transformers/kv_cache.py:30-33): FWHT over the last axis, scale
    1/sqrt(n) (a Python float here, math.sqrt), computed in fp16 i/o (fp32 internally) or in fp32,
    returned in x's dtype."""
    x = np.asarray(x)
    n = x.shape[-1]
    y = fwht_natural(x.astype(np.float64)) * np.float64(F32(1.0 / np.sqrt(np.float64(n))))
    if fp32:
        y = y.astype(F32)
    return y.astype(x.dtype)


def kv_asym_quant(x):
    """asym_quantize_and_pack_i4 (quarot/transformers/kv_cache.py:10-22), fp16 throughout:
    scale = (max - min).clamp(min=1e-5) / 15; zero = -min; q = clamp(round((x + zero) / scale), 0, 15);
    low nibble = even element.  Returns (packed uint8 [..., D/2], scale fp16 [..., 1], zero fp16 [..., 1])."""
    x = np.asarray(x, dtype=F16)
    xmax = np.max(x, axis=-1, keepdims=True)
    xmin = np.min(x, axis=-1, keepdims=True)
    rng = (xmax.astype(F32) - xmin.astype(F32)).astype(F16)
    rng = np.maximum(rng, F16(1e-5))
    scale = (rng.astype(F32) / F32(15)).astype(F16)
    zero = (-xmin).astype(F16)
    shifted = (x.astype(F32) + zero.astype(F32)).astype(F16)
    d = (shifted.astype(F32) / scale.astype(F32)).astype(F16)
    q = np.clip(np.rint(d.astype(F32)), 0, 15).astype(np.uint8)
    return (q[..., 0::2] | (q[..., 1::2] << 4)).astype(np.uint8), scale, zero


def kv_asym_dequant(packed, scale, zero):
    """unpack_i4_and_asym_dequantize (quarot/transformers/kv_cache.py:24-28): nib * scale - zero in
    fp16 (two rounded operations)."""
    p = np.asarray(packed, dtype=np.uint8)
    nib = np.stack([p & 0xF, p >> 4], axis=-1).reshape(*p.shape[:-1], 2 * p.shape[-1])
    prod = (nib.astype(F32) * np.asarray(scale, F16).astype(F32)).astype(F16)
    return (prod.astype(F32) - np.asarray(zero, F16).astype(F32)).astype(F16)


# ----------------------------------------------------------------------------------------------
# paged int4 KV cache: append and single-query attention

def paged_seq_lens(kv_indptr, last_page_offset, page_size):
    """Tokens held by every sequence: (pages - 1) * page_size + last_page_offset
    (quarot/kernels/include/flashinfer/page.cuh:131-133, decode.cuh:516)."""
    indptr = np.asarray(kv_indptr, dtype=np.int64)
    pages = indptr[1:] - indptr[:-1]
    return (pages - 1) * int(page_size) + np.asarray(last_page_offset, dtype=np.int64)


def paged_append(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, k, v, k_param, v_param, layer_idx,
                 append_indptr=None):
    """AppendPagedKVCachePrefillKernel / AppendPagedKVCacheDecodeKernel (page.cuh:120-219) on numpy arrays,
    in place.  kv_data uint8 [pages, L, 2, H, P, D/2], kv_param fp16 [pages, L, 2, H, P, 2];
    k, v uint8 [tokens, H, D/2], k_param, v_param fp16 [tokens, H, 2].  append_indptr None: one token per
    sequence at position seq_len - 1 (page.cuh:136-140); else the tokens append_indptr[b] ..
    append_indptr[b + 1] - 1 of sequence b fill its last positions (page.cuh:183-193)."""
    page_size = kv_data.shape[4]
    seq = paged_seq_lens(kv_indptr, last_page_offset, page_size)
    batch = len(seq)
    for b in range(batch):
        if append_indptr is None:
            first, count = b, 1
        else:
            first, count = int(append_indptr[b]), int(append_indptr[b + 1] - append_indptr[b])
        start = int(seq[b]) - count
        for j in range(count):
            pos = start + j
            page = int(kv_indices[int(kv_indptr[b]) + pos // page_size])
            entry = pos % page_size
            kv_data[page, layer_idx, 0, :, entry, :] = k[first + j]
            kv_data[page, layer_idx, 1, :, entry, :] = v[first + j]
            kv_param[page, layer_idx, 0, :, entry, :] = k_param[first + j]
            kv_param[page, layer_idx, 1, :, entry, :] = v_param[first + j]


def paged_gather(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, layer_idx, b):
    """The cached vectors of sequence b in position order: (k codes [seq, H, D/2], k param [seq, H, 2],
    v codes, v param), walking its page list as decode.cuh:560-600 does."""
    page_size = kv_data.shape[4]
    n = int(paged_seq_lens(kv_indptr, last_page_offset, page_size)[b])
    out = [[], [], [], []]
    for pos in range(n):
        page = int(kv_indices[int(kv_indptr[b]) + pos // page_size])
        entry = pos % page_size
        out[0].append(kv_data[page, layer_idx, 0, :, entry, :])
        out[1].append(kv_param[page, layer_idx, 0, :, entry, :])
        out[2].append(kv_data[page, layer_idx, 1, :, entry, :])
        out[3].append(kv_param[page, layer_idx, 1, :, entry, :])
    heads, half = kv_data.shape[3], kv_data.shape[5]
    shapes = [(0, heads, half), (0, heads, 2), (0, heads, half), (0, heads, 2)]
    return tuple(np.stack(o) if o else np.zeros(s, kv_data.dtype if i % 2 == 0 else kv_param.dtype)
                 for i, (o, s) in enumerate(zip(out, shapes)))


def paged_dequant(codes, param):
    """dequantize_impl (quarot/kernels/include/flashinfer/quantization.cuh:59-84): float(nibble) * scale - zero
    in float32, low nibble = even element; scale, zero = the half2 parameter widened to float
    (decode.cuh:631-636).  codes uint8 [..., D/2], param fp16 [..., 2] -> float32 [..., D]."""
    p = np.asarray(codes, dtype=np.uint8)
    nib = np.stack([p & 0xF, p >> 4], axis=-1).reshape(*p.shape[:-1], 2 * p.shape[-1]).astype(F32)
    prm = np.asarray(param, dtype=F16).astype(F32)
    return (nib * prm[..., 0:1]).astype(F32) - prm[..., 1:2]


def paged_batch_decode(q, kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, layer_idx):
    """BatchDecodeWithPagedKVCacheKernel (decode.cuh:492-689) without rotary embedding, as
    quarot/kernels/flashinfer.cu:10-46 instantiates it: per sequence and head,
    softmax(q . K^T / sqrt(D)) . V over the dequantised cache.  float64 here (the kernel works in
    float32 with an online softmax); q fp16 [B, H, D] -> float64 [B, H, D]."""
    q = np.asarray(q, dtype=F16).astype(np.float64)
    batch, heads, dim = q.shape
    out = np.zeros((batch, heads, dim), np.float64)
    for b in range(batch):
        kc, kp, vc, vp = paged_gather(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, layer_idx, b)
        kf = paged_dequant(kc, kp).astype(np.float64)          # [seq, H, D]
        vf = paged_dequant(vc, vp).astype(np.float64)
        logits = np.einsum("hd,shd->hs", q[b], kf) / np.sqrt(np.float64(dim))
        logits -= logits.max(axis=1, keepdims=True)
        w = np.exp(logits)
        w /= w.sum(axis=1, keepdims=True)
        out[b] = np.einsum("hs,shd->hd", w, vf)
    return out


def paged_batch_decode_f16(q, kv_data, kv_indptr, kv_indices, last_page_offset, layer_idx):
    """The same kernel over fp16 pages (quarot/kernels/bindings.cpp:247-285, the reference's disable_quant cache,
    quarot/transformers/kv_cache.py:134-151): kv_data fp16 [pages, L, 2, H, P, D] holds the vectors themselves, the
    parameters are not read.  float64 here; q fp16 [B, H, D] -> float64 [B, H, D]."""
    q = np.asarray(q, dtype=F16).astype(np.float64)
    batch, heads, dim = q.shape
    page_size = kv_data.shape[4]
    seq = paged_seq_lens(kv_indptr, last_page_offset, page_size)
    out = np.zeros((batch, heads, dim), np.float64)
    for b in range(batch):
        pos = np.arange(int(seq[b]))
        pages = np.asarray(kv_indices)[int(kv_indptr[b]) + pos // page_size]
        kf = kv_data[pages, layer_idx, 0, :, pos % page_size, :].astype(np.float64)      # [seq, H, D]
        vf = kv_data[pages, layer_idx, 1, :, pos % page_size, :].astype(np.float64)
        logits = np.einsum("hd,shd->hs", q[b], kf) / np.sqrt(np.float64(dim))
        logits -= logits.max(axis=1, keepdims=True)
        w = np.exp(logits)
        w /= w.sum(axis=1, keepdims=True)
        out[b] = np.einsum("hs,shd->hd", w, vf)
    return out
