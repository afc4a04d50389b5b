"""quarot_amd: QuaRot's quantized-linear hot path on MI355X (gfx950).

Drop-in for the top level of the reference's ``quarot`` package (quarot/__init__.py:9-71):
``matmul``, ``sym_quant``, ``sym_dequant``, ``PackedQuantizedTensor`` keep their signatures,
assertions and output shapes; they call hand-written HIP kernels in ``libquarot_hip.so`` through
its C ABI.  Extras that fuse adjacent steps are listed after the reference's names.

    import quarot_amd as quarot
"""
import functools

import weakref

import torch

from . import _lib
from . import functional
from . import nn

__all__ = [
    "matmul", "sym_quant", "sym_dequant", "PackedQuantizedTensor",      # the reference's names
    "quantize_rows", "hadamard_quantize", "rmsnorm_quantize", "heads_hadamard_quantize", "linear_i4", "quantized_linear", "convert_i4_f6", "linear_f6",   # fused entry points
]


def _flat2d(x: torch.Tensor):
    """[..., C] -> ([R, C] view, leading shape).  Same contract as the reference's
    flatten_last_dim_and_return_shape (quarot/__init__.py:31-34): `view`, so it raises on
    layouts that cannot be flattened without a copy."""
    lead = x.shape[:-1]
    return x.view(-1, x.shape[-1]), lead


def _require_gpu_contiguous(fn, **tensors):
    """The checks of quarot/kernels/bindings.cpp:11-16,29-34,52-64 (contiguous, on the GPU, one
    device) raised as RuntimeError like torch::check* does."""
    dev = None
    for name, t in tensors.items():
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(f"{fn}: expected {name} to be a GPU tensor, got {t.device}")
        if not t.is_contiguous():
            raise RuntimeError(f"{fn}: expected {name} to be contiguous")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"{fn}: expected all tensors on {dev}, but {name} is on {t.device}")
    return dev


def _ptr(t):
    return None if t is None else t.data_ptr()


def matmul(A, B):
    """int4 x int4 -> int32: unpack(A) @ unpack(B).T  (quarot/__init__.py:37-41).
    A uint8 [..., K/2], B uint8 [..., K/2] -> int32 [*A.shape[:-1], *B.shape[:-1]]."""
    assert A.shape[-1] % 32 == 0, "A.shape[-1]: {} must be multiplication of 32".format(A.shape[-1])
    A2, a_lead = _flat2d(A)
    B2, b_lead = _flat2d(B)
    dev = _require_gpu_contiguous("matmul", A=A2, B=B2)
    if A2.dtype != torch.uint8 or B2.dtype != torch.uint8:
        raise RuntimeError("matmul: expected packed uint8 operands")
    if A2.shape[1] != B2.shape[1]:
        raise RuntimeError(f"matmul: inner sizes differ ({A2.shape[1]} vs {B2.shape[1]} packed bytes)")
    M, N, K = A2.shape[0], B2.shape[0], A2.shape[1] * 2
    C = torch.empty((M, N), dtype=torch.int32, device=dev)
    with _lib.on_device(dev):
        _lib.check(_lib.lib().qr_matmul_i4_i32(_ptr(A2), _ptr(B2), M, N, K, _ptr(C), _lib.stream_ptr(dev)))
    return C.view(*a_lead, *b_lead)


def sym_quant(x, scale):
    """Symmetric int4 quantise + pack with given per-row scales (quarot/__init__.py:43-46).
    x fp16 [..., C], scale fp16 (one per row, any shape) -> uint8 [..., ceil(C/2)]."""
    assert x.dtype == scale.dtype == torch.float16
    x2, lead = _flat2d(x)
    s = scale.view(-1)
    dev = _require_gpu_contiguous("sym_quant", x=x2, scale=s)
    if s.shape[0] != x2.shape[0]:
        raise RuntimeError(f"sym_quant: expected scale of size {x2.shape[0]}, got {s.shape[0]}")
    rows, cols = x2.shape
    q = torch.empty((rows, (cols + 1) // 2), dtype=torch.uint8, device=dev)
    with _lib.on_device(dev):
        _lib.check(_lib.lib().qr_sym_quant_f16_i4(_ptr(x2), _ptr(s), rows, cols, _ptr(q), _lib.stream_ptr(dev)))
    return q.view(*lead, q.shape[-1])


def sym_dequant(q, scale_row, scale_col, bits=32):
    """fp16((scale_row * scale_col) * half(q))  (quarot/__init__.py:48-52)."""
    assert q.dtype == torch.int32
    assert scale_row.dtype == scale_col.dtype == torch.float16
    q2, lead = _flat2d(q)
    sr = scale_row.view(-1)
    dev = _require_gpu_contiguous("sym_dequant", q=q2, scale_row=sr, scale_col=scale_col)
    rows, cols = q2.shape
    if sr.shape[0] != rows:
        raise RuntimeError(f"sym_dequant: expected scale_row of size {rows}, got {sr.shape[0]}")
    if scale_col.shape[0] != cols:
        raise RuntimeError(f"sym_dequant: expected scale_col of size {cols}, got {scale_col.shape[0]}")
    if bits != 32:
        raise RuntimeError("Unsupported data type")       # quarot/kernels/bindings.cpp:76-84
    y = torch.empty((rows, cols), dtype=torch.float16, device=dev)
    with _lib.on_device(dev):
        _lib.check(_lib.lib().qr_sym_dequant_i32_f16(_ptr(q2), _ptr(sr), _ptr(scale_col), rows, cols, _ptr(y),
                                                     _lib.stream_ptr(dev)))
    return y.view(*lead, y.shape[-1])


class PackedQuantizedTensor:
    """Carrier of packed int4 codes and their per-row scales (quarot/__init__.py:55-71)."""

    def __init__(self, quantized_x: torch.Tensor, scales_x: torch.Tensor):
        self.quantized_x = quantized_x
        self.scales_x = scales_x

    def size(self):
        return self.quantized_x.size()

    @property
    def device(self):
        return self.quantized_x.device

    @property
    def dtype(self):
        return self.quantized_x.dtype


# ------------------------------------------------------------------------------------------------
# fused entry points (no counterpart of their own in the reference; each equals a chain of its calls)

def quantize_rows(x, clip_ratio=1.0):
    """Quantizer.forward in one kernel (quarot/nn/quantization.py:9-13): returns
    (packed uint8 [..., C/2], scales fp16 with the reference's [R, 1]-after-unsqueeze(1) shape)."""
    assert x.dtype == torch.float16
    x2, lead = _flat2d(x)
    dev = _require_gpu_contiguous("quantize_rows", x=x2)
    rows, cols = x2.shape
    q = torch.empty((rows, (cols + 1) // 2), dtype=torch.uint8, device=dev)
    s = torch.empty((rows,), dtype=torch.float16, device=dev)
    with _lib.on_device(dev):
        _lib.check(_lib.lib().qr_quantize_rows_f16_i4(_ptr(x2), float(clip_ratio), rows, cols, _ptr(q), _ptr(s),
                                                      _lib.stream_ptr(dev)))
    # torch.max(dim=-1)[0].unsqueeze(1) on [..., C] gives shape lead[:1] + (1,) + lead[1:]
    s_shape = tuple(lead[:1]) + (1,) + tuple(lead[1:])
    return q.view(*lead, q.shape[-1]), s.view(s_shape)


_SIGNS = {}                 # id(table) -> (weak reference to the table, its version, sign words or None)
_SIGNS_REFUSED = set()      # (n, K) for which the library takes the table itself


def _hadamard_sign_words(hadK, n, K):
    """The table's sign words -- uint32 [K][ceil(K / 32)] as bytes, bit j of word w of row r set where
    hadK[r][32 w + j] = -1 -- for the widths whose fused kernel takes them (n / K = 64 behind a table of order
    97 .. 192: the down_proj width 11008 = 172 x 64), or None.  A prepared operand: packed once per table
    (4 KB for order 172, where the fp16 table is 59 KB that every workgroup of the kernel would fetch) and
    kept while the table object lives and is not written to; tables with entries other than +-1 are never
    packed."""
    if hadK is None or K <= 96 or K > 192 or n != 64 * K or (n, K) in _SIGNS_REFUSED:
        return None
    key = id(hadK)
    hit = _SIGNS.get(key)
    if hit is not None and hit[0]() is hadK and hit[1] == hadK._version:
        return hit[2]
    words = None
    if tuple(hadK.shape) == (K, K) and bool((hadK.abs() == 1).all()):
        import numpy as np
        neg = (hadK < 0).cpu().numpy()
        padded = np.zeros((K, (K + 31) // 32 * 32), dtype=bool)
        padded[:, :K] = neg
        words = torch.from_numpy(np.packbits(padded, axis=1, bitorder="little")).to(hadK.device)
    if len(_SIGNS) > 64:
        for k in [k for k, v in _SIGNS.items() if v[0]() is None]:
            del _SIGNS[k]
    _SIGNS[key] = (weakref.ref(hadK), hadK._version, words)
    return words


def hadamard_quantize(x, hadK, K, clip_ratio=1.0, force_fp32=False, return_transformed=False):
    """OnlineHadamard.forward followed by Quantizer.forward in one kernel
    (quarot/nn/hadamard.py:17-23 + quarot/nn/quantization.py:9-13)."""
    assert x.dtype == torch.float16
    x2, lead = _flat2d(x)
    dev = _require_gpu_contiguous("hadamard_quantize", x=x2, hadK=hadK)
    rows, n = x2.shape
    want = torch.float32 if force_fp32 else torch.float16
    table = hadK                                   # (the caller's object: what the sign words are remembered for)
    if hadK is not None and hadK.dtype != want:
        hadK = hadK.to(want)
    q = torch.empty((rows, n // 2), dtype=torch.uint8, device=dev)
    s = torch.empty((rows,), dtype=torch.float16, device=dev)
    y = torch.empty_like(x2) if return_transformed else None
    scale = functional.hadamard.had_scale(n)
    mode = _lib.QR_DTYPE_F32 if force_fp32 else _lib.QR_DTYPE_F16
    signs = None if return_transformed else _hadamard_sign_words(table, n, int(K))
    with _lib.on_device(dev):
        rc = _lib.QR_E_UNSUPPORTED
        if signs is not None:
            rc = _lib.lib().qr_hadamard_quantize_f16_i4(_ptr(x2), rows, n, int(K), _ptr(signs), mode | _lib.QR_HADK_SIGNS, scale,
                                                        float(clip_ratio), _ptr(q), _ptr(s), None, _lib.stream_ptr(dev))
            if rc == _lib.QR_E_UNSUPPORTED:
                _SIGNS_REFUSED.add((n, int(K)))
        if rc == _lib.QR_E_UNSUPPORTED:
            rc = _lib.lib().qr_hadamard_quantize_f16_i4(_ptr(x2), rows, n, int(K), _ptr(hadK), mode, scale,
                                                        float(clip_ratio), _ptr(q), _ptr(s), _ptr(y), _lib.stream_ptr(dev))
        if rc == _lib.QR_E_UNSUPPORTED and (n <= 128 or n > functional.hadamard.MAX_FUSED_ROW):
            # rows this short are not fused (rows of 128 only with a place for the transformed rows), rows beyond 32768
            # neither: the steps that Sequential(OnlineHadamard, Quantizer) runs, so the bits are those of the two modules
            y = functional.matmul_hadU_cuda(x2.float() if force_fp32 else x2, hadK, int(K)).to(torch.float16)
            q, s = quantize_rows(y, clip_ratio)
            rc = 0
        _lib.check(rc)
    s_shape = tuple(lead[:1]) + (1,) + tuple(lead[1:])
    packed = PackedQuantizedTensor(q.view(*lead, q.shape[-1]), s.view(s_shape))
    return (packed, y.view(x.shape)) if return_transformed else packed


def rmsnorm_quantize(x, mean_dim, eps=1e-5, clip_ratio=1.0, return_normalized=False):
    """RMSNorm.forward followed by Quantizer.forward in one kernel
    (quarot/nn/normalization.py:15-21 + quarot/nn/quantization.py:9-13)."""
    assert x.dtype == torch.float16
    x2, lead = _flat2d(x)
    dev = _require_gpu_contiguous("rmsnorm_quantize", x=x2)
    rows, cols = x2.shape
    q = torch.empty((rows, cols // 2), dtype=torch.uint8, device=dev)
    s = torch.empty((rows,), dtype=torch.float16, device=dev)
    y = torch.empty_like(x2) if return_normalized else None
    with _lib.on_device(dev):
        _lib.check(_lib.lib().qr_rmsnorm_quantize_f16_i4(_ptr(x2), rows, cols, int(mean_dim), float(eps),
                                                         float(clip_ratio), _ptr(q), _ptr(s), _ptr(y),
                                                         _lib.stream_ptr(dev)))
    s_shape = tuple(lead[:1]) + (1,) + tuple(lead[1:])
    packed = PackedQuantizedTensor(q.view(*lead, q.shape[-1]), s.view(s_shape))
    return (packed, y.view(x.shape)) if return_normalized else packed


def heads_hadamard_quantize(x, num_heads, clip_ratio=1.0, return_transformed=False, hadK=None):
    """The chain in front of o_proj in one kernel (e2e/quantized_llama/modeling_llama.py:108-110):
    OnlineHadamard(num_heads) over the head axis of attention's output, then Quantizer.forward on the
    rows reshaped to [..., hidden].  x is [..., num_heads, head_dim], contiguous, as attention writes
    it; no transposed copies are made.  head_dim 128 and 16, 32 or 64 heads; or a head count that is
    the order of one of the reference's tables (40 for Llama-2-13B, 52 for Llama-30B, ...) with hadK =
    that table (OnlineHadamard's had_rem_dim buffer)."""
    assert x.dtype == torch.float16
    if x.dim() < 2 or x.shape[-2] != num_heads:
        raise RuntimeError("heads_hadamard_quantize: x must be [..., num_heads, head_dim]")
    x2, lead = _flat2d(x.view(*x.shape[:-2], x.shape[-2] * x.shape[-1]))
    if hadK is not None:
        if hadK.shape != (num_heads, num_heads):
            raise RuntimeError("heads_hadamard_quantize: hadK must be [num_heads, num_heads]")
        if hadK.dtype != torch.float16 or hadK.device != x2.device:     # (a module left on the CPU: as matmul_hadU_cuda does)
            hadK = hadK.to(device=x2.device, dtype=torch.float16)
    dev = _require_gpu_contiguous("heads_hadamard_quantize", x=x2, hadK=hadK)
    rows, cols = x2.shape
    q = torch.empty((rows, cols // 2), dtype=torch.uint8, device=dev)
    s = torch.empty((rows,), dtype=torch.float16, device=dev)
    y = torch.empty_like(x2) if return_transformed else None
    with _lib.on_device(dev):
        _lib.check(_lib.lib().qr_heads_hadamard_quantize_f16_i4(_ptr(x2), rows, int(num_heads), cols // int(num_heads),
                                                                _ptr(hadK), float(clip_ratio), _ptr(q), _ptr(s), _ptr(y),
                                                                _lib.stream_ptr(dev)))
    s_shape = tuple(lead[:1]) + (1,) + tuple(lead[1:])
    packed = PackedQuantizedTensor(q.view(*lead, q.shape[-1]), s.view(s_shape))
    return (packed, y.view(*lead, cols)) if return_transformed else packed


@functools.lru_cache(maxsize=4096)
def _workspace_bytes(M, N, K, device_index=None):
    # (the library's split plan depends on the CURRENT device's compute-unit count: callers make the
    # device current first, and the device index is part of the cache key)
    return _lib.lib().qr_workspace_bytes(M, N, K)


def linear_i4(x_q, scales_x, weight, weight_scales, bias=None):
    """Linear4bit.forward in one kernel (quarot/nn/linear.py:42-56): matmul + sym_dequant (+ bias)."""
    assert x_q.shape[-1] % 32 == 0, "A.shape[-1]: {} must be multiplication of 32".format(x_q.shape[-1])
    assert scales_x.dtype == weight_scales.dtype == torch.float16
    a2, lead = _flat2d(x_q)
    sx = scales_x.view(-1)
    sw = weight_scales.view(-1)
    dev = _require_gpu_contiguous("linear_i4", x=a2, scales_x=sx, weight=weight, weight_scales=sw, bias=bias)
    M, N, K = a2.shape[0], weight.shape[0], a2.shape[1] * 2
    if weight.shape[1] != a2.shape[1] or sx.shape[0] != M or sw.shape[0] != N:
        raise RuntimeError("linear_i4: inconsistent operand sizes")
    if bias is not None and (bias.dtype != torch.float16 or bias.numel() != N):
        raise RuntimeError("linear_i4: bias must be fp16 of size out_features")
    y = torch.empty((M, N), dtype=torch.float16, device=dev)
    L = _lib.lib()
    with _lib.on_device(dev):
        ws_bytes = _workspace_bytes(M, N, K, dev.index)
        if ws_bytes:
            # few output tiles: the library splits K across workgroups and needs int32 scratch for the sums
            ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
            _lib.check(L.qr_linear_i4_f16_ws(_ptr(a2), _ptr(sx), _ptr(weight), _ptr(sw), _ptr(bias), M, N, K, _ptr(y),
                                             _ptr(ws), ws_bytes, _lib.stream_ptr(dev)))
        else:
            _lib.check(L.qr_linear_i4_f16(_ptr(a2), _ptr(sx), _ptr(weight), _ptr(sw), _ptr(bias), M, N, K, _ptr(y),
                                          _lib.stream_ptr(dev)))
    return y.view(*lead, N)


def convert_i4_f6(codes):
    """Packed int4 codes uint8 [..., K/2] (K % 64 == 0) -> the 6-bit operand layout of linear_f6: uint8
    [K/64, rows, 48], every code as its FP6 E3M2 value, stage-major.  For weights once after loading, for
    activations after the quantiser."""
    c2, lead = _flat2d(codes)
    dev = _require_gpu_contiguous("convert_i4_f6", codes=c2)
    rows, K = c2.shape[0], c2.shape[1] * 2
    assert K % 64 == 0, "in_features: {} must be a multiple of 64".format(K)
    out = torch.empty((K // 64, rows, 48), dtype=torch.uint8, device=dev)
    with _lib.on_device(dev):
        _lib.check(_lib.lib().qr_convert_i4_f6(_ptr(c2), rows, K, _ptr(out), _lib.stream_ptr(dev)))
    return out


def linear_f6(x6, scales_x, weight6, weight_scales, bias=None):
    """Linear4bit.forward (quarot/nn/linear.py:42-56) on operands converted by convert_i4_f6: the int4
    product on the FP6 matrix path (exact: every code is an FP6 value, sums stay integers below 2^24) with the
    same fused fp16 epilogue as linear_i4, bit for bit.  x6 [K/64, M, 48], weight6 [K/64, N, 48] -> fp16 [M, N]."""
    assert scales_x.dtype == weight_scales.dtype == torch.float16
    sx, sw = scales_x.view(-1), weight_scales.view(-1)
    dev = _require_gpu_contiguous("linear_f6", x6=x6, scales_x=sx, weight6=weight6, weight_scales=sw, bias=bias)
    if x6.dim() != 3 or weight6.dim() != 3 or x6.shape[0] != weight6.shape[0] or x6.shape[2] != 48 or weight6.shape[2] != 48:
        raise RuntimeError("linear_f6: operands must be [K/64, rows, 48] from convert_i4_f6 with the same K")
    M, N, K = x6.shape[1], weight6.shape[1], x6.shape[0] * 64
    if sx.shape[0] != M or sw.shape[0] != N:
        raise RuntimeError("linear_f6: inconsistent operand sizes")
    if bias is not None and (bias.dtype != torch.float16 or bias.numel() != N):
        raise RuntimeError("linear_f6: bias must be fp16 of size out_features")
    y = torch.empty((M, N), dtype=torch.float16, device=dev)
    with _lib.on_device(dev):
        _lib.check(_lib.lib().qr_linear_f6_f16(_ptr(x6), _ptr(sx), _ptr(weight6), _ptr(sw), _ptr(bias), M, N, K, _ptr(y),
                                               _lib.stream_ptr(dev)))
    return y


@functools.lru_cache(maxsize=4096)
def _quantized_linear_workspace_bytes(M, N, K, device_index=None):
    return _lib.lib().qr_quantized_linear_workspace_bytes(M, N, K)       # (per device, like _workspace_bytes)


def quantized_linear(x, weight, weight_scales, bias=None, hadK=None, K=0, clip_ratio=1.0, force_fp32=False):
    """Sequential(OnlineHadamard, Quantizer, Linear4bit) -- or, with K == 0, Sequential(Quantizer,
    Linear4bit) -- in ONE call into the library (e2e/quantized_llama/modeling_llama.py:99-102,111-115):
    the same two launches as hadamard_quantize / quantize_rows followed by linear_i4 (one or two tokens, plain or behind a
    1024-point Hadamard factor: one kernel that does both), same results bit for bit, half the host-side
    cost.  x fp16 [..., in_features] -> fp16 [..., out_features]."""
    assert x.dtype == torch.float16
    assert x.shape[-1] % 64 == 0, "in_features: {} must be a multiple of 64".format(x.shape[-1])
    x2, lead = _flat2d(x)
    sw = weight_scales.view(-1)
    dev = _require_gpu_contiguous("quantized_linear", x=x2, weight=weight, weight_scales=sw, bias=bias, hadK=hadK)
    M, n = x2.shape
    N = weight.shape[0]
    if weight.shape[1] * 2 != n or sw.shape[0] != N or sw.dtype != torch.float16 or weight.dtype != torch.uint8:
        raise RuntimeError("quantized_linear: inconsistent operand sizes or dtypes")
    if bias is not None and (bias.dtype != torch.float16 or bias.numel() != N):
        raise RuntimeError("quantized_linear: bias must be fp16 of size out_features")
    want = torch.float32 if force_fp32 else torch.float16
    table = hadK
    if hadK is not None and hadK.dtype != want:
        hadK = hadK.to(want)
    y = torch.empty((M, N), dtype=torch.float16, device=dev)
    mode = _lib.QR_DTYPE_F32 if force_fp32 else _lib.QR_DTYPE_F16
    signs = _hadamard_sign_words(table, n, int(K)) if K else None
    with _lib.on_device(dev):
        ws_bytes = _quantized_linear_workspace_bytes(M, N, n, dev.index)
        ws = torch.empty((max(ws_bytes, 16),), dtype=torch.uint8, device=dev)
        call = lambda table, md: _lib.lib().qr_quantized_linear_f16(
            _ptr(x2), M, n, int(K), _ptr(table), md, functional.hadamard.had_scale(n), float(clip_ratio), _ptr(weight),
            _ptr(sw), _ptr(bias), N, _ptr(y), _ptr(ws), ws_bytes, _lib.stream_ptr(dev))
        rc = _lib.QR_E_UNSUPPORTED
        if signs is not None:
            rc = call(signs, mode | _lib.QR_HADK_SIGNS)                  # (refused before anything is launched)
            if rc == _lib.QR_E_UNSUPPORTED:
                _SIGNS_REFUSED.add((n, int(K)))
        if rc == _lib.QR_E_UNSUPPORTED:
            rc = call(hadK, mode)
        if rc == _lib.QR_E_UNSUPPORTED and K and n > functional.hadamard.MAX_FUSED_ROW:
            # rows beyond the fused front's reach: the front's own fall-back, then the linear layer
            p = hadamard_quantize(x2, table, K, clip_ratio, force_fp32)
            return linear_i4(p.quantized_x, p.scales_x, weight, weight_scales, bias).view(*lead, N)
        _lib.check(rc)
    return y.view(*lead, N)
