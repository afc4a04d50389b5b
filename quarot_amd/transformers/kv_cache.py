"""KV-cache quantisation helpers (mirror of quarot/transformers/kv_cache.py:10-33) on HIP kernels.
The paged cache and decode attention of that file are outside this package."""
import math

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
