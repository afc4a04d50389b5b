"""Pure-torch quantisation primitives and the packed-nibble format
(mirror of quarot/functional/quantization.py:4-74; device-agnostic torch ops as in the reference)."""
import torch


def two_compl(x, bits: int):
    """Two's-complement image of a signed value in `bits` bits (quantization.py:4)."""
    return torch.where(x < 0, x + (1 << bits), x)


def get_minq_maxq(bits: int, sym: bool):
    """(minq, maxq) as 0-dim tensors (quantization.py:7-15)."""
    if sym:
        hi = (1 << (bits - 1)) - 1
        return torch.tensor(-hi - 1), torch.tensor(hi)
    return torch.tensor(0), torch.tensor((1 << bits) - 1)


def asym_quant(x, scale, zero, maxq):
    scale, zero = scale.to(x.device), zero.to(x.device)
    return torch.clamp(torch.round(x / scale) + zero, 0, maxq), scale, zero


def asym_dequant(q, scale, zero):
    return scale * (q - zero)


def asym_quant_dequant(x, scale, zero, maxq):
    return asym_dequant(*asym_quant(x, scale, zero, maxq))


def sym_quant(x, scale, maxq):
    scale = scale.to(x.device)
    return torch.clamp(torch.round(x / scale), -(maxq + 1), maxq), scale


def sym_dequant(q, scale):
    return scale * q


def sym_quant_dequant(x, scale, maxq):
    return sym_dequant(*sym_quant(x, scale, maxq))


def pack_i4(q):
    """Signed int4 values [R, C] -> uint8 [R, C/2]; even column in the low nibble
    (quantization.py:42-49).  Asserts the [-8, 7] range like the reference."""
    assert torch.is_signed(q), 'The tensor to be packed should be signed int'
    minq, maxq = get_minq_maxq(4, True)
    assert torch.all(torch.logical_and(q >= minq, q <= maxq))
    nib = two_compl(q.to(torch.int8), 4).to(torch.uint8)
    return nib[:, 0::2] | (nib[:, 1::2] << 4)


def unpack_i4(x: torch.Tensor):
    """uint8 [..., C] -> int32 [..., 2C] (quantization.py:52-74)."""
    assert x.dtype == torch.uint8, 'The tensor to be unpacked should be stored in uint8'
    lo = (x & 0x0F).to(torch.int32)
    hi = (x >> 4).to(torch.int32)
    lo = lo - ((lo & 8) << 1)
    hi = hi - ((hi & 8) << 1)
    return torch.stack((lo, hi), dim=-1).reshape(*x.shape[:-1], x.shape[-1] * 2)
