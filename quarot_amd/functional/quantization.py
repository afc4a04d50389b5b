"""Torch-level quantisation primitives and the packed-nibble storage format.

Same public names and results as quarot/functional/quantization.py:4-74 (these run on any device and
are what the reference itself uses on the host); the GPU hot path does not go through them.
Storage format: two signed 4-bit codes per byte, the even-indexed code in the low nibble.
"""
import torch

__all__ = ["two_compl", "get_minq_maxq", "asym_quant", "asym_dequant", "asym_quant_dequant", "sym_quant",
           "sym_dequant", "sym_quant_dequant", "pack_i4", "unpack_i4"]


def _grid(bits: int, sym: bool):
    """Smallest and largest code of a `bits`-bit grid as Python ints."""
    if sym:
        half = 1 << (bits - 1)
        return -half, half - 1
    return 0, (1 << bits) - 1


def _snap(x, scale, lo, hi, shift=0):
    """round(x / scale) + shift, limited to [lo, hi]."""
    return torch.clamp(torch.round(x / scale) + shift, lo, hi)


def two_compl(x, bits: int):
    """Image of signed codes in `bits`-bit two's complement: negative values wrap upwards
    (quantization.py:4-5)."""
    return torch.where(x < 0, x + (1 << bits), x)


def get_minq_maxq(bits: int, sym: bool):
    """(minq, maxq) of the grid as 0-dim tensors (quantization.py:7-15)."""
    lo, hi = _grid(bits, sym)
    return torch.tensor(lo), torch.tensor(hi)


def asym_quant(x, scale, zero, maxq):
    """Codes in [0, maxq] with an integer zero point; also returns scale and zero moved to x's device
    (quantization.py:17-21)."""
    scale, zero = scale.to(x.device), zero.to(x.device)
    return _snap(x, scale, 0, maxq, zero), scale, zero


def asym_dequant(q, scale, zero):
    return (q - zero) * scale


def asym_quant_dequant(x, scale, zero, maxq):
    q, s, z = asym_quant(x, scale, zero, maxq)
    return asym_dequant(q, s, z)


def sym_quant(x, scale, maxq):
    """Codes in [-(maxq + 1), maxq]; also returns the scale moved to x's device (quantization.py:29-32)."""
    scale = scale.to(x.device)
    return _snap(x, scale, -(maxq + 1), maxq), scale


def sym_dequant(q, scale):
    return q * scale


def sym_quant_dequant(x, scale, maxq):
    q, s = sym_quant(x, scale, maxq)
    return sym_dequant(q, s)


def pack_i4(q):
    """Signed codes [R, C] (C even) -> uint8 [R, C / 2], code 2j in the low nibble of byte j and code
    2j + 1 in the high one (quantization.py:42-49).  Values outside [-8, 7] are an error, as in the
    reference."""
    assert torch.is_signed(q), 'The tensor to be packed should be signed int'
    lo, hi = _grid(4, True)
    assert bool(((q >= lo) & (q <= hi)).all())
    nibbles = two_compl(q.to(torch.int8), 4).to(torch.uint8)
    even, odd = nibbles[:, 0::2], nibbles[:, 1::2]
    return even | (odd << 4)


def unpack_i4(x: torch.Tensor):
    """uint8 [..., C] -> int32 [..., 2 C], the inverse of pack_i4 (quantization.py:52-74)."""
    assert x.dtype == torch.uint8, 'The tensor to be unpacked should be stored in uint8'
    wide = x.to(torch.int32)
    pair = torch.stack((wide & 0xF, wide >> 4), dim=-1)            # [..., C, 2]: low nibble first
    pair = pair - ((pair & 8) << 1)                                 # sign-extend the 4-bit codes
    return pair.reshape(*x.shape[:-1], 2 * x.shape[-1])
