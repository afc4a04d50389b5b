"""Hadamard utilities (mirror of quarot/functional/hadamard.py:5-147).

`matmul_hadU_cuda` runs the HIP kernel; `matmul_hadU` is the reference's device-agnostic torch
butterfly (used offline, e.g. by random_hadamard_matrix); the tables are the reference's eleven
+-1 matrices, shipped bit-packed in hadamard_tables.bin.
"""
import functools
import math
import pathlib

import numpy as np
import torch

from .. import _lib

_ORDERS = (12, 20, 28, 36, 40, 52, 60, 108, 140, 156, 172)
# divisibility is probed in this order (hadamard.py:7-50): 28 before 40 before 20
_PROBE = (172, 156, 140, 108, 60, 52, 36, 28, 40, 20, 12)
_TABLE_FILE = pathlib.Path(__file__).resolve().parent / "hadamard_tables.bin"


@functools.lru_cache(maxsize=None)
def _tables():
    raw = np.frombuffer(_TABLE_FILE.read_bytes(), dtype=np.uint8)
    out, pos = {}, 0
    for k in _ORDERS:
        nbytes = (k * k + 7) // 8
        bits = np.unpackbits(raw[pos:pos + nbytes])[:k * k].astype(np.float32)
        out[k] = (bits * 2 - 1).reshape(k, k)
        pos += nbytes
    return out


def _had(k):
    return torch.from_numpy(_tables()[k].copy())


def get_had12(): return _had(12)
def get_had20(): return _had(20)
def get_had28(): return _had(28)
def get_had36(): return _had(36)
def get_had40(): return _had(40)
def get_had52(): return _had(52)
def get_had60(): return _had(60)
def get_had108(): return _had(108)
def get_had140(): return _had(140)
def get_had156(): return _had(156)
def get_had172(): return _had(172)


def is_pow2(n):
    return (n & (n - 1) == 0) and (n > 0)


def get_hadK(n, transpose=False):
    """(hadK FloatTensor [K, K] or None, K): the largest-first table order of the reference; the
    cofactor n / K must be a power of two (AssertionError otherwise)."""
    for k in _PROBE:
        if n % k == 0:
            assert is_pow2(n // k)
            h = _had(k)
            return (h.T if transpose else h), k
    assert is_pow2(n)
    return None, 1


def matmul_hadU(X, transpose=False):
    """Device-agnostic torch statement of the transform (hadamard.py:58-79): radix-2 butterflies on
    adjacent pairs until K entries remain per block, then hadK @ (.), then / sqrt(n); in X's dtype."""
    n = X.shape[-1]
    hadK, K = get_hadK(n, transpose)
    cur = X.reshape(-1, n, 1).clone()
    while cur.shape[1] > K:
        r, L, t = cur.shape
        pairs = cur.view(r, L // 2, 2, t)
        cur = torch.cat((pairs[:, :, 0, :] + pairs[:, :, 1, :], pairs[:, :, 0, :] - pairs[:, :, 1, :]), dim=-1)
    if K > 1:
        cur = hadK.view(1, K, K).to(cur) @ cur
    return cur.reshape(X.shape) / torch.tensor(n).sqrt()


def matmul_hadUt(X):
    return matmul_hadU(X, transpose=True)


def random_hadamard_matrix(size, device):
    """Random-sign diagonal times Hadamard, float64 (hadamard.py:85-90)."""
    signs = torch.randint(low=0, high=2, size=(size,)).to(torch.float64) * 2 - 1
    return matmul_hadU(torch.diag(signs)).to(device)


MAX_FUSED_ROW = 32768      # longest row of the library's Hadamard kernels (qr_hadamard: n <= 32768)


def hadamard_transform(x, scale=1.0):
    """Power-of-two Walsh-Hadamard transform along the last axis times `scale`: the call the
    reference makes into fast_hadamard_transform (hadamard.py:95,99; kv_cache.py:32).
    fp16 or fp32 GPU tensor, last dim a power of two in [8, 32768]."""
    return _run(x, None, 1, float(scale))


def _run(x, hadK, K, scale):
    if x.dtype not in (torch.float16, torch.float32):
        raise RuntimeError(f"hadamard: unsupported dtype {x.dtype}")
    if not x.is_cuda:
        raise RuntimeError(f"hadamard: expected a GPU tensor, got {x.device}")
    xc = x.contiguous()
    n = xc.shape[-1]
    rows = xc.numel() // n if n else 0
    if hadK is not None:
        hadK = hadK.to(device=xc.device, dtype=xc.dtype).contiguous()
    y = torch.empty_like(xc)
    code = _lib.QR_DTYPE_F16 if xc.dtype == torch.float16 else _lib.QR_DTYPE_F32
    with _lib.on_device(xc.device):
        _lib.check(_lib.lib().qr_hadamard(xc.data_ptr(), y.data_ptr(), rows, n, int(K),
                                          None if hadK is None else hadK.data_ptr(), code, scale,
                                          _lib.stream_ptr(xc.device)))
    return y


@functools.lru_cache(maxsize=None)
def had_scale(n):
    """The reference's scale, 1.0 / torch.tensor(n).sqrt() (a float32; hadamard.py:95,99), as a Python float."""
    return float(1.0 / torch.tensor(n).sqrt())


def matmul_hadU_cuda(X, hadK, K):
    """X . (hadK (x) H_{n/K})^T / sqrt(n) on the GPU (hadamard.py:92-101); output in X's dtype and shape."""
    n = X.shape[-1]
    scale = had_scale(n)
    if K > 1 and n > MAX_FUSED_ROW:
        # rows longer than the two-factor kernels hold (e.g. 53248 = 52 x 1024): the reference's own two steps
        # (hadamard.py:97-101) -- the power-of-two factor by the FWHT kernel on the [.., K, n / K] view, rounded to X's
        # dtype, then the table by a library GEMM
        t = _run(X.reshape(-1, K, n // K), None, 1, scale)
        return (hadK.to(t.device).to(t.dtype) @ t).reshape(X.shape)
    return _run(X, hadK if K > 1 else None, K, scale).reshape(X.shape)


def matmul_hadUt_cuda(X, hadK, K):
    return matmul_hadU_cuda(X, hadK.T if hadK is not None else None, K)


def apply_exact_had_to_linear(module, had_dim=-1, output=False):
    """Offline weight-side Hadamard (hadamard.py:109-142): W <- W.H (input side) or H.W (output
    side), computed in fp32 on the GPU and stored back in W's dtype and device."""
    assert isinstance(module, torch.nn.Linear)
    in_features, out_features = module.in_features, module.out_features
    if had_dim != -1:
        assert is_pow2(had_dim), "Hadamard dimension must be a power of 2!"
    W = module.weight.data
    dtype, dev = W.dtype, W.device
    W_ = W.float().cuda()
    if had_dim == -1:
        if output:
            had_K, K = get_hadK(out_features)
            W_ = matmul_hadU_cuda(W_.t(), had_K, K).t()
        else:
            had_K, K = get_hadK(in_features)
            W_ = matmul_hadU_cuda(W_, had_K, K)
    else:
        if not output:
            raise NotImplementedError("Not implemented (or tested) yet!")
        Wt = W_.t()
        shape_t = Wt.shape
        Wt = hadamard_transform(Wt.reshape(-1, shape_t[-1] // had_dim, had_dim), scale=1 / math.sqrt(had_dim))
        W_ = Wt.reshape(shape_t).t()
    module.weight.data = W_.to(device=dev, dtype=dtype)
