"""The reference's CPU-capable statement of the path, in torch, for TIMING on host cores.
TEST/BENCHMARK INFRASTRUCTURE ONLY (never imported by the shipped package).

It chains the reference's CPU-capable pieces: its PyTorch Hadamard (matmul_hadU,
fake_quant/hadamard_utils.py:58-79), per-token symmetric quantisation
(fake_quant/quant_utils.py:30-33 with the scale of quarot/nn/quantization.py:10), a torch integer
matmul on unpacked int32 codes (what quarot/kernels/gemm.cu:7-46 computes), and the fp16 dequant of
quarot/kernels/quant.cu:79-80.  Its results are checked against quarot_oracle in tests/test_oracle.py.
"""
import numpy as np
import torch

from . import quarot_oracle as o


def matmul_hadU(X):
    """fake_quant/hadamard_utils.py:58-79 in torch (fp32 input here: fp16 input would round at every
    butterfly stage)."""
    n = X.shape[-1]
    hadk, K = o.get_hadK(n)
    cur = X.reshape(-1, n, 1).clone()
    while cur.shape[1] > K:
        r, L, t = cur.shape
        v = cur.view(r, L // 2, 2, t)
        cur = torch.cat((v[:, :, 0, :] + v[:, :, 1, :], v[:, :, 0, :] - v[:, :, 1, :]), dim=-1)
    if K > 1:
        cur = torch.from_numpy(hadk).to(cur).view(1, K, K) @ cur
    return cur.reshape(X.shape) / torch.tensor(n).sqrt()


def quantize(x16):
    """scale = (amax / 7).half(); q = clamp(round(x / scale), -8, 7) on fp16 tensors."""
    scale = (x16.abs().amax(dim=-1, keepdim=True) / 7).to(torch.float16)
    q = torch.clamp(torch.round(x16 / scale), -8, 7)
    return q.to(torch.int32), scale


def rmsnorm(x16, eps=1e-5):
    """quarot/nn/normalization.py:15-21 in torch on the host."""
    xf = x16.to(torch.float32)
    var = xf.pow(2).sum(-1, keepdim=True) / x16.shape[-1]
    return (xf * torch.rsqrt(var + eps)).to(torch.float16)


def linear4bit_path(x16, w_codes_i32, w_scales16, hadamard=True, norm=False, heads=0):
    """x fp16 [M, K] -> fp16 [M, N]: (RMSNorm ->) Hadamard (fp32) -> quantise -> int32 matmul -> dequant.
    heads > 0: the Hadamard runs over the head axis of rows seen as [heads, K / heads], on the
    transposed view as in e2e/quantized_llama/modeling_llama.py:108-109."""
    if norm:
        x16 = rmsnorm(x16)
    if heads:
        v = x16.float().view(x16.shape[0], heads, -1).transpose(-1, -2).contiguous()
        x16 = matmul_hadU(v).transpose(-1, -2).reshape(x16.shape).contiguous().to(torch.float16)
    xh = matmul_hadU(x16.float()).to(torch.float16) if hadamard else x16
    q, sx = quantize(xh)
    acc = q @ w_codes_i32.t()
    return (sx * w_scales16.view(1, -1)) * acc.to(torch.float16)


def unpacked_codes(w_packed_np):
    return torch.from_numpy(o.unpack_i4(w_packed_np))
