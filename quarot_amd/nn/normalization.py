import torch

import quarot_amd


class RMSNorm(torch.nn.Module):
    """Weight-less RMS normalisation in fp32 (quarot/nn/normalization.py:3-21); the learned gain
    has been folded into the following linear layer offline."""

    def __init__(self, mean_dim: int, eps=1e-5):
        super().__init__()
        self.eps = eps
        self.mean_dim = mean_dim

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        dt = x.dtype
        xf = x.to(torch.float32) if dt == torch.float16 else x
        var = xf.pow(2).sum(-1, keepdim=True) / self.mean_dim
        return (xf * torch.rsqrt(var + self.eps)).to(dt)


class RMSNormQuantizer(torch.nn.Module):
    """RMSNorm(mean_dim, eps) followed by Quantizer(input_clip_ratio) in one kernel: the chain in
    front of q/k/v_proj and gate/up_proj (e2e/quantized_llama/modeling_llama.py:40-44,108-110).  The
    normalised fp16 tensor does not go through HBM.  Widths the fused kernel does not take (not a
    multiple of 8, beyond 32768) run as the two separate steps."""

    def __init__(self, mean_dim: int, eps=1e-5, input_clip_ratio=1.0):
        super().__init__()
        self.eps = eps
        self.mean_dim = mean_dim
        self.input_clip_ratio = input_clip_ratio

    def forward(self, x: torch.Tensor):
        if x.dtype != torch.float16 or x.shape[-1] % 8 != 0 or x.shape[-1] > 32768:
            y = RMSNorm(self.mean_dim, self.eps)(x)
            return quarot_amd.PackedQuantizedTensor(*quarot_amd.quantize_rows(y, self.input_clip_ratio))
        return quarot_amd.rmsnorm_quantize(x, self.mean_dim, self.eps, self.input_clip_ratio)
