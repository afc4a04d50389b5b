import torch


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
