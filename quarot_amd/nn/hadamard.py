import torch

import quarot_amd


class OnlineHadamard(torch.nn.Module):
    """Online Hadamard over the last axis (quarot/nn/hadamard.py:5-23): buffer `had_rem_dim` holds
    the non-power-of-two factor (fp16 unless force_fp32), None for power-of-two widths."""

    def __init__(self, hadamard_dim, force_fp32=False):
        super().__init__()
        self.fp32_had = force_fp32
        had_rem_dim, self.rem_dim = quarot_amd.functional.hadamard.get_hadK(hadamard_dim)
        if had_rem_dim is not None:
            self.register_buffer("had_rem_dim", had_rem_dim)
            if not self.fp32_had:
                self.had_rem_dim = self.had_rem_dim.to(torch.float16)
        else:
            self.had_rem_dim = None

    def forward(self, x):
        x_dtype = x.dtype
        if self.fp32_had:
            x = x.float()
        x = quarot_amd.functional.matmul_hadU_cuda(x, self.had_rem_dim, self.rem_dim)
        return x.to(x_dtype)


class OnlineHadamardQuantizer(torch.nn.Module):
    """Sequential(OnlineHadamard(dim, force_fp32), Quantizer(clip)) in one kernel: same codes and
    scales, without the transformed fp16 tensor going through HBM.  Same buffer name, so a
    state-dict written for the two-module form loads."""

    def __init__(self, hadamard_dim, force_fp32=False, input_clip_ratio=1.0):
        super().__init__()
        self.fp32_had = force_fp32
        self.input_clip_ratio = input_clip_ratio
        had_rem_dim, self.rem_dim = quarot_amd.functional.hadamard.get_hadK(hadamard_dim)
        if had_rem_dim is not None:
            self.register_buffer("had_rem_dim", had_rem_dim if force_fp32 else had_rem_dim.to(torch.float16))
        else:
            self.had_rem_dim = None

    def forward(self, x):
        return quarot_amd.hadamard_quantize(x, self.had_rem_dim, self.rem_dim, self.input_clip_ratio,
                                            force_fp32=self.fp32_had)


class HeadsHadamardQuantizer(torch.nn.Module):
    """The three steps in front of o_proj (e2e/quantized_llama/modeling_llama.py:108-110) in one
    kernel: OnlineHadamard(num_heads) over the head axis of attention's output [..., heads, head_dim]
    (the reference applies it to a transposed view and transposes back), the reshape to
    [..., hidden], and o_proj's Quantizer(input_clip_ratio).  Neither the transposed copies nor the
    transformed fp16 tensor go through HBM.  Shapes the fused kernels do not take (head_dim other
    than 128, a head count that is neither 16, 32, 64 nor the order of one of the reference's tables
    up to 60, a dtype other than fp16, a strided input) run as the separate steps."""

    def __init__(self, num_heads, input_clip_ratio=1.0):
        super().__init__()
        self.num_heads = num_heads
        self.input_clip_ratio = input_clip_ratio
        self.had = OnlineHadamard(num_heads)

    def forward(self, x):
        assert x.shape[-2] == self.num_heads
        if x.dtype == torch.float16 and x.shape[-1] == 128 and x.is_contiguous() and x.is_cuda:
            if self.num_heads in (16, 32, 64):
                return quarot_amd.heads_hadamard_quantize(x, self.num_heads, self.input_clip_ratio)
            if self.had.rem_dim == self.num_heads and self.num_heads <= 64:      # hadK alone (40, 52, ... heads)
                return quarot_amd.heads_hadamard_quantize(x, self.num_heads, self.input_clip_ratio,
                                                          hadK=self.had.had_rem_dim)
        y = self.had(x.transpose(-1, -2)).transpose(-1, -2)
        y = y.reshape(*x.shape[:-2], x.shape[-2] * x.shape[-1]).contiguous()
        return quarot_amd.PackedQuantizedTensor(*quarot_amd.quantize_rows(y, self.input_clip_ratio))
