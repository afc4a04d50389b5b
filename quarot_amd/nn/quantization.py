import torch

import quarot_amd


class Quantizer(torch.nn.Module):
    """Per-token symmetric int4 activation quantiser: one scale per row of the last axis,
    `(max|x| / 7).half() * input_clip_ratio`, codes packed two per byte.  Interface and results of
    quarot/nn/quantization.py:4-13; the row maximum, the scale and the codes come from one HIP kernel
    (qr_quantize_rows_f16_i4) instead of four torch kernels and sym_quant."""

    def __init__(self, input_clip_ratio=1.0):
        super().__init__()
        self.input_clip_ratio = input_clip_ratio

    def extra_repr(self):
        return f"input_clip_ratio={self.input_clip_ratio}"

    def forward(self, x):
        codes, scales = quarot_amd.quantize_rows(x, self.input_clip_ratio)
        return quarot_amd.PackedQuantizedTensor(codes, scales)
