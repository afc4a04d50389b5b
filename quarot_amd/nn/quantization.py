import torch

import quarot_amd


class Quantizer(torch.nn.Module):
    """Per-token symmetric int4 activation quantiser (quarot/nn/quantization.py:4-13):
    scales = (max|x| / 7).half() * clip, codes packed two per byte."""

    def __init__(self, input_clip_ratio=1.0):
        super().__init__()
        self.input_clip_ratio = input_clip_ratio

    def forward(self, x):
        quantized_x, scales_x = quarot_amd.quantize_rows(x, self.input_clip_ratio)
        return quarot_amd.PackedQuantizedTensor(quantized_x, scales_x)
