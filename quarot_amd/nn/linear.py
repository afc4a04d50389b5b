import torch

import quarot_amd
from .hadamard import OnlineHadamard


def _pack_weight(weight, weight_scales):
    """Codes round(W / scales), packed: the GPU quantiser with the given per-row scales
    (qr_sym_quant_f16_i4 rounds and packs exactly like the reference's (W / s).round() followed by
    pack_i4) after checking, as pack_i4 would, that no code leaves [-8, 7]."""
    w = weight.cuda()
    s = weight_scales.to(device=w.device, dtype=w.dtype)
    if w.dtype == torch.float16 and w.is_contiguous():
        ratio_max = float((w.float().abs() / s.float().abs().clamp_min(1e-30)).max()) if w.numel() else 0.0
        if ratio_max < 7.4:                                  # every |W / s| rounds inside the grid: nothing to clamp
            return quarot_amd.sym_quant(w, s.reshape(-1).contiguous())
    codes = (w / s).round()
    return quarot_amd.functional.pack_i4(codes.to(torch.int8))


class Linear4bit(torch.nn.Module):
    """W4A4 linear layer with the interface and state-dict layout of quarot/nn/linear.py:24-79:
    buffers `weight` (uint8 [out, in / 2], packed int4), `weight_scales` ([out, 1]) and optionally
    `bias` ([out]).  forward() takes the PackedQuantizedTensor a Quantizer produces and runs the
    int4 GEMM with the dequantisation (and bias) fused into its epilogue."""

    def __init__(self, in_features, out_features, bias=False, dtype=torch.float16):
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        packed_shape = (out_features, in_features // 2)
        self.register_buffer('weight_scales', torch.zeros((out_features, 1), requires_grad=False))
        self.register_buffer('weight', torch.randint(1, 7, packed_shape, dtype=torch.uint8, requires_grad=False))
        if bias:
            self.register_buffer('bias', torch.zeros((out_features), dtype=dtype))
        else:
            self.bias = None

    def extra_repr(self):
        return f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}"

    # Opt-in: prompts of fp6_min_rows rows and more through the FP6 matrix path (quarot_amd.linear_f6:
    # bit-identical results, the GEMM 20-30 % faster wherever its tiles fill the machine, at the price of
    # a 6-bit copy of the weights -- 1.5 x their packed size, made at the first such call -- and of one
    # conversion pass over the activations' codes).
    prefill_fp6 = False
    fp6_min_rows = 1024          # (measured: ahead of the int8 path from 1024 rows on at every Llama-2 width, conversion included)

    def _weight_f6(self):
        key = (self.weight.data_ptr(), self.weight._version)
        cached = getattr(self, "_f6_cache", None)
        if cached is None or cached[0] != key:
            cached = (key, quarot_amd.convert_i4_f6(self.weight))
            self._f6_cache = cached
        return cached[1]

    def forward(self, x):
        assert type(x) == quarot_amd.PackedQuantizedTensor  # Quantized input is given
        q = x.quantized_x
        rows = q.numel() // max(q.shape[-1], 1)
        if (self.prefill_fp6 and q.is_cuda and rows >= self.fp6_min_rows and self.in_features % 64 == 0
                and max(rows, self.out_features) * self.in_features * 3 // 4 < 4290000000):     # (32-bit offsets inside the kernel)
            y = quarot_amd.linear_f6(quarot_amd.convert_i4_f6(q), x.scales_x, self._weight_f6(), self.weight_scales,
                                     self.bias)
            return y.view(*q.shape[:-1], self.out_features)     # the converter flattens the leading dimensions
        return quarot_amd.linear_i4(q, x.scales_x, self.weight, self.weight_scales, self.bias)

    @staticmethod
    def from_float(module: torch.nn.Linear, weight_scales=None):
        """A Linear4bit with module's shape; with `weight_scales` ([out, 1]) the weights, which must
        already lie on the int4 grid times those scales, are converted to codes and packed
        (linear.py:58-79).  Without scales only the shapes are taken over, as in the reference."""
        w = module.weight.data
        q4 = Linear4bit(module.in_features, module.out_features, bias=module.bias is not None, dtype=w.dtype).to(w.dtype)
        if weight_scales is None:
            return q4
        assert weight_scales.shape == (module.out_features, 1), 'weight_scales should have shape (out_features, 1)'
        q4.weight_scales.copy_(weight_scales.to(w.dtype))
        q4.weight.copy_(_pack_weight(w, weight_scales).cpu())
        if module.bias is not None:
            q4.bias.copy_(module.bias)
        return q4


class Linear4bitSequential(torch.nn.Sequential):
    """torch.nn.Sequential for the module chains the reference builds around Linear4bit
    (e2e/quantized_llama/modeling_llama.py:99-102,111-115):
        Linear4bitSequential(OnlineHadamard(n), Quantizer(), Linear4bit.from_float(...))
        Linear4bitSequential(Quantizer(), Linear4bit.from_float(...))
    Same constructor, same state-dict keys ("0.had_rem_dim", "2.weight", ...) and same results; when
    the chain has one of these two shapes and the input is a contiguous fp16 GPU tensor the forward
    pass is ONE call into the library instead of one per module.  Anything else runs module by
    module like the base class."""

    def _plan(self):
        from .quantization import Quantizer
        mods = list(self)
        had = None
        if len(mods) == 3 and isinstance(mods[0], OnlineHadamard):
            had, mods = mods[0], mods[1:]
        if len(mods) == 2 and isinstance(mods[0], Quantizer) and isinstance(mods[1], Linear4bit):
            return had, mods[0], mods[1]
        return None

    def forward(self, x):
        plan = self._plan()
        if (plan is None or not isinstance(x, torch.Tensor) or x.dtype != torch.float16 or not x.is_cuda
                or not x.is_contiguous() or x.shape[-1] % 64 != 0):
            return super().forward(x)
        had, quantizer, lin = plan
        if lin.prefill_fp6 and x.numel() // x.shape[-1] >= lin.fp6_min_rows and lin.in_features % 64 == 0:
            # long prompt on the opt-in FP6 matrix path: the fused front, then Linear4bit's own route
            if had is None:
                return lin(quantizer(x))
            return lin(quarot_amd.hadamard_quantize(x, had.had_rem_dim, had.rem_dim, quantizer.input_clip_ratio,
                                                    force_fp32=had.fp32_had))
        if had is None:
            return quarot_amd.quantized_linear(x, lin.weight, lin.weight_scales, lin.bias,
                                               clip_ratio=quantizer.input_clip_ratio)
        return quarot_amd.quantized_linear(x, lin.weight, lin.weight_scales, lin.bias, had.had_rem_dim, had.rem_dim,
                                           quantizer.input_clip_ratio, force_fp32=had.fp32_had)


def enable_fp6_prefill(module, min_rows=1024, convert_now=True):
    """Opt every Linear4bit under `module` into the FP6 matrix path for inputs of at least `min_rows`
    rows (prompts): the same results bit for bit, whole steps 10-16 % faster at 2048 rows of the 13B / 70B
    widths and 16 % at 32768 rows of the 7B ones (level at 2048 rows of the 7B widths), for a
    6-bit copy of each weight (1.5 x its packed size, kept beside the 4-bit one that decode streams)
    and a conversion pass over the activations' codes.  convert_now: make the copies here rather
    than at the first long input.  Returns the number of layers switched."""
    count = 0
    for m in module.modules():
        if isinstance(m, Linear4bit) and m.in_features % 64 == 0:
            m.prefill_fp6, m.fp6_min_rows = True, int(min_rows)
            if convert_now and m.weight.is_cuda:
                m._weight_f6()
            count += 1
    return count
