"""The reference's package name: code written against `quarot` (benchmarks/qlinear_benchmark.py:2,
e2e/quantized_llama/modeling_llama.py) must import and build its modules without an edit."""
import numpy as np
import pytest
import torch


def test_reference_import_lines_resolve():
    import quarot
    from quarot.nn import Linear4bit, Quantizer, OnlineHadamard          # qlinear_benchmark.py:2
    from quarot.nn import RMSNorm                                         # quarot/nn/__init__.py:2
    import quarot.functional.hadamard as had
    from quarot.functional import pack_i4, unpack_i4, asym_quant_dequant, sym_quant_dequant
    from quarot.functional import matmul_hadU_cuda, random_hadamard_matrix, apply_exact_had_to_linear
    from quarot.functional.quantization import sym_quant as torch_sym_quant
    from quarot.transformers.kv_cache import asym_quantize_and_pack_i4, unpack_i4_and_asym_dequantize, matmul_had_cuda
    import quarot_amd
    for name in ("matmul", "sym_quant", "sym_dequant", "PackedQuantizedTensor"):   # quarot/__init__.py:9-12
        assert getattr(quarot, name) is getattr(quarot_amd, name)
    assert Linear4bit is quarot_amd.nn.Linear4bit and Quantizer is quarot_amd.nn.Quantizer
    assert OnlineHadamard is quarot_amd.nn.OnlineHadamard and RMSNorm is quarot_amd.nn.RMSNorm
    assert had.get_hadK(11008)[1] == 172 and had.is_pow2(64) and callable(had.matmul_hadU)
    # the hot path's entry points under quarot.functional; the torch primitive keeps its own home
    assert quarot.functional.matmul is quarot.matmul
    assert quarot.functional.sym_quant is quarot.sym_quant and quarot.functional.sym_dequant is quarot.sym_dequant
    assert quarot.functional.hadamard_transform is had.hadamard_transform
    assert torch_sym_quant is not quarot.sym_quant
    with pytest.raises(AttributeError):
        quarot.functional.no_such_name


def test_modules_build_as_the_reference_benchmark_builds_them_without_scales():
    """qlinear_benchmark.py:60-84 minus the GPU calls: the three Sequential chains, their buffers
    and state-dict keys (Linear4bit.from_float without scales only takes the shapes over)."""
    from quarot.nn import Linear4bit, Quantizer, OnlineHadamard
    for fin, fout in ((4096, 4096), (5120, 5120), (4096, 11008)):
        base = torch.nn.Linear(fin, fout, bias=False).to(torch.float16)
        int4_mod = torch.nn.Sequential(Quantizer(input_clip_ratio=1.0), Linear4bit.from_float(base))
        int4_had = torch.nn.Sequential(OnlineHadamard(base.in_features, force_fp32=True), Quantizer(input_clip_ratio=1.0),
                                       Linear4bit.from_float(base))
        int4_had16 = torch.nn.Sequential(OnlineHadamard(base.in_features, force_fp32=False), Quantizer(input_clip_ratio=1.0),
                                         Linear4bit.from_float(base))
        assert int4_mod[1].weight.shape == (fout, fin // 2) and int4_mod[1].weight.dtype == torch.uint8
        assert int4_mod[1].weight_scales.shape == (fout, 1) and int4_mod[1].weight_scales.dtype == torch.float16
        assert list(int4_mod.state_dict()) == ["1.weight_scales", "1.weight"]
        if fin == 5120:                                                     # had_40 (x) H_128
            assert int4_had[0].had_rem_dim.dtype == torch.float32 and int4_had16[0].had_rem_dim.dtype == torch.float16
            assert int4_had[0].rem_dim == 40 and list(int4_had.state_dict())[0] == "0.had_rem_dim"
        else:
            assert int4_had[0].had_rem_dim is None and int4_had[0].rem_dim == 1


@pytest.mark.gpu
def test_reference_benchmark_chains_run_under_the_quarot_name():
    """The chains of qlinear_benchmark.py:56-84 at reduced token count, built with the reference's own
    statements (uniform inputs, integer weights, unit scales), against the oracle: packed weights, the
    plain chain bit for bit, and the two Hadamard chains through their own transformed rows."""
    from quarot.nn import Linear4bit, Quantizer, OnlineHadamard
    from oracle import quarot_oracle as o
    torch.manual_seed(0)
    for fin, fout in ((4096, 4096), (5120, 5120), (4096, 11008)):
        x = torch.rand((1, 48, fin)).cuda().to(torch.float16)
        base = torch.nn.Linear(fin, fout, bias=False).cuda().to(torch.float16)
        base.weight.data = torch.randint_like(base.weight.data, low=-8, high=7).to(torch.float16)
        s_w = torch.ones((fout, 1), dtype=torch.float16, device="cuda")
        int4_mod = torch.nn.Sequential(Quantizer(input_clip_ratio=1.0), Linear4bit.from_float(base, weight_scales=s_w)).cuda()
        wq = int4_mod[1].weight.cpu().numpy()
        assert np.array_equal(wq, o.pack_i4(base.weight.data.cpu().numpy().astype(np.int8)))
        xq, xs = o.quantizer(x.view(48, fin).cpu().numpy())
        y = int4_mod(x)
        assert y.shape == (1, 48, fout) and y.dtype == torch.float16
        want = o.linear4bit(xq, xs, wq, np.ones(fout, np.float16))
        assert np.array_equal(y.view(48, fout).cpu().numpy().view(np.uint16), want.view(np.uint16))
        for fp32 in (True, False):
            chain = torch.nn.Sequential(OnlineHadamard(base.in_features, force_fp32=fp32), Quantizer(input_clip_ratio=1.0),
                                        Linear4bit.from_float(base, weight_scales=s_w)).cuda()
            xh = chain[0](x)
            ref_h = o.online_hadamard(x.view(48, fin).cpu().numpy(), force_fp32=fp32)
            got_h = xh.view(48, fin).cpu().numpy()
            assert np.all(np.abs(got_h.astype(np.float64) - ref_h) <= 1e-3 + 1e-3 * np.abs(ref_h.astype(np.float64)))
            hq, hs = o.quantizer(got_h)
            want = o.linear4bit(hq, hs, wq, np.ones(fout, np.float16))
            assert np.array_equal(chain(x).view(48, fout).cpu().numpy().view(np.uint16), want.view(np.uint16))
