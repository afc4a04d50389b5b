"""Parity of the HIP path against the CPU oracle, through the C ABI (ctypes) and the Python mirror
of the reference interface.  Bars: int4 codes, scales, int32 accumulators and fp16 dequantised
values BIT-EXACT; Hadamard outputs within rtol 1e-3 / atol 1e-3 of the oracle."""
import numpy as np
import pytest
import torch

import quarot_amd
from oracle import quarot_oracle as o
from quarot_amd import _lib
from quarot_amd.transformers import kv_cache as kv

pytestmark = pytest.mark.gpu
F16, F32 = np.float16, np.float32
RTOL = ATOL = 1e-3


def dev():
    return torch.device("cuda:0")


def gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev())


def bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


def synth_x(m, k, seed=0, outliers=True):
    """Activations of the benchmark configs: N(0,1) with 1 % of channels scaled by 20."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g)
    if outliers:
        idx = torch.randperm(k, generator=g)[: -(-k // 100)]
        x[:, idx] *= 20
    return x.half().numpy()


def synth_w(n, k, seed=1):
    """Weights: N(0, 0.02), per-row fp16 scale amax/7, round-to-nearest codes, packed."""
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(n, k, generator=g) * 0.02).half().numpy()
    s = (np.max(np.abs(w), axis=1, keepdims=True).astype(F32) / F32(7)).astype(F16)
    codes = np.clip(np.rint((w.astype(F32) / s.astype(F32)).astype(F16).astype(F32)), -8, 7).astype(np.int8)
    return o.pack_i4(codes), s


# ------------------------------------------------------------------------------ quantiser

@pytest.mark.parametrize("rows,cols", [(1, 8), (5, 64), (33, 4096), (16, 11008), (7, 28672), (4, 32768), (2048, 4096),
                                       (9, 37), (3, 7), (2, 1), (6, 40000), (5, 12)])
def test_quantizer_codes_and_scales_bit_exact(rows, cols):
    x = synth_x(rows, cols, seed=rows * 7 + cols) * F16(1.7)
    for clip in (1.0, 0.9):
        q, s = quarot_amd.quantize_rows(gpu(x), clip)
        wq, ws = o.quantizer(x, clip)
        assert q.shape == (rows, (cols + 1) // 2) and s.shape == (rows, 1)
        assert np.array_equal(s.cpu().numpy().reshape(-1), ws)
        assert np.array_equal(q.cpu().numpy(), wq)


def test_quantizer_module_shapes_follow_reference_quirk():
    x = gpu(synth_x(6 * 5, 64).reshape(6, 5, 64))
    p = quarot_amd.nn.Quantizer()(x)
    assert p.quantized_x.shape == (6, 5, 32)
    assert p.scales_x.shape == (6, 1, 5)            # max(dim=-1)[0].unsqueeze(1) on a 3-D input
    wq, ws = o.quantizer(x.cpu().numpy().reshape(30, 64))
    assert np.array_equal(p.quantized_x.cpu().numpy().reshape(30, 32), wq)
    assert np.array_equal(p.scales_x.cpu().numpy().reshape(-1), ws)


def test_quantizer_zero_rows_and_extremes():
    x = np.zeros((4, 64), F16)
    x[1, 3] = 65504
    x[2, :] = -65504
    x[3, 0] = 6e-8          # smallest subnormal: scale rounds to 0 -> division by zero -> +inf -> 7
    q, s = quarot_amd.quantize_rows(gpu(x))
    wq, ws = o.quantizer(x)
    assert np.array_equal(s.cpu().numpy().reshape(-1), ws) and np.array_equal(q.cpu().numpy(), wq)
    assert not q.cpu().numpy()[0].any()


def test_scale_for_every_finite_fp16_amax():
    v = np.arange(65536, dtype=np.uint16).view(F16)
    v = v[np.isfinite(v)]
    x = np.zeros((v.size, 8), F16)
    x[:, 5] = v
    for clip in (1.0, 0.85):
        _, s = quarot_amd.quantize_rows(gpu(x), clip)
        assert np.array_equal(s.cpu().numpy().reshape(-1), o.quantizer_scales(x, clip))


def test_sym_quant_every_fp16_value_times_many_scales():
    """Brute force of the division + rounding: all finite fp16 x against 240 scales (ties, values
    that round up into a tie, subnormal quotients, overflow), plus zero / inf / NaN scales."""
    v = np.arange(65536, dtype=np.uint16).view(F16)
    v = v[np.isfinite(v)].reshape(2, -1)                                   # 2 x 31744
    rng = np.random.default_rng(0)
    scales = np.concatenate([
        np.abs(rng.standard_normal(100)).astype(F16) + F16(1e-3),
        (2.0 ** rng.integers(-14, 12, 40)).astype(F16),
        rng.integers(1, 65536, 80).astype(np.uint16).view(F16),           # arbitrary bit patterns
        np.array([0.0, -0.0, np.inf, -np.inf, 6e-8, 65504, -1.5, 1 / 3, 7.0, 1 / 7, np.nan, 0.3, 3e-5, -2e-4, 1e-3,
                  0.1, 0.7, 1.1, 13.0, 100.0], F16)])
    x = np.tile(v, (scales.size, 1))
    s = np.repeat(scales, 2)
    got = quarot_amd.sym_quant(gpu(x), gpu(s)).cpu().numpy()
    finite_scale = np.isfinite(s) | np.isinf(s)
    want = o.pack_i4(o.sym_quant_codes(x, s))
    assert np.array_equal(got[finite_scale], want[finite_scale])
    # NaN scale: every quotient is NaN -> code 0
    assert not got[~finite_scale].any()


def test_sym_quant_every_fp16_value_against_every_positive_scale():
    """The lean quantiser forms x / s as ONE fp32 multiplication by the correctly rounded reciprocal of s: every
    finite fp16 value against every positive finite fp16 scale (2 x 31744 x 31743 pairs), judged on the GPU
    against the IEEE sequence the reference's kernel runs (fp32 division, rounding to fp16, round half even,
    clamp), and every 257th scale's rows against the oracle on the CPU as well."""
    pos = torch.from_numpy(np.arange(0, 0x7c00, dtype=np.uint16).view(F16).copy()).cuda()
    scales = pos[1:]
    for sign in (1.0, -1.0):
        vals = (pos * sign).contiguous()
        for c0 in range(0, scales.numel(), 2048):
            s = scales[c0:c0 + 2048].contiguous()
            x = vals.unsqueeze(0).expand(s.numel(), -1).contiguous()
            q = quarot_amd.sym_quant(x, s)
            want = torch.clamp(torch.round((x.float() / s.float().unsqueeze(1)).half().float()), -8, 7).to(torch.int8)
            got = torch.stack([(q & 15).to(torch.int8), (q >> 4).to(torch.int8)], dim=-1).reshape(s.numel(), -1)
            got = torch.where(got > 7, got - 16, got)
            assert torch.equal(got, want), (sign, c0)
            rows = list(range(c0 % 257, s.numel(), 257))
            assert np.array_equal(q[rows].cpu().numpy(), o.pack_i4(o.sym_quant_codes(x[rows].cpu().numpy(), s[rows].cpu().numpy())))


def test_sym_quant_odd_columns_and_views():
    x = synth_x(11, 75, seed=3)
    s = o.quantizer_scales(x)
    got = quarot_amd.sym_quant(gpu(x), gpu(s).view(11, 1))
    assert got.shape == (11, 38)
    assert np.array_equal(got.cpu().numpy(), o.pack_i4(o.sym_quant_codes(x, s)))
    x3 = gpu(x[:10, :64].copy()).view(2, 5, 64)
    got3 = quarot_amd.sym_quant(x3, gpu(s[:10]).view(2, 5))
    assert got3.shape == (2, 5, 32)
    with pytest.raises(RuntimeError):
        quarot_amd.sym_quant(gpu(x), gpu(s[:5]))                            # scale size mismatch
    with pytest.raises(RuntimeError):
        quarot_amd.sym_quant(gpu(x).t().contiguous().t(), gpu(s))           # not contiguous -> view fails


# ------------------------------------------------------------------------------ GEMM / dequant / linear

GEMM_SHAPES = [(1, 1, 64), (32, 32, 64), (33, 65, 128), (64, 64, 192), (100, 200, 192), (128, 128, 256), (1, 256, 4096),
               (8, 300, 1024), (40, 512, 512), (64, 1000, 2048), (65, 256, 320), (129, 257, 448), (256, 512, 4096),
               (300, 700, 11008), (512, 1024, 2048), (1000, 3000, 1024), (2048, 4096, 4096),
               # the pipelined kernels: whole and partly filled K stages, whole and ragged tiles
               (2048, 4096, 320), (2050, 4100, 448), (4096, 4096, 256), (4090, 4090, 192), (2304, 8192, 64),
               # whole stages loaded straight into LDS: every remainder of the stage count modulo the
               # buffer rotation (three buffers at 128x256 tiles, two at 256x256), ragged tiles included
               (2048, 4096, 256), (2048, 4096, 512), (2048, 4096, 768), (2048, 4096, 1280), (2048, 4096, 1536),
               (4096, 4096, 512), (4096, 4096, 768), (4096, 4096, 1024), (2050, 4100, 1024), (4090, 4090, 768)]


@pytest.mark.parametrize("m,n,k", GEMM_SHAPES)
def test_matmul_int32_bit_exact(m, n, k):
    rng = np.random.default_rng(m * 31 + n * 7 + k)
    a = o.pack_i4(rng.integers(-8, 8, (m, k)))
    b = o.pack_i4(rng.integers(-8, 8, (n, k)))
    c = quarot_amd.matmul(gpu(a), gpu(b))
    assert c.dtype == torch.int32 and c.shape == (m, n)
    assert np.array_equal(c.cpu().numpy(), o.int4_matmul(a, b))


def test_matmul_and_linear_random_shapes_across_every_kernel_boundary():
    """Seeded random shapes around the dispatcher's thresholds (matrix-vector <= 4 rows, decode <= 64,
    tile counts that select the 64x256, 128x256 and 256x256 kernels, whole and ragged K stages, the
    workspace split): int32 product and fused fp16 output against the oracle, bit for bit."""
    rng = np.random.default_rng(2024)
    shapes = []
    for _ in range(14):
        shapes.append((int(rng.integers(1, 200)), int(rng.integers(1, 700)), 64 * int(rng.integers(1, 17))))
    for m in (4, 5, 64, 65):
        shapes.append((m, int(rng.integers(250, 530)), 64 * int(rng.integers(1, 9))))
    for _ in range(6):                                   # enough tiles for the pipelined kernels
        shapes.append((int(rng.integers(1800, 2300)), int(rng.integers(3900, 4300)), 64 * int(rng.integers(1, 13))))
    shapes += [(70, 300, 4096), (140, 1030, 2048), (2048, 8192, 256), (4100, 4100, 512)]
    # few tokens and many weight rows: the decode kernel with K split four ways (N > 8192) and two ways
    # (N > 16384) within a row group, every token-count variant, ragged N and a ragged last K step
    shapes += [(5, 8207, 320), (16, 8450, 1024), (17, 9001, 192), (32, 8333, 576),
               (8, 16531, 192), (9, 16700, 768), (24, 17001, 320), (32, 16385, 128)]
    for (m, n, k) in shapes:
        a = o.pack_i4(rng.integers(-8, 8, (m, k)))
        w = o.pack_i4(rng.integers(-8, 8, (n, k)))
        want = o.int4_matmul(a, w)
        c = quarot_amd.matmul(gpu(a), gpu(w))
        assert np.array_equal(c.cpu().numpy(), want), (m, n, k)
        sa = (np.abs(rng.standard_normal(m)) * 0.2 + 0.01).astype(F16)
        sw = (np.abs(rng.standard_normal(n)) * 0.01 + 0.001).astype(F16)
        bias = rng.standard_normal(n).astype(F16)
        y = quarot_amd.linear_i4(gpu(a), gpu(sa), gpu(w), gpu(sw), gpu(bias))
        assert np.array_equal(bits(y.cpu().numpy()), bits(o.sym_dequant(want, sa, sw, bias))), (m, n, k)


@pytest.mark.parametrize("m,n,k", [(2047, 4096, 256), (2049, 4096, 320), (1900, 4096, 128), (1153, 8192, 128), (1025, 8192, 192),
                                   (300, 512, 192), (130, 4096, 1024), (97, 1024, 2048), (65, 768, 64), (4001, 4096, 64),
                                   (257, 2048, 448), (161, 256, 4096),
                                   # 192-row tiles (fewer rounds over the CUs than 128- or 256-row ones), whole K stages
                                   (2049, 4096, 512), (1153, 8192, 256), (1920, 5120, 256), (2048, 5120, 768)])
def test_linear_token_counts_that_end_inside_a_row_tile(m, n, k):
    """Prompt lengths that are no multiple of the kernels' tile heights (32-row slabs of 64/128/256-row tiles)
    against weights whose rows fill whole tiles: the last row tile stores exactly the rows that exist.  Through
    the C-ABI into a buffer with a guard band behind the last row, with and without bias, on the int8 and the
    FP6 matrix paths; the oracle decides bit for bit."""
    from quarot_amd import _lib
    rng = np.random.default_rng(m * 3 + n + k)
    a, w = o.pack_i4(rng.integers(-8, 8, (m, k))), o.pack_i4(rng.integers(-8, 8, (n, k)))
    sa = (np.abs(rng.standard_normal(m)) * 0.2 + 0.01).astype(F16)
    sw = (np.abs(rng.standard_normal(n)) * 0.01 + 0.001).astype(F16)
    bias = rng.standard_normal(n).astype(F16)
    acc = o.int4_matmul(a, w)
    ga, gw, gsa, gsw, gb = gpu(a), gpu(w), gpu(sa), gpu(sw), gpu(bias)
    a6, w6 = quarot_amd.convert_i4_f6(ga), quarot_amd.convert_i4_f6(gw)
    L = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    guard = 40                                               # rows behind the output that no kernel may touch
    for b, nb in ((gb, bias), (None, None)):
        want = bits(o.sym_dequant(acc, sa, sw, nb))
        for path in ("i8", "f6"):
            buf = torch.full((m + guard, n), 12345.0, dtype=torch.float16, device="cuda")
            bp = b.data_ptr() if b is not None else None
            if path == "i8":
                rc = L.qr_linear_i4_f16(ga.data_ptr(), gsa.data_ptr(), gw.data_ptr(), gsw.data_ptr(), bp, m, n, k,
                                        buf.data_ptr(), stream)
            else:
                rc = L.qr_linear_f6_f16(a6.data_ptr(), gsa.data_ptr(), w6.data_ptr(), gsw.data_ptr(), bp, m, n, k,
                                        buf.data_ptr(), stream)
            assert rc == 0, (path, rc)
            got = buf.cpu().numpy()
            assert np.array_equal(bits(got[:m]), want), (path, nb is not None)
            assert (got[m:] == 12345.0).all(), (path, "rows behind the output were written")


@pytest.mark.parametrize("n", [25600, 35200, 44800, 57344, 65536, 57339, 65500])
def test_decode_with_many_weight_rows_shares_the_tokens_through_lds(n):
    """Decode batches (5..64 tokens) against enough weight rows to give every CU a workgroup of 4..8 groups
    of 32 rows (the five listed multiples pick 4, 5, 6, 7 and 8 groups; the last two end in a ragged
    group): one and two token tiles, a token count that is not a multiple of 32, a single K stage, a
    ragged last stage, and workgroups that start their walk over K at different stages."""
    rng = np.random.default_rng(n)
    for k in (64, 1088):
        w = o.pack_i4(rng.integers(-8, 8, (n, k)))
        sw = (np.abs(rng.standard_normal(n)) * 0.01 + 0.001).astype(F16)
        bias = rng.standard_normal(n).astype(F16)
        wg = gpu(w)
        for m in ((5, 33, 64) if n != 57344 else (5, 17, 32, 33, 48, 64)):
            a = o.pack_i4(rng.integers(-8, 8, (m, k)))
            sa = (np.abs(rng.standard_normal(m)) * 0.2 + 0.01).astype(F16)
            want = o.int4_matmul(a, w)
            c = quarot_amd.matmul(gpu(a), wg)
            assert np.array_equal(c.cpu().numpy(), want), (m, n, k)
            y = quarot_amd.linear_i4(gpu(a), gpu(sa), wg, gpu(sw), gpu(bias))
            assert np.array_equal(bits(y.cpu().numpy()), bits(o.sym_dequant(want, sa, sw, bias))), (m, n, k)
            y = quarot_amd.linear_i4(gpu(a), gpu(sa), wg, gpu(sw))
            assert np.array_equal(bits(y.cpu().numpy()), bits(o.sym_dequant(want, sa, sw))), (m, n, k)


def f6_value(code):
    """The real value of a 6-bit FP6 E3M2 code (sign, 3 exponent bits with bias 3, 2 mantissa bits)."""
    s, e, f = code >> 5, (code >> 2) & 7, code & 3
    mag = f * 0.0625 if e == 0 else (1 + f / 4) * 2.0 ** (e - 3)
    return -mag if s else mag


def test_fp6_conversion_holds_every_code_exactly():
    """convert_i4_f6 against the format's definition: every 6-bit field of the converted operand decodes to
    an int4 value, and each (row, stage, half) group of 32 fields holds exactly the 32 codes of that part of
    the row (the order inside a group is the converter's own: both GEMM operands share it)."""
    rng = np.random.default_rng(6)
    rows, k = 37, 192
    vals = rng.integers(-8, 8, (rows, k))
    vals[0, :16] = np.arange(-8, 8)
    out = quarot_amd.convert_i4_f6(gpu(o.pack_i4(vals))).cpu().numpy()
    assert out.shape == (k // 64, rows, 48) and out.dtype == np.uint8
    bits = np.unpackbits(out.reshape(k // 64, rows, 2, 24), axis=-1, bitorder="little")      # [stage, row, half, 192 bits]
    for half in (0, 1):
        b = bits[:, :, half, :]
        if half == 1:                                       # stored as [last 8 bytes][first 16 bytes]
            b = np.concatenate([b[..., 64:], b[..., :64]], axis=-1)
        fields = (b.reshape(k // 64, rows, 32, 6) * (1 << np.arange(6))).sum(-1)
        decoded = np.vectorize(f6_value)(fields)
        for st in range(k // 64):
            want = vals[:, st * 64 + half * 32: st * 64 + half * 32 + 32]
            assert np.array_equal(np.sort(decoded[st], axis=-1), np.sort(want, axis=-1)), (st, half)


@pytest.mark.parametrize("m,n,k", [(1, 1, 64), (33, 65, 128), (256, 256, 64), (300, 520, 192), (257, 511, 320),
                                   (1024, 768, 4096), (2048, 4096, 11008), (4100, 4090, 448), (8200, 8190, 128)])
def test_linear_on_the_fp6_matrix_path_bit_exact(m, n, k):
    """qr_linear_f6_f16 on converted operands: the fused fp16 output against the oracle bit for bit (small shapes:
    every element; large: the int8 path, itself checked against the oracle elsewhere, plus oracle rows), ragged
    tiles, one and many K stages, extreme codes, with and without bias."""
    rng = np.random.default_rng(m + n + k)
    av, wv = rng.integers(-8, 8, (m, k)), rng.integers(-8, 8, (n, k))
    av[0, :], wv[0, :] = -8, -8                          # the largest possible sum: 64 k
    a, w = o.pack_i4(av), o.pack_i4(wv)
    sa = (np.abs(rng.standard_normal(m)) * 0.2 + 0.01).astype(F16)
    sw = (np.abs(rng.standard_normal(n)) * 0.01 + 0.001).astype(F16)
    bias = rng.standard_normal(n).astype(F16)
    ga, gw, gsa, gsw, gb = gpu(a), gpu(w), gpu(sa), gpu(sw), gpu(bias)
    a6, w6 = quarot_amd.convert_i4_f6(ga), quarot_amd.convert_i4_f6(gw)
    for b, nb in ((gb, bias), (None, None)):
        y = quarot_amd.linear_f6(a6, gsa, w6, gsw, b)
        assert y.dtype == torch.float16 and y.shape == (m, n)
        if m * n * k <= 1 << 27:
            assert np.array_equal(bits(y.cpu().numpy()), bits(o.sym_dequant(o.int4_matmul(a, w), sa, sw, nb)))
        else:
            assert torch.equal(y, quarot_amd.linear_i4(ga, gsa, gw, gsw, b))
            rows = sorted(set([0, m - 1] + [int(v) for v in rng.integers(0, m, 6)]))
            want = o.sym_dequant(o.int4_matmul(a[rows], w), sa[rows], sw, nb)
            assert np.array_equal(bits(y[rows].cpu().numpy()), bits(want))


def test_linear4bit_opt_in_fp6_prefill_equals_the_default_path():
    lin = quarot_amd.nn.Linear4bit(512, 384, bias=True).half().cuda()
    rng = np.random.default_rng(5)
    lin.weight.copy_(gpu(o.pack_i4(rng.integers(-8, 8, (384, 512)))))
    lin.weight_scales.copy_(gpu((np.abs(rng.standard_normal((384, 1))) * 0.01 + 0.001).astype(F16)))
    lin.bias.copy_(gpu(rng.standard_normal(384).astype(F16)))
    x = quarot_amd.nn.Quantizer()(gpu(rng.standard_normal((600, 512)).astype(F16)))
    want = lin(x)
    lin.prefill_fp6, lin.fp6_min_rows = True, 256
    assert torch.equal(lin(x), want)
    lin.weight.copy_(gpu(o.pack_i4(rng.integers(-8, 8, (384, 512)))))      # new weights: the 6-bit copy is rebuilt
    got = lin(x)
    lin.prefill_fp6 = False
    assert torch.equal(got, lin(x))


def test_enable_fp6_prefill_on_a_module_tree_changes_no_result():
    """enable_fp6_prefill switches every Linear4bit of a model; the reference-shaped chains (Linear4bitSequential with
    and without the online Hadamard) then take the FP6 route for long inputs and the usual one for short ones,
    with identical outputs."""
    nn_ = quarot_amd.nn
    rng = np.random.default_rng(11)
    def lin(k, n):
        m = nn_.Linear4bit(k, n).half().cuda()
        m.weight.copy_(gpu(o.pack_i4(rng.integers(-8, 8, (n, k)))))
        m.weight_scales.copy_(gpu((np.abs(rng.standard_normal((n, 1))) * 0.01 + 0.001).astype(F16)))
        return m
    model = torch.nn.ModuleDict({
        "down": nn_.Linear4bitSequential(nn_.OnlineHadamard(2304), nn_.Quantizer(0.9), lin(2304, 320)),
        "q": nn_.Linear4bitSequential(nn_.Quantizer(), lin(512, 384)),
    }).cuda()
    xs = {"down": gpu(synth_x(700, 2304, seed=3)), "q": gpu(synth_x(700, 512, seed=4))}
    want = {k: model[k](xs[k]) for k in xs}
    assert nn_.enable_fp6_prefill(model, min_rows=256) == 2
    for k in xs:
        assert model[k][-1]._f6_cache is not None                       # converted at once
        assert torch.equal(model[k](xs[k]), want[k])                    # long input: FP6 route
        assert torch.equal(model[k](xs[k][:100]), want[k][:100])        # short input: the usual route


def test_fp6_prefill_keeps_the_leading_dimensions_of_a_batched_input():
    """[batch, seq, hidden] inputs: the FP6 route returns [batch, seq, out] like the default route and the reference's
    matmul (quarot/__init__.py:37-41 views the result as (*A.shape[:-1], -1)), directly and through the chains."""
    nn_ = quarot_amd.nn
    rng = np.random.default_rng(17)
    def lin(k, n):
        m = nn_.Linear4bit(k, n, bias=True).half().cuda()
        m.weight.copy_(gpu(o.pack_i4(rng.integers(-8, 8, (n, k)))))
        m.weight_scales.copy_(gpu((np.abs(rng.standard_normal((n, 1))) * 0.01 + 0.001).astype(F16)))
        m.bias.copy_(gpu(rng.standard_normal(n).astype(F16)))
        return m
    chains = {"plain": nn_.Linear4bitSequential(nn_.Quantizer(), lin(512, 384)),
              "had": nn_.Linear4bitSequential(nn_.OnlineHadamard(2304), nn_.Quantizer(), lin(2304, 320))}
    for name, chain in chains.items():
        chain = chain.cuda()
        k = chain[-1].in_features
        x = gpu(synth_x(600, k, seed=21).reshape(2, 300, k))
        want = chain(x)
        packed = chain[-2](x if name == "plain" else chain[0](x))
        want_direct = chain[-1](packed)
        assert want.shape == want_direct.shape == (2, 300, chain[-1].out_features)
        assert nn_.enable_fp6_prefill(chain, min_rows=256) == 1
        got, got_direct = chain(x), chain[-1](packed)
        assert got.shape == want.shape and torch.equal(got, want)
        assert got_direct.shape == want_direct.shape and torch.equal(got_direct, want_direct)


def test_matmul_known_answers_and_leading_dims():
    k = 28672                                      # the largest K of the configs: |acc| = 64 K = 1 835 008
    a = np.full((3, k // 2), 0x88, np.uint8)       # all -8
    b = np.full((5, k // 2), 0x88, np.uint8)
    assert (quarot_amd.matmul(gpu(a), gpu(b)).cpu().numpy() == 64 * k).all()
    b7 = np.full((5, k // 2), 0x77, np.uint8)      # all 7
    assert (quarot_amd.matmul(gpu(a), gpu(b7)).cpu().numpy() == -56 * k).all()
    rng = np.random.default_rng(1)
    a3 = o.pack_i4(rng.integers(-8, 8, (6, 128))).reshape(2, 3, 64)
    b2 = o.pack_i4(rng.integers(-8, 8, (7, 128)))
    c = quarot_amd.matmul(gpu(a3), gpu(b2))
    assert c.shape == (2, 3, 7)
    assert np.array_equal(c.cpu().numpy().reshape(6, 7), o.int4_matmul(a3.reshape(6, 64), b2))


@pytest.mark.parametrize("rows,cols", [(1, 1), (7, 13), (64, 64), (100, 4096), (33, 1000), (2048, 4096)])
def test_sym_dequant_bit_exact(rows, cols):
    rng = np.random.default_rng(rows + cols)
    q = rng.integers(-70000, 70000, (rows, cols)).astype(np.int32)          # crosses 2048 (11-bit) and 65520 (inf)
    q.reshape(-1)[:4] = [2049, 65519, 65520, -(1 << 30)][: min(4, q.size)]
    sr = (np.abs(rng.standard_normal(rows)) * 0.1).astype(F16)
    sc = (np.abs(rng.standard_normal(cols)) * 0.01).astype(F16)
    y = quarot_amd.sym_dequant(gpu(q), gpu(sr).view(rows, 1), gpu(sc).view(cols, 1))
    assert y.dtype == torch.float16 and y.shape == (rows, cols)
    assert np.array_equal(bits(y.cpu().numpy()), bits(o.sym_dequant(q, sr, sc)))
    with pytest.raises(RuntimeError, match="Unsupported"):
        quarot_amd.sym_dequant(gpu(q), gpu(sr), gpu(sc), bits=8)


@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (33, 65, 128), (64, 512, 1024), (100, 200, 192), (300, 700, 11008),
                                   (512, 1024, 2048), (2048, 4096, 4096), (2048, 4096, 320), (2050, 4100, 448),
                                   (4096, 4096, 256), (4090, 4096, 192), (2048, 4096, 512), (2048, 4096, 1280),
                                   (4096, 4096, 768), (2050, 4096, 1024), (8, 8192, 2048), (16, 8192, 1024),
                                   (24, 8192, 512), (48, 8192, 1024)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_linear_fused_equals_staged_reference_ops(m, n, k, with_bias):
    rng = np.random.default_rng(m + n + k)
    a = o.pack_i4(rng.integers(-8, 8, (m, k)))
    w = o.pack_i4(rng.integers(-8, 8, (n, k)))
    sa = (np.abs(rng.standard_normal(m)) * 0.2).astype(F16)
    sw = (np.abs(rng.standard_normal(n)) * 0.01).astype(F16)
    bias = rng.standard_normal(n).astype(F16) if with_bias else None
    y = quarot_amd.linear_i4(gpu(a), gpu(sa).view(m, 1), gpu(w), gpu(sw).view(n, 1), None if bias is None else gpu(bias))
    want = o.linear4bit(a, sa, w, sw, bias)
    assert np.array_equal(bits(y.cpu().numpy()), bits(want))
    # and equals the staged calls of the reference API
    staged = quarot_amd.sym_dequant(quarot_amd.matmul(gpu(a), gpu(w)), gpu(sa), gpu(sw).view(n, 1))
    if bias is not None:
        staged = staged + gpu(bias)
    assert torch.equal(staged, y)


@pytest.mark.parametrize("m,n,k", [(128, 4096, 4096), (300, 700, 11008), (96, 512, 8192), (130, 520, 4160),
                                   (256, 4096, 11008)])
def test_linear_with_workspace_splits_k_and_matches_bit_for_bit(m, n, k):
    """Shapes with few output tiles: with the scratch buffer the library splits K across workgroups
    (int32 partial sums in slabs, then one summing dequantisation); the result must equal both the
    oracle and the single-launch path bit for bit, with and without bias, and a missing or too small
    workspace must silently select the single-launch path."""
    L = _lib.lib()
    ws_bytes = L.qr_workspace_bytes(m, n, k)
    assert ws_bytes > 0
    rng = np.random.default_rng(m + n + k)
    a = o.pack_i4(rng.integers(-8, 8, (m, k)))
    w = o.pack_i4(rng.integers(-8, 8, (n, k)))
    sa = (np.abs(rng.standard_normal(m)) * 0.2).astype(F16)
    sw = (np.abs(rng.standard_normal(n)) * 0.01).astype(F16)
    bias = rng.standard_normal(n).astype(F16)
    ga, gw, gsa, gsw, gb = gpu(a), gpu(w), gpu(sa), gpu(sw), gpu(bias)
    st = torch.cuda.current_stream().cuda_stream
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=ga.device)
    for b_np, b_gpu in ((None, None), (bias, gb)):
        want = o.linear4bit(a, sa, w, sw, b_np)
        outs = []
        for wptr, wbytes in ((ws.data_ptr(), ws_bytes), (None, 0), (ws.data_ptr(), ws_bytes - 4)):
            y = torch.full((m, n), float("nan"), dtype=torch.float16, device=ga.device)
            rc = L.qr_linear_i4_f16_ws(ga.data_ptr(), gsa.data_ptr(), gw.data_ptr(), gsw.data_ptr(),
                                       None if b_gpu is None else b_gpu.data_ptr(), m, n, k, y.data_ptr(), wptr, wbytes, st)
            assert rc == 0
            outs.append(y.cpu().numpy())
        for got in outs:
            assert np.array_equal(bits(got), bits(want))
        # the Python entry point takes the split path by itself
        y = quarot_amd.linear_i4(ga, gsa, gw, gsw, b_gpu)
        assert np.array_equal(bits(y.cpu().numpy()), bits(want))


def test_linear4bit_module_from_float_and_state_dict():
    w = (torch.randn(96, 128, generator=torch.Generator().manual_seed(4)) * 0.02).half()
    s = (w.abs().amax(dim=1, keepdim=True) / 7).half()
    lin = torch.nn.Linear(128, 96, bias=True).half()
    lin.weight.data = w
    lin.bias.data = torch.randn(96, generator=torch.Generator().manual_seed(5)).half()
    q4 = quarot_amd.nn.Linear4bit.from_float(lin, weight_scales=s).cuda()
    assert np.array_equal(q4.weight.cpu().numpy(), o.weight_codes_from_float(w.numpy(), s.numpy()))
    x = gpu(synth_x(10, 128, seed=6))
    seq = torch.nn.Sequential(quarot_amd.nn.Quantizer(), q4)
    y = seq(x)
    xq, xs = o.quantizer(x.cpu().numpy())
    want = o.linear4bit(xq, xs, q4.weight.cpu().numpy(), s.numpy(), lin.bias.data.numpy())
    assert np.array_equal(bits(y.cpu().numpy()), bits(want))
    clone = quarot_amd.nn.Linear4bit(128, 96, bias=True).half().cuda()   # buffers are fp32 until cast, as in the reference
    clone.load_state_dict(q4.state_dict())
    assert torch.equal(clone(quarot_amd.nn.Quantizer()(x)), y)


# ------------------------------------------------------------------------------ Hadamard

HAD_SIZES = [4, 12, 24, 40, 112, 120, 8, 16, 32, 64, 128, 512, 1024, 2048, 4096, 8192, 16384, 32768, 96, 224, 320, 1376, 2304, 3840, 5120, 6912, 8960, 9984, 11008, 13824, 14336, 28672, 12288, 20480, 6656, 17920]


def close(got, want):
    g, w = got.astype(np.float64), want.astype(np.float64)
    return np.all(np.abs(g - w) <= ATOL + RTOL * np.abs(w))


@pytest.mark.parametrize("n", HAD_SIZES)
@pytest.mark.parametrize("dtype", [F16, F32])
def test_hadamard_within_tolerance(n, dtype):
    x = (synth_x(6, n, seed=n) if dtype == F16 else synth_x(6, n, seed=n).astype(F32) * F32(1.001))
    hadk, k = quarot_amd.functional.hadamard.get_hadK(n)
    y = quarot_amd.functional.matmul_hadU_cuda(gpu(x), None if hadk is None else hadk.cuda(), k)
    assert y.dtype == (torch.float16 if dtype == F16 else torch.float32) and y.shape == (6, n)
    ho, ko = o.get_hadK(n)
    got = y.cpu().numpy()
    assert close(got, o.hadamard_staged(x, ho, ko, dtype))
    # float64 closed form: the transform itself (kron orientation, natural order, scale)
    cf = o.hadamard_closed_form(x.astype(np.float64))
    tol = 3e-3 if dtype == F16 else 1e-5
    assert np.all(np.abs(got - cf) <= tol * (1 + np.abs(cf)))


def test_hadamard_across_forty_heads():
    """Llama-2-13B has 40 attention heads: OnlineHadamard(40) is had_40 alone (power-of-two factor 1),
    applied by the reference to a transposed view.  Row counts that leave a partly filled last block of
    64, fp16 and fp32, and the module that chains it with the quantiser (separate steps for this head
    count) against the oracle."""
    hadk, k = quarot_amd.functional.hadamard.get_hadK(40)
    assert k == 40
    for rows in (1, 63, 1000):
        x = synth_x(rows, 40, seed=rows)
        y = quarot_amd.functional.matmul_hadU_cuda(gpu(x), hadk.cuda(), k)
        assert close(y.cpu().numpy(), o.online_hadamard(x))
        xf = x.astype(F32) * F32(1.003)
        yf = quarot_amd.functional.matmul_hadU_cuda(gpu(xf), hadk.cuda(), k)
        assert np.allclose(yf.cpu().numpy(), o.hadamard_closed_form(xf.astype(np.float64)), rtol=1e-5, atol=1e-5)
    # the module for 40 and 52 heads (Llama-2-13B, Llama-30B): one kernel with the table as a matrix;
    # its own fp16 rows within tolerance of the oracle, codes and scales bit-exact on those rows
    for heads, rows in ((40, 7), (52, 70), (12, 3)):
        xa = gpu(synth_x(rows, heads * 128, seed=heads)).view(rows, heads, 128)
        mod = quarot_amd.nn.HeadsHadamardQuantizer(heads, input_clip_ratio=0.95).cuda()
        p = mod(xa)
        p2, y = quarot_amd.heads_hadamard_quantize(xa, heads, 0.95, return_transformed=True, hadK=mod.had.had_rem_dim)
        assert torch.equal(p.quantized_x, p2.quantized_x) and torch.equal(p.scales_x, p2.scales_x)
        yk = y.cpu().numpy()
        want_y = o.heads_hadamard(xa.cpu().numpy(), heads)
        assert close(yk, want_y) and np.mean(yk == want_y) > 0.99
        wq, ws = o.quantizer(yk, 0.95)
        assert np.array_equal(p.quantized_x.cpu().numpy(), wq)
        assert np.array_equal(p.scales_x.cpu().numpy().reshape(-1), ws)
        staged = mod.had(xa.transpose(-1, -2)).transpose(-1, -2).reshape(rows, heads * 128).contiguous()
        assert close(staged.cpu().numpy(), want_y)
    # 24 heads = had_12 (x) H_2: neither form of the fused kernel, the module runs the separate steps
    xb = gpu(synth_x(5, 24 * 128, seed=6)).view(5, 24, 128)
    pb = quarot_amd.nn.HeadsHadamardQuantizer(24).cuda()(xb)
    wq, _ = o.quantizer(o.heads_hadamard(xb.cpu().numpy(), 24), 1.0)
    assert pb.quantized_x.shape == (5, 12 * 128) and np.mean(pb.quantized_x.cpu().numpy() == wq) > 0.99


@pytest.mark.parametrize("n", [8, 16, 32, 64])
def test_hadamard_short_rows_many_per_workgroup(n):
    """Short rows (the transform across attention heads on a transposed copy): row counts that leave
    a partly filled last wave and more chunks than one pass of the grid covers, out of place and in
    place, against the oracle and through the involution H(H(x)) = x."""
    for rows in (1, 37, 1000, 262144 + 3):
        x = gpu(synth_x(min(rows, 4096), n, seed=n + rows))
        if rows > 4096:
            x = x.repeat((rows + 4095) // 4096, 1)[:rows].contiguous()
        y = quarot_amd.functional.matmul_hadU_cuda(x, None, 1)
        sl = slice(None, None, max(1, rows // 500))
        assert close(y[sl].cpu().numpy(), o.online_hadamard(x[sl].cpu().numpy()))
        assert close(y[-3:].cpu().numpy(), o.online_hadamard(x[-3:].cpu().numpy()))
        # two fp16 roundings, each relative to the largest element of the row (outlier channels)
        back = quarot_amd.functional.matmul_hadU_cuda(y, None, 1)
        err = (back.float() - x.float()).abs().amax(dim=1)
        assert bool((err <= 2e-3 * x.float().abs().amax(dim=1) + 1e-3).all())


@pytest.mark.parametrize("n", [64, 1024, 4096, 8192, 16384, 224, 3840, 6912, 8960, 11008, 28672, 13824, 5120, 6656, 4608, 7680, 17920, 22016, 12288, 20480])
@pytest.mark.parametrize("fp32", [False, True])
def test_fused_hadamard_quantize_equals_staged(n, fp32):
    """Codes of the fused kernel are judged on the kernel's OWN fp16 Hadamard output (returned on
    request): they must equal the oracle quantiser applied to it, bit for bit.  That output in
    turn must agree with the staged module chain (identical in fp16 mode, where both run the same
    arithmetic; within tolerance in fp32 mode, where the staged chain goes through fp32 tensors)."""
    x = gpu(synth_x(9, n, seed=n + 1))
    had = quarot_amd.nn.OnlineHadamard(n, force_fp32=fp32).cuda()
    fused = quarot_amd.nn.OnlineHadamardQuantizer(n, force_fp32=fp32, input_clip_ratio=0.95).cuda()
    p2, y2 = quarot_amd.hadamard_quantize(x, fused.had_rem_dim, fused.rem_dim, 0.95, force_fp32=fp32, return_transformed=True)
    wq, ws = o.quantizer(y2.cpu().numpy(), 0.95)
    assert np.array_equal(p2.quantized_x.cpu().numpy(), wq)
    assert np.array_equal(p2.scales_x.cpu().numpy().reshape(-1), ws)
    p = fused(x)                                                   # without the extra output: same codes
    assert torch.equal(p.quantized_x, p2.quantized_x) and torch.equal(p.scales_x, p2.scales_x)
    staged = quarot_amd.nn.Quantizer(0.95)(y2)                     # the standalone quantiser kernel agrees
    assert torch.equal(staged.quantized_x, p2.quantized_x) and torch.equal(staged.scales_x, p2.scales_x)
    y = had(x)                                                     # the staged module
    if fp32:
        assert close(y2.cpu().numpy(), y.cpu().numpy()) and float((y2 == y).float().mean()) > 0.99
    else:
        assert torch.equal(y2, y)
    assert close(y2.cpu().numpy(), o.online_hadamard(x.cpu().numpy(), force_fp32=fp32))


def test_fused_fronts_random_shapes_scales_and_clips():
    """Seeded random sweep over the fused Hadamard+quantise kernels: widths of every kernel family, 1 .. 1500 rows,
    data from 1e-5 to 300 with outlier columns, clip ratios 1.0 / 0.95 / 0.9, both precisions, a zero row, rows
    with an infinity, a NaN or saturating values.  The call without the transformed copy (the lean kernels), the
    call with it and the standalone quantiser on that copy must agree bit for bit, and on every finite non-zero
    row the codes and scales must be those of the IEEE sequence the reference runs (amax / 7, * clip, fp32
    division, rounding to fp16, round half even, clamp), evaluated by torch on the GPU."""
    rng = np.random.default_rng(11)
    sizes = [64, 128, 1024, 4096, 8192, 224, 3840, 6912, 8960, 11008, 28672, 13824, 5120, 6656, 4608, 7680, 17920, 22016]

    def unpack(p):
        v = torch.stack([(p & 15).to(torch.int8), (p >> 4).to(torch.int8)], dim=-1).reshape(p.shape[0], -1)
        return torch.where(v > 7, v - 16, v)

    for case in range(48):
        n = int(sizes[case % len(sizes)])
        rows = int(rng.choice([rng.integers(1, 40), rng.integers(40, 1500)]))
        clip = float(rng.choice([1.0, 1.0, 0.9, 0.95]))
        fp32 = bool(rng.random() < 0.3)
        x = torch.randn(rows, n, device="cuda") * float(rng.choice([1e-5, 1e-3, 1.0, 30.0, 300.0]))
        x[:, ::int(rng.integers(50, 200))] *= 20
        x = x.half()
        if rows > 3:
            x[1] = 0
            x[2, int(rng.integers(0, n))] = float("inf")
            x[3, int(rng.integers(0, n))] = float("nan")
            x[0] = 60000.0
        fused = quarot_amd.nn.OnlineHadamardQuantizer(n, force_fp32=fp32, input_clip_ratio=clip).cuda()
        p2, y2 = quarot_amd.hadamard_quantize(x, fused.had_rem_dim, fused.rem_dim, clip, force_fp32=fp32, return_transformed=True)
        p = fused(x)
        tag = (n, rows, clip, fp32)
        assert torch.equal(p.quantized_x, p2.quantized_x) and torch.equal(p.scales_x.view(torch.int16), p2.scales_x.view(torch.int16)), tag
        st = quarot_amd.nn.Quantizer(clip)(y2)
        assert torch.equal(st.quantized_x, p2.quantized_x) and torch.equal(st.scales_x.view(torch.int16), p2.scales_x.view(torch.int16)), tag
        ok = torch.isfinite(y2).all(dim=1) & (y2.abs().amax(dim=1) > 0)
        scale = ((y2.abs().amax(dim=1, keepdim=True).float() / 7).half().float() * clip).half()
        want = torch.clamp(torch.round((y2.float() / scale.float()).half().float()), -8, 7).to(torch.int8)
        assert torch.equal(unpack(p2.quantized_x)[ok], want[ok]), tag
        assert torch.equal(p2.scales_x.reshape(-1)[ok].view(torch.int16), scale.reshape(-1)[ok].view(torch.int16)), tag


@pytest.mark.parametrize("n", [53248, 40960])
def test_rows_longer_than_the_fused_kernels_take_the_references_two_steps(n):
    """53248 = 52 x 1024 (the widest Llama-3.1 MLP) and 40960 = 40 x 1024 are beyond the library's two-factor
    kernels (n <= 32768): the Python layer runs the reference's own sequence (quarot/functional/hadamard.py:97-101) --
    the FWHT kernel over the [.., K, n / K] view, then the table as a library GEMM -- and the quantiser kernel behind
    it.  Transform within tolerance of the oracle's staged arithmetic, codes and scales the oracle quantiser's on the
    transformed rows, the fused module and the one-call linear layer bit for bit the chain."""
    x = gpu(synth_x(5, n, seed=n))
    for fp32 in (False, True):
        had = quarot_amd.nn.OnlineHadamard(n, force_fp32=fp32).cuda()
        assert had.rem_dim == o.get_hadK(n)[1]
        y = had(x)
        assert y.dtype == torch.float16 and y.shape == x.shape
        assert close(y.cpu().numpy(), o.online_hadamard(x.cpu().numpy(), force_fp32=fp32))
        fused = quarot_amd.nn.OnlineHadamardQuantizer(n, force_fp32=fp32, input_clip_ratio=0.9).cuda()
        p = fused(x)
        wq, ws = o.quantizer(y.cpu().numpy(), 0.9)
        assert np.array_equal(p.quantized_x.cpu().numpy(), wq) and np.array_equal(p.scales_x.cpu().numpy().reshape(-1), ws)
        p2, y2 = quarot_amd.hadamard_quantize(x, fused.had_rem_dim, fused.rem_dim, 0.9, force_fp32=fp32, return_transformed=True)
        assert torch.equal(y2, y) and torch.equal(p2.quantized_x, p.quantized_x)
    g = torch.Generator().manual_seed(n)
    w = torch.randint(0, 256, (70, n // 2), dtype=torch.uint8, generator=g).cuda()
    sw = (torch.rand(70, 1, generator=g) * 0.02 + 1e-3).half().cuda()
    b = torch.randn(70, generator=g).half().cuda()
    fused = quarot_amd.nn.OnlineHadamardQuantizer(n, input_clip_ratio=1.0).cuda()
    for m in (1, 5):
        pm = fused(x[:m])
        want = quarot_amd.linear_i4(pm.quantized_x, pm.scales_x, w, sw, b)
        got = quarot_amd.quantized_linear(x[:m], w, sw, b, fused.had_rem_dim, fused.rem_dim, 1.0)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
        ref = o.linear4bit(pm.quantized_x.cpu().numpy(), pm.scales_x.cpu().numpy().reshape(-1), w.cpu().numpy(), sw.cpu().numpy(), b.cpu().numpy())
        assert np.array_equal(bits(got.cpu().numpy()), bits(np.asarray(ref).reshape(m, 70)))


@pytest.mark.parametrize("n", [128, 112, 80, 48, 24])
def test_fused_front_on_short_rows_carries_the_bits_of_the_two_modules(n):
    """Rows of 128 (the head dimension: qr_hadamard has a kernel of its own for them, which adds in another order
    than the general one) and rows too short for the fused kernels: OnlineHadamardQuantizer must return what
    Sequential(OnlineHadamard, Quantizer) returns, bit for bit, also on data whose dynamic range makes the order of
    the fp32 additions visible in the last fp16 bit; the one-call linear layer likewise."""
    torch.manual_seed(n)
    rows = 20000 if n == 128 else 3000
    x = torch.randn(rows, n, device="cuda") * 300
    x[:, ::7] *= 20
    x = x.half()
    for fp32 in (False, True):
        had = quarot_amd.nn.OnlineHadamard(n, force_fp32=fp32).cuda()
        fused = quarot_amd.nn.OnlineHadamardQuantizer(n, force_fp32=fp32, input_clip_ratio=0.9).cuda()
        y = had(x)
        want = quarot_amd.nn.Quantizer(0.9)(y)
        p = fused(x)
        p2, y2 = quarot_amd.hadamard_quantize(x, fused.had_rem_dim, fused.rem_dim, 0.9, force_fp32=fp32, return_transformed=True)
        assert torch.equal(y2, y), (n, fp32)
        for got in (p, p2):
            assert torch.equal(got.quantized_x, want.quantized_x), (n, fp32)
            assert torch.equal(got.scales_x.view(torch.int16), want.scales_x.view(torch.int16)), (n, fp32)
        wq, ws = o.quantizer(y[:500].cpu().numpy(), 0.9)
        assert np.array_equal(p.quantized_x[:500].cpu().numpy(), wq)
        assert np.array_equal(p.scales_x.reshape(-1)[:500].cpu().numpy(), ws)
        # (values of a few thousand next to values of a few: the roundings of the large ones are what separates two
        # correct fp16 results, so the tolerance follows the row's largest magnitude)
        ref = o.online_hadamard(x[:64].cpu().numpy(), force_fp32=fp32).astype(np.float64)
        err = np.abs(y[:64].cpu().numpy().astype(np.float64) - ref).max(axis=1)
        assert np.all(err <= 2e-3 * np.abs(ref).max(axis=1) + ATOL), (n, fp32)
    if n % 64 == 0:
        g = torch.Generator().manual_seed(n)
        w = torch.randint(0, 256, (96, n // 2), dtype=torch.uint8, generator=g).cuda()
        sw = (torch.rand(96, 1, generator=g) * 0.02 + 1e-3).half().cuda()
        for m in (1, 2, 70, 700):
            pm = quarot_amd.nn.Quantizer(0.9)(quarot_amd.nn.OnlineHadamard(n).cuda()(x[:m]))
            want_y = quarot_amd.linear_i4(pm.quantized_x, pm.scales_x, w, sw)
            got_y = quarot_amd.quantized_linear(x[:m], w, sw, None, None, 1, 0.9)
            assert torch.equal(got_y.view(torch.int16), want_y.view(torch.int16)), m


@pytest.mark.parametrize("n", [11008, 8960, 6912, 13824, 5120, 4608, 17920])
def test_fused_hadamard_quantize_lean_kernel_rows_of_every_kind(n):
    """Without the copy of the transformed rows the m = 64 widths (and m = 128 behind a table of order 36 .. 60 or
    108: the 13B widths 13824 and 5120; 4608 = 36 x 128 has hadK rows in only part of a wave's tile) take a kernel of their own (results of
    the hadK stage kept in registers, the previous row quantised between the next row's matrix
    instructions, every workgroup walking several rows): more rows than workgroups, and rows holding an
    infinity, a NaN, only zeros, huge and tiny values (the quantiser's slow path) next to ordinary ones.
    Codes and scales must equal those of the kernel that also returns the rows, whose codes are checked
    against the oracle on exactly those rows."""
    rows = 1500
    x = synth_x(rows, n, seed=n + 7)
    x[3, 17] = np.inf
    x[700, 5] = np.nan
    x[701] = 0
    x[1499] = 0
    x[1200, 9] = 60000.0
    x[44] *= F16(1e-4)
    x[0, :] = 0
    xg = gpu(x)
    mod = quarot_amd.nn.OnlineHadamardQuantizer(n, input_clip_ratio=0.9).cuda()
    p = mod(xg)
    p2, y = quarot_amd.hadamard_quantize(xg, mod.had_rem_dim, mod.rem_dim, 0.9, return_transformed=True)
    assert torch.equal(p.quantized_x, p2.quantized_x)
    assert np.array_equal(bits(p.scales_x.cpu().numpy()), bits(p2.scales_x.cpu().numpy()))
    with np.errstate(all="ignore"):
        wq, ws = o.quantizer(y.cpu().numpy(), 0.9)
    assert np.array_equal(p.quantized_x.cpu().numpy(), wq)
    got_s = p.scales_x.cpu().numpy().reshape(-1)
    nan = np.isnan(ws)                                             # (a NaN scale may carry any payload bits)
    assert np.array_equal(np.isnan(got_s), nan) and np.array_equal(bits(got_s[~nan]), bits(ws[~nan]))
    one = mod(xg[5:6])                                             # a single row: the first turn is also the last
    assert torch.equal(one.quantized_x, p.quantized_x[5:6])


@pytest.mark.parametrize("n", [11008, 8960, 6912, 8192])
@pytest.mark.parametrize("clip", [1.0, 0.9])
def test_fused_hadamard_quantize_lean_kernel_in_fp32_precision(n, clip):
    """force_fp32=True without the copy of the transformed rows: the lean m = 64 kernel with T kept as fp16 hi + lo planes
    (tables of order 108 .. 172 staged through LDS from their fp32 form; 8192 = 128 x 64 with the generated Sylvester
    outer factor).  Same rows of every kind as above; codes and scales must equal those of the kernels that also
    return the rows (same arithmetic in the same order), whose codes are checked against the oracle on those rows,
    and the rows against the oracle's fp32 transform."""
    rows = 1100
    x = synth_x(rows, n, seed=n + 11)
    x[3, 17] = np.inf
    x[700, 5] = np.nan
    x[701] = 0
    x[1099] = 0
    x[900, 9] = 60000.0
    x[44] *= F16(1e-4)
    x[0, :] = 0
    xg = gpu(x)
    mod = quarot_amd.nn.OnlineHadamardQuantizer(n, force_fp32=True, input_clip_ratio=clip).cuda()
    p = mod(xg)
    p2, y = quarot_amd.hadamard_quantize(xg, mod.had_rem_dim, mod.rem_dim, clip, force_fp32=True, return_transformed=True)
    assert torch.equal(p.quantized_x, p2.quantized_x)
    assert np.array_equal(bits(p.scales_x.cpu().numpy()), bits(p2.scales_x.cpu().numpy()))
    with np.errstate(all="ignore"):
        wq, ws = o.quantizer(y.cpu().numpy(), clip)
    assert np.array_equal(p.quantized_x.cpu().numpy(), wq)
    got_s = p.scales_x.cpu().numpy().reshape(-1)
    nan = np.isnan(ws)
    assert np.array_equal(np.isnan(got_s), nan) and np.array_equal(bits(got_s[~nan]), bits(ws[~nan]))
    fin = np.isfinite(x.astype(np.float32)).all(axis=1)
    sample = np.flatnonzero(fin)[::97]
    with np.errstate(all="ignore"):
        assert close(y.cpu().numpy()[sample], o.online_hadamard(x[sample], force_fp32=True))
    one = mod(xg[5:6])
    assert torch.equal(one.quantized_x, p.quantized_x[5:6])


def sign_words(table):
    """uint32 [K][ceil(K / 32)]: bit j of word w of row r set where table[r][32 w + j] is -1 (include/quarot_hip.h)."""
    k = table.shape[0]
    padded = np.zeros((k, (k + 31) // 32 * 32), dtype=bool)
    padded[:, :k] = np.asarray(table) < 0
    return np.packbits(padded, axis=1, bitorder="little").view(np.uint32)


@pytest.mark.parametrize("n", [6912, 8960, 9984, 11008])
@pytest.mark.parametrize("fp32", [False, True])
def test_fused_hadamard_quantize_with_the_table_as_sign_words(n, fp32):
    """QR_HADK_SIGNS through the C entry points: hadK passed as packed sign bits gives the codes and scales of the call
    that passes the table, bit for bit (orders 108, 140, 156, 172 behind FWHT-64; both precisions; rows of every
    kind), also through the one-call chain; shapes outside the lean kernel and calls that want the transformed rows
    are refused with QR_E_UNSUPPORTED before anything is written."""
    from quarot_amd.functional import hadamard as fh
    table, K = fh.get_hadK(n)
    rows = 700
    x = synth_x(rows, n, seed=n + 31)
    x[3, 17] = np.inf
    x[5, 5] = np.nan
    x[7] = 0
    xg = gpu(x)
    L, st = _lib.lib(), torch.cuda.current_stream().cuda_stream
    mode = _lib.QR_DTYPE_F32 if fp32 else _lib.QR_DTYPE_F16
    tab = gpu(np.asarray(table, dtype=np.float32 if fp32 else F16))
    sw = gpu(sign_words(np.asarray(table)).view(np.uint8))
    scale = fh.had_scale(n)
    out = {}
    for name, ptr, md in (("table", tab, mode), ("signs", sw, mode | _lib.QR_HADK_SIGNS)):
        q = torch.full((rows, n // 2), 0x5A, dtype=torch.uint8, device="cuda:0")
        s = torch.zeros(rows, dtype=torch.float16, device="cuda:0")
        rc = L.qr_hadamard_quantize_f16_i4(xg.data_ptr(), rows, n, K, ptr.data_ptr(), md, scale, 0.9, q.data_ptr(), s.data_ptr(), None, st)
        assert rc == 0, (name, rc)
        out[name] = (q, s)
    assert torch.equal(out["signs"][0], out["table"][0])
    assert np.array_equal(bits(out["signs"][1].cpu().numpy()), bits(out["table"][1].cpu().numpy()))
    # refused, nothing written: the transformed rows wanted; a width of another kernel family
    q = torch.full((rows, n // 2), 0x5A, dtype=torch.uint8, device="cuda:0")
    s = torch.zeros(rows, dtype=torch.float16, device="cuda:0")
    y = torch.zeros(rows, n, dtype=torch.float16, device="cuda:0")
    rc = L.qr_hadamard_quantize_f16_i4(xg.data_ptr(), rows, n, K, sw.data_ptr(), mode | _lib.QR_HADK_SIGNS, scale, 0.9, q.data_ptr(),
                                       s.data_ptr(), y.data_ptr(), st)
    assert rc == _lib.QR_E_UNSUPPORTED and bool((q == 0x5A).all()) and not bool(y.any())
    t28, k28 = fh.get_hadK(28672)
    x28 = gpu(synth_x(4, 28672, seed=1))
    q28 = torch.full((4, 14336), 0x5A, dtype=torch.uint8, device="cuda:0")
    sw28 = gpu(sign_words(np.asarray(t28)).view(np.uint8))
    rc = L.qr_hadamard_quantize_f16_i4(x28.data_ptr(), 4, 28672, k28, sw28.data_ptr(), mode | _lib.QR_HADK_SIGNS, fh.had_scale(28672), 1.0,
                                       q28.data_ptr(), s.data_ptr(), None, st)
    assert rc == _lib.QR_E_UNSUPPORTED and bool((q28 == 0x5A).all())


def test_sign_words_follow_the_table_object():
    """The Python layer packs a table's sign words once and reuses them while that table object is unchanged: a table
    written to in place is packed again (the results follow it), a table with entries other than +-1 is never packed
    (the call passes the table), and either way the results equal those of the call that returns the transformed rows,
    which always passes the table."""
    n = 11008
    x = gpu(synth_x(300, n, seed=5))
    mod = quarot_amd.nn.OnlineHadamardQuantizer(n, input_clip_ratio=1.0).cuda()
    def both():
        p = quarot_amd.hadamard_quantize(x, mod.had_rem_dim, mod.rem_dim, 1.0)
        p2, _ = quarot_amd.hadamard_quantize(x, mod.had_rem_dim, mod.rem_dim, 1.0, return_transformed=True)
        assert torch.equal(p.quantized_x, p2.quantized_x) and torch.equal(p.scales_x, p2.scales_x)
        return p.quantized_x.clone()
    first = both()
    assert quarot_amd._SIGNS[id(mod.had_rem_dim)][2] is not None              # packed
    assert torch.equal(both(), first)
    mod.had_rem_dim[5].neg_()                                                 # in place: another +-1 table
    second = both()
    assert not torch.equal(second, first)
    mod.had_rem_dim[5].neg_()
    assert torch.equal(both(), first)
    mod.had_rem_dim[0, 0] = 0.5                                               # no longer +-1: never packed
    third = both()
    assert quarot_amd._SIGNS[id(mod.had_rem_dim)][2] is None and not torch.equal(third, first)


@pytest.mark.parametrize("shape", [(5, 64), (9, 4096), (7, 5120), (3, 8192), (4, 11008), (2, 32768), (6, 24), (3, 100)])
@pytest.mark.parametrize("clip", [1.0, 0.9])
def test_fused_rmsnorm_quantize(shape, clip):
    """RMSNorm + Quantizer in one kernel.  The normalised rows (returned on request) must agree with
    the oracle to the stated floating-point tolerance -- only the order of the fp32 sum of squares
    differs, so almost every element is identical -- and the codes and scales must equal the oracle
    quantiser applied to the kernel's OWN normalised rows, bit for bit."""
    rows, cols = shape
    x = gpu(synth_x(rows, cols, seed=cols + 3))
    mod = quarot_amd.nn.RMSNormQuantizer(cols, eps=1e-5, input_clip_ratio=clip)
    p = mod(x)
    staged_y = quarot_amd.nn.RMSNorm(cols, eps=1e-5)(x)
    staged = quarot_amd.nn.Quantizer(clip)(staged_y)
    want_y = o.rmsnorm(x.cpu().numpy(), cols, 1e-5)
    if cols % 8 == 0:
        p2, y = quarot_amd.rmsnorm_quantize(x, cols, 1e-5, clip, return_normalized=True)
        assert torch.equal(p.quantized_x, p2.quantized_x) and torch.equal(p.scales_x, p2.scales_x)
        yk = y.cpu().numpy()
        assert close(yk, want_y) and np.mean(yk == want_y) > 0.999
        wq, ws = o.quantizer(yk, clip)
        assert np.array_equal(p.quantized_x.cpu().numpy(), wq)
        assert np.array_equal(p.scales_x.cpu().numpy().reshape(-1), ws)
        assert float((y == staged_y).float().mean()) > 0.999
    assert p.quantized_x.shape == staged.quantized_x.shape and p.scales_x.shape == staged.scales_x.shape
    assert float((p.quantized_x == staged.quantized_x).float().mean()) > 0.995
    assert close(staged_y.cpu().numpy(), want_y)


def test_fused_rmsnorm_quantize_full_size_and_errors():
    """Benchmark-size input (2048 x 4096) on strided rows; mean_dim different from the width;
    argument errors of the C entry point."""
    x = gpu(synth_x(2048, 4096, seed=5))
    p, y = quarot_amd.rmsnorm_quantize(x, 4096, 1e-5, 1.0, return_normalized=True)
    rows = slice(None, None, 129)
    want_y = o.rmsnorm(x[rows].cpu().numpy(), 4096, 1e-5)
    assert close(y[rows].cpu().numpy(), want_y)
    wq, ws = o.quantizer(y[rows].cpu().numpy(), 1.0)
    assert np.array_equal(p.quantized_x[rows].cpu().numpy(), wq)
    assert np.array_equal(p.scales_x.view(-1)[rows].cpu().numpy(), ws)
    assert torch.allclose(y.float().pow(2).mean(-1), torch.ones(2048, device=y.device), rtol=2e-3)
    p4, y4 = quarot_amd.rmsnorm_quantize(x[:8], 1024, 1e-5, 1.0, return_normalized=True)
    assert close(y4.cpu().numpy(), o.rmsnorm(x[:8].cpu().numpy(), 1024, 1e-5))
    L = _lib.lib()
    q = torch.empty(8, 2048, dtype=torch.uint8, device=x.device)
    s = torch.empty(8, dtype=torch.float16, device=x.device)
    st = torch.cuda.current_stream().cuda_stream
    assert L.qr_rmsnorm_quantize_f16_i4(x.data_ptr(), 8, 4092, 4092, 1e-5, 1.0, q.data_ptr(), s.data_ptr(), None, st) == _lib.lib().qr_rmsnorm_quantize_f16_i4(x.data_ptr(), 8, 40000, 40000, 1e-5, 1.0, q.data_ptr(), s.data_ptr(), None, st) < 0
    assert L.qr_rmsnorm_quantize_f16_i4(x.data_ptr() + 2, 8, 4096, 4096, 1e-5, 1.0, q.data_ptr(), s.data_ptr(), None, st) == -4
    assert L.qr_rmsnorm_quantize_f16_i4(x.data_ptr(), 0, 4096, 4096, 1e-5, 1.0, q.data_ptr(), s.data_ptr(), None, st) == 0
    assert L.qr_rmsnorm_quantize_f16_i4(None, 8, 4096, 4096, 1e-5, 1.0, q.data_ptr(), s.data_ptr(), None, st) < 0


@pytest.mark.parametrize("heads,rows,clip", [(32, 37, 1.0), (64, 19, 0.9), (16, 64, 1.0), (32, 1, 1.0)])
def test_fused_heads_hadamard_quantize(heads, rows, clip):
    """Hadamard across attention heads + Quantizer in one kernel (the chain in front of o_proj).  The
    transformed rows (returned on request) against the oracle to the floating-point tolerance (the
    sums are formed in a different order, so nearly every element is identical), codes and scales
    equal to the oracle quantiser applied to the kernel's OWN rows bit for bit, and the module
    against the three separate steps of the reference's model code."""
    x = gpu(synth_x(rows, heads * 128, seed=heads + rows)).view(rows, heads, 128)
    mod = quarot_amd.nn.HeadsHadamardQuantizer(heads, input_clip_ratio=clip)
    p = mod(x)
    p2, y = quarot_amd.heads_hadamard_quantize(x, heads, clip, return_transformed=True)
    assert torch.equal(p.quantized_x, p2.quantized_x) and torch.equal(p.scales_x, p2.scales_x)
    assert p.quantized_x.shape == (rows, heads * 64) and y.shape == (rows, heads * 128)
    yk = y.cpu().numpy()
    want_y = o.heads_hadamard(x.cpu().numpy(), heads)
    assert close(yk, want_y) and np.mean(yk == want_y) > 0.995
    wq, ws = o.quantizer(yk, clip)
    assert np.array_equal(p.quantized_x.cpu().numpy(), wq)
    assert np.array_equal(p.scales_x.cpu().numpy().reshape(-1), ws)
    # the reference's own sequence: transform on the transposed view, transpose back, reshape, quantise
    had = quarot_amd.nn.OnlineHadamard(heads)
    staged_y = had(x.transpose(-1, -2)).transpose(-1, -2).reshape(rows, heads * 128).contiguous()
    assert close(staged_y.cpu().numpy(), want_y)
    staged = quarot_amd.nn.Quantizer(clip)(staged_y)
    assert p.scales_x.shape == staged.scales_x.shape
    assert float((p.quantized_x == staged.quantized_x).float().mean()) > 0.99


@pytest.mark.parametrize("heads", [32, 64, 40])
def test_fused_heads_hadamard_quantize_infinite_nan_zero_huge_and_tiny_rows(heads):
    """Rows holding an infinity, a NaN, only zeros, a value near the fp16 maximum, and values near the
    subnormal range: codes and scales of both kernel forms must still equal the oracle quantiser applied
    to the kernel's own transformed rows, bit for bit (the quantiser's slow paths)."""
    rng = np.random.default_rng(3)
    x = rng.standard_normal((6, heads, 128)).astype(F16)
    x[1, 3, 5] = np.inf
    x[2, 0, 0] = np.nan
    x[3] = 0
    x[4, 7, 9] = 60000.0
    x[5] *= F16(1e-4)
    mod = quarot_amd.nn.HeadsHadamardQuantizer(heads).cuda()
    p, y = quarot_amd.heads_hadamard_quantize(gpu(x), heads, 1.0, return_transformed=True, hadK=mod.had.had_rem_dim)
    with np.errstate(all="ignore"):
        wq, ws = o.quantizer(y.cpu().numpy(), 1.0)
    assert np.array_equal(p.quantized_x.cpu().numpy(), wq)
    assert np.array_equal(bits(p.scales_x.cpu().numpy().reshape(-1)), bits(ws))


def test_fused_heads_hadamard_quantize_full_size_fallback_and_errors():
    """Prefill-size input ([2, 1024, 32, 128]) checked on strided rows and through norm preservation;
    shapes the fused kernel does not take go through the separate steps; argument errors of the C
    entry point."""
    x = gpu(synth_x(2048, 4096, seed=9)).view(2, 1024, 32, 128)
    p, y = quarot_amd.heads_hadamard_quantize(x, 32, 1.0, return_transformed=True)
    assert p.quantized_x.shape == (2, 1024, 2048) and p.scales_x.shape == (2, 1, 1024)
    y2 = y.view(2048, 4096)
    rows = slice(None, None, 131)
    xs = x.view(2048, 32, 128)[rows].cpu().numpy()
    assert close(y2[rows].cpu().numpy(), o.heads_hadamard(xs, 32))
    wq, ws = o.quantizer(y2[rows].cpu().numpy(), 1.0)
    assert np.array_equal(p.quantized_x.view(2048, -1)[rows].cpu().numpy(), wq)
    assert np.array_equal(p.scales_x.reshape(-1)[rows].cpu().numpy(), ws)
    assert torch.allclose(y2.float().norm(dim=1), x.view(2048, 4096).float().norm(dim=1), rtol=2e-3)
    # 8 heads of 64: the module runs the separate steps
    xs = gpu(synth_x(5, 512, seed=3)).view(5, 8, 64)
    pf = quarot_amd.nn.HeadsHadamardQuantizer(8)(xs)
    yf = o.heads_hadamard(xs.cpu().numpy(), 8)
    wq, _ = o.quantizer(yf, 1.0)
    assert pf.quantized_x.shape == (5, 256) and np.mean(pf.quantized_x.cpu().numpy() == wq) > 0.99
    L = _lib.lib()
    xf = x.view(2048, 4096)
    q = torch.empty(8, 2048, dtype=torch.uint8, device=x.device)
    s = torch.empty(8, dtype=torch.float16, device=x.device)
    st = torch.cuda.current_stream().cuda_stream
    assert L.qr_heads_hadamard_quantize_f16_i4(xf.data_ptr(), 8, 8, 64, None, 1.0, q.data_ptr(), s.data_ptr(), None, st) < 0
    assert L.qr_heads_hadamard_quantize_f16_i4(xf.data_ptr(), 8, 40, 128, None, 1.0, q.data_ptr(), s.data_ptr(), None, st) < 0
    assert L.qr_heads_hadamard_quantize_f16_i4(xf.data_ptr() + 2, 8, 32, 128, None, 1.0, q.data_ptr(), s.data_ptr(), None, st) == -4
    assert L.qr_heads_hadamard_quantize_f16_i4(xf.data_ptr(), 0, 32, 128, None, 1.0, q.data_ptr(), s.data_ptr(), None, st) == 0
    assert L.qr_heads_hadamard_quantize_f16_i4(None, 8, 32, 128, None, 1.0, q.data_ptr(), s.data_ptr(), None, st) < 0
    with pytest.raises(RuntimeError):
        quarot_amd.heads_hadamard_quantize(xf, 32)


def test_hadamard_full_size_properties():
    """Benchmark-size rows (2048 x 11008 and 2048 x 4096): norm preservation, linearity in a row
    scaling by 2 (exact in floating point), power-of-two transform is an involution."""
    for n in (11008, 4096):
        x = gpu(synth_x(2048, n, seed=0))
        had = quarot_amd.nn.OnlineHadamard(n).cuda()
        y = had(x)
        nx, ny = x.float().norm(dim=1), y.float().norm(dim=1)
        assert torch.allclose(nx, ny, rtol=2e-3)
        # doubling the input doubles the output, except where an fp16 subnormal or a rounding boundary
        # is crossed (then by one fp16 ulp)
        y2 = had(x * 2)
        assert float((y2 == y * 2).float().mean()) > 0.999
        assert torch.allclose(y2.float(), 2 * y.float(), rtol=1e-3, atol=1e-4)
        sub = o.online_hadamard(x[::257].cpu().numpy())
        assert close(y[::257].cpu().numpy(), sub)
    x = gpu(synth_x(512, 4096, seed=2, outliers=False))
    had = quarot_amd.nn.OnlineHadamard(4096).cuda()
    assert torch.allclose(had(had(x)).float(), x.float(), atol=4e-3, rtol=4e-3)


def test_hadamard_in_place_and_leading_dims():
    n = 1024
    x = gpu(synth_x(12, n, seed=9)).view(3, 4, n)
    y = quarot_amd.functional.hadamard.hadamard_transform(x, scale=1 / 32)
    assert y.shape == (3, 4, n)
    flat = x.clone().view(12, n)
    rc = _lib.lib().qr_hadamard(flat.data_ptr(), flat.data_ptr(), 12, n, 1, None, 0, 1 / 32,
                                torch.cuda.current_stream().cuda_stream)
    assert rc == 0 and torch.equal(flat.view(3, 4, n), y)


# ------------------------------------------------------------------------------ KV cache

@pytest.mark.parametrize("dim", [16, 64, 128, 256])
@pytest.mark.parametrize("hadamard", [False, True])
def test_kv_quant_dequant_bit_exact(dim, hadamard):
    rng = np.random.default_rng(dim)
    v = 1500
    x = rng.standard_normal((v, dim))
    x[rng.random((v, dim)) < 0.005] *= 15
    x[3], x[4] = 0.5, 0.0                                          # constant vectors: range clamps to fp16(1e-5)
    x = x.astype(F16).reshape(3, 500, dim)
    q, s, z = kv.asym_quantize_and_pack_i4(gpu(x), hadamard=hadamard)
    assert q.shape == (3, 500, dim // 2) and s.shape == (3, 500, 1) and z.shape == (3, 500, 1)
    xin = x
    if hadamard:        # codes are judged on the kernel's own Hadamard output (same arithmetic as matmul_had_cuda)
        xh = kv.matmul_had_cuda(gpu(x), torch.float16)
        assert close(xh.cpu().numpy(), o.kv_hadamard(x))
        xin = xh.cpu().numpy()
    wq, ws, wz = o.kv_asym_quant(xin)
    assert np.array_equal(q.cpu().numpy(), wq)
    assert np.array_equal(bits(s.cpu().numpy()), bits(ws)) and np.array_equal(bits(z.cpu().numpy()), bits(wz))
    y = kv.unpack_i4_and_asym_dequantize(q, s, z)
    assert np.array_equal(bits(y.cpu().numpy()), bits(o.kv_asym_dequant(wq, ws, wz)))
    err = (y.float() - gpu(xin).float()).abs()
    # half a step plus the fp16 roundings of x + zero, q * scale and the final subtraction
    assert bool((err <= s.float() / 2 + 0.004 * (15 * s.float() + z.float().abs()) + 1e-3).all())


@pytest.mark.parametrize("dim", [64, 128])
@pytest.mark.parametrize("hadamard", [False, True])
def test_kv_tiny_ranges_and_sums_too_large_for_fp16(dim, hadamard):
    """The corners of the quantiser's lean path: ranges so small that the scale is a subnormal fp16 number (its
    rounding error then reaches several per cent and the largest quotient passes 15.5: the clamp decides), ranges
    at the 1e-5 floor, and -- behind the Hadamard -- finite vectors whose transform overflows fp16 in SOME outputs
    only (all elements 60000: the first output is 128 * 60000 / sqrt(128) = inf, every other one 0).  Mixed with
    ordinary vectors in the same waves; codes, scales and zeros against the oracle bit for bit."""
    rng = np.random.default_rng(dim + hadamard)
    v = 640
    x = rng.standard_normal((v, dim)).astype(np.float64)
    for i in range(0, 200):                                  # ranges from 5e-6 to 2e-3 around various offsets
        span = 5e-6 * (400.0 ** (i / 199.0))
        base = (0.0, 0.01, -0.3, 1.0)[i % 4]
        x[i] = base + span * rng.random(dim)
        x[i, 0], x[i, 1] = base, base + span
    if hadamard:                                             # (transformed ranges: scaled so that the outputs are tiny)
        x[200:260] = rng.standard_normal((60, dim)) * (10.0 ** rng.uniform(-5.5, -2.5, (60, 1)))
        x[300] = 60000.0
        x[301] = -60000.0
        x[302] = 60000.0 * np.where(np.arange(dim) % 2 == 0, 1.0, -1.0)
        x[303, :] = 0.0
        x[303, :4] = 65504.0
    x = x.astype(F16)
    q, s, z = kv.asym_quantize_and_pack_i4(gpu(x), hadamard=hadamard)
    xin = x
    if hadamard:
        xin = kv.matmul_had_cuda(gpu(x), torch.float16).cpu().numpy()
        with np.errstate(over="ignore", invalid="ignore"):
            assert close(xin[:300], o.kv_hadamard(x[:300]))
        assert np.isinf(xin[300]).sum() == 1 and np.isinf(xin[301]).sum() == 1 and np.isinf(xin[302]).sum() == 1
    with np.errstate(over="ignore", invalid="ignore", divide="ignore"):
        wq, ws, wz = o.kv_asym_quant(xin)
    assert np.array_equal(q.cpu().numpy(), wq)
    assert np.array_equal(bits(s.cpu().numpy()), bits(ws)) and np.array_equal(bits(z.cpu().numpy()), bits(wz))
    assert (wq[:200] >> 4).max() == 15 and (wq[:200] & 15).min() == 0


@pytest.mark.parametrize("dim", [16, 64, 128, 256])
def test_kv_sign_of_a_zero_minimum_does_not_depend_on_where_the_zeros_stand(dim):
    """`zero` = -min carries the sign of the minimum when that is a zero.  A vector that holds -0.0 and +0.0 must give
    the same `zero` in every kernel, wherever its zeros stand: the minimum is -0.0 if the vector holds one (zero =
    +0.0) and +0.0 otherwise (zero = -0.0, as the reference's -min gives for a vector without negative zeros).  The
    fused Hadamard + quantiser and the quantiser on the transformed vectors agree bit for bit on inputs whose
    transform is full of zeros of both signs."""
    from quarot_amd.transformers import kv_cache as kvc
    g = torch.Generator().manual_seed(dim)
    vecs = 4096
    x = torch.rand(vecs, dim, generator=g)                                     # >= 0
    z = torch.rand(vecs, dim, generator=g)
    x = torch.where(z < 0.3, torch.zeros(()), x)
    x = torch.where(z < 0.15, -torch.zeros(()), x)                             # both zeros, in random places
    x[::4] = x[::4].abs()                                                      # every fourth vector: +0.0 only
    x[1::8] = x[1::8] + 0.5                                                    # and some without a zero at all
    x = x.half().cuda()
    has_neg0 = ((x == 0) & torch.signbit(x)).any(dim=1)
    min0 = x.amin(dim=1) == 0
    assert bool((has_neg0 & min0).any()) and bool((~has_neg0 & min0).any()) and bool((~min0).any())
    for xin in (x, x.flip(1).contiguous()):                                    # the same values in the opposite order
        q, s, zero = kvc.asym_quantize_and_pack_i4(xin)
        zb = zero.view(-1).view(torch.int16)
        assert bool((zb[min0 & has_neg0] == 0).all())                          # +0.0
        assert bool((zb[min0 & ~has_neg0] == -32768).all())                    # -0.0
        wq, ws, wz = o.kv_asym_quant(xin.cpu().numpy())
        assert np.array_equal(q.cpu().numpy(), wq) and np.array_equal(s.cpu().numpy(), ws) and np.array_equal(zero.cpu().numpy(), wz)
        plain = ~has_neg0.cpu().numpy()                                        # (no tie between zeros: the oracle's bits too)
        assert np.array_equal(bits(zero.cpu().numpy())[plain], bits(wz)[plain])
    if dim == 128:
        # one subnormal entry per vector: every transformed value is a sum too small for fp16, -0.0 or +0.0 by the
        # signs of that entry's Hadamard column; constant vectors: one large value and exact (+0.0) zeros
        t = torch.zeros(vecs, dim)
        t[torch.arange(vecs), torch.randint(0, dim, (vecs,), generator=g)] = 6e-8
        t[::2] = -t[::2]
        t[::5] = 0.75
        t = t.half().cuda()
        y = kvc.matmul_had_cuda(t, torch.float16)
        q1, s1, z1 = kvc.asym_quantize_and_pack_i4(t, hadamard=True)
        q2, s2, z2 = kvc.asym_quantize_and_pack_i4(y)
        assert torch.equal(q1, q2) and torch.equal(s1.view(torch.int16), s2.view(torch.int16))
        assert torch.equal(z1.view(torch.int16), z2.view(torch.int16))
        mins0 = y.amin(dim=1) == 0
        neg0 = ((y == 0) & torch.signbit(y)).any(dim=1)
        assert bool((mins0 & neg0).any()) and bool((mins0 & ~neg0).any())
        zb = z1.view(-1).view(torch.int16)
        assert bool((zb[mins0 & neg0] == 0).all()) and bool((zb[mins0 & ~neg0] == -32768).all())


def test_kv_vectors_with_infinities_take_the_ieee_path():
    """An infinite element makes range and scale infinite: every finite element then gets code 0 and
    inf / inf (NaN) converts to 0, as round/clamp/cast give in the reference; neighbouring finite
    vectors in the same wave are unaffected."""
    rng = np.random.default_rng(7)
    x = rng.standard_normal((64, 128)).astype(F16)
    x[5, 17] = np.inf
    x[9, 3] = -np.inf
    q, s, z = kv.asym_quantize_and_pack_i4(gpu(x), hadamard=False)
    q, s, z = q.cpu().numpy(), s.cpu().numpy(), z.cpu().numpy()
    assert np.isposinf(s[5, 0]) and np.all(q[5] == 0) and z[5, 0] == -x[5][np.isfinite(x[5])].min()
    assert np.isposinf(s[9, 0]) and np.isposinf(z[9, 0])
    keep = [i for i in range(64) if i not in (5, 9)]
    wq, ws, wz = o.kv_asym_quant(x[keep])
    assert np.array_equal(q[keep], wq) and np.array_equal(bits(s[keep]), bits(ws)) and np.array_equal(bits(z[keep]), bits(wz))


@pytest.mark.parametrize("dim,hadamard", [(128, False), (64, False), (64, True), (16, False), (256, True), (128, True)])
def test_kv_vector_with_nan_gets_nan_scale_and_zero(dim, hadamard):
    """torch.amax / torch.amin propagate a NaN (kv_cache.py:13-14): the vector's scale and zero are NaN
    and its codes 0 (NaN converts to 0), wherever in the vector the NaN sits; the other vectors of the
    same wave keep the oracle's codes."""
    rng = np.random.default_rng(dim)
    x = rng.standard_normal((70, dim)).astype(F16)
    where = {3: 0, 20: dim - 1, 41: dim // 2 + 1, 69: 9}
    for vec, el in where.items():
        x[vec, el] = np.nan
    x[50, 2] = np.inf                                              # an infinity next to them still takes the IEEE path
    q, s, z = kv.asym_quantize_and_pack_i4(gpu(x), hadamard=hadamard)
    q, s, z = q.cpu().numpy(), s.cpu().numpy(), z.cpu().numpy()
    for vec in where:
        assert np.isnan(s[vec, 0]) and np.isnan(z[vec, 0]) and not q[vec].any(), vec
    keep = [i for i in range(70) if i not in where and i != 50]
    xin = kv.matmul_had_cuda(gpu(x), torch.float16).cpu().numpy() if hadamard else x
    wq, ws, wz = o.kv_asym_quant(xin[keep])
    assert np.array_equal(q[keep], wq) and np.array_equal(bits(s[keep]), bits(ws)) and np.array_equal(bits(z[keep]), bits(wz))
    assert np.isposinf(s[50, 0])


def test_empty_and_leading_dimensions_through_the_python_interface():
    """Zero rows are legal everywhere (nothing is launched, shapes follow the non-empty case); leading
    dimensions are flattened and restored as the reference's wrappers do."""
    e = torch.empty(0, 4096, dtype=torch.float16, device=dev())
    q, s = quarot_amd.quantize_rows(e)
    assert q.shape == (0, 2048) and s.numel() == 0
    assert quarot_amd.nn.OnlineHadamard(4096).cuda()(e).shape == (0, 4096)
    assert quarot_amd.nn.OnlineHadamardQuantizer(11008).cuda()(e.new_empty(0, 11008)).quantized_x.shape == (0, 5504)
    assert quarot_amd.nn.RMSNormQuantizer(4096)(e).quantized_x.shape == (0, 2048)
    w = torch.randint(0, 255, (64, 2048), dtype=torch.uint8, device=dev())
    sw = torch.rand(64, 1, device=dev()).half()
    assert quarot_amd.linear_i4(w.new_empty(0, 2048), sw.new_empty(0), w, sw).shape == (0, 64)
    assert quarot_amd.matmul(w.new_empty(0, 2048), w).shape == (0, 64)
    qk, sk, zk = kv.asym_quantize_and_pack_i4(e.new_empty(0, 8, 128), hadamard=True)
    assert qk.shape == (0, 8, 64) and sk.shape == (0, 8, 1) and zk.shape == (0, 8, 1)
    x3 = gpu(synth_x(10, 4096, seed=3)).view(2, 5, 4096)
    p = quarot_amd.nn.Quantizer()(x3)
    assert p.quantized_x.shape == (2, 5, 2048) and p.scales_x.shape == (2, 1, 5)      # the reference's unsqueeze(1) quirk
    lin = quarot_amd.nn.Linear4bit(4096, 64).half().cuda()
    lin.weight_scales.fill_(0.01)
    assert lin(p).shape == (2, 5, 64)
    with pytest.raises(RuntimeError, match="contiguous"):
        quarot_amd.quantize_rows(gpu(synth_x(8, 8192, seed=1))[:, ::2])
    with pytest.raises(RuntimeError, match="GPU tensor"):
        quarot_amd.quantize_rows(torch.zeros(8, 64, dtype=torch.float16))


def test_decode_step_replays_from_a_hip_graph():
    """A decode step (fused Hadamard+quantise, then the decode GEMM) captured into a HIP graph: every
    replay, with fresh inputs copied into the static buffer and eager work plus synchronisation between
    the replays, must equal the eager result bit for bit.  The library launches on the stream it is
    given and allocates nothing, so capture needs no special path."""
    k, n = 5120, 1024                                   # had_40 x FWHT(128), decode-size GEMM
    w, sw = synth_w(n, k, seed=11)
    lin = quarot_amd.nn.Linear4bit(k, n).half().cuda()
    lin.weight.copy_(gpu(w)); lin.weight_scales.copy_(gpu(sw))
    front = quarot_amd.nn.OnlineHadamardQuantizer(k).cuda()
    xs = [gpu(synth_x(8, k, seed=20 + i)) for i in range(4)]
    static_x = xs[0].clone()
    for _ in range(2):                                  # warm-up outside capture (launch attributes are cached here)
        lin(front(static_x))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = lin(front(static_x))
    for i, x in enumerate(xs):
        eager = lin(front(x))                           # eager work between replays
        torch.cuda.synchronize()
        static_x.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, eager), f"replay {i}"
        p = front(x)
        wq, ws = o.quantizer(quarot_amd.nn.OnlineHadamard(k).cuda()(x).cpu().numpy())
        assert np.array_equal(p.quantized_x.cpu().numpy(), wq)


@pytest.mark.parametrize("k,m,had", [(12288, 1, True), (28672, 1, True), (20480, 2, True), (4096, 1, False), (8192, 2, False)])
def test_one_launch_decode_steps_replay_from_a_hip_graph(k, m, had):
    """The decode steps that are ONE kernel (one token behind a 1024-point Hadamard factor; one or two tokens behind the
    plain quantiser) captured into a HIP graph: every replay, with fresh inputs copied into the static buffer and eager
    work plus synchronisation in between, equals the eager two-launch chain bit for bit."""
    n = 2048
    w, sw = synth_w(n, k, seed=12)
    gw, gsw = gpu(w), gpu(sw)
    hadK, K = (quarot_amd.functional.hadamard.get_hadK(k) if had else (None, 0))
    if hadK is not None:
        hadK = hadK.to(dev()).half()
    xs = [gpu(synth_x(m, k, seed=30 + i, outliers=i % 2 == 0)) for i in range(4)]
    static_x = xs[0].clone()
    step = lambda x: quarot_amd.quantized_linear(x, gw, gsw, None, hadK, K)

    def chain(x):
        if had:
            p = quarot_amd.hadamard_quantize(x, hadK, K)
            return quarot_amd.linear_i4(p.quantized_x, p.scales_x, gw, gsw, None)
        q, s = quarot_amd.quantize_rows(x, 1.0)
        return quarot_amd.linear_i4(q, s, gw, gsw, None)

    for _ in range(2):
        step(static_x)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = step(static_x)
    for i, x in enumerate(xs):
        eager = chain(x)
        torch.cuda.synchronize()
        static_x.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, eager), f"replay {i}"


def test_kv_hadamard_128_blocks_tails_and_infinities():
    """Head dimension 128 with the Hadamard runs on the matrix cores, 32 vectors per wave step: vector
    counts around the block size, equality of the fused codes with the quantiser applied to the plain
    transform of the same kernel, and an infinite input (every output of that vector is +-inf: scale
    and zero infinite, all codes 0) that must not disturb its neighbours."""
    rng = np.random.default_rng(128)
    for vecs in (1, 31, 32, 33, 95, 257, 4100):
        x = rng.standard_normal((vecs, 128)).astype(F16)
        q, s, z = kv.asym_quantize_and_pack_i4(gpu(x), hadamard=True)
        xh = kv.matmul_had_cuda(gpu(x), torch.float16).cpu().numpy()
        assert close(xh, o.kv_hadamard(x))
        wq, ws, wz = o.kv_asym_quant(xh)
        assert np.array_equal(q.cpu().numpy(), wq)
        assert np.array_equal(bits(s.cpu().numpy()), bits(ws)) and np.array_equal(bits(z.cpu().numpy()), bits(wz))
    x = rng.standard_normal((70, 128)).astype(F16)
    x[40, 9] = np.inf
    q, s, z = kv.asym_quantize_and_pack_i4(gpu(x), hadamard=True)
    xh = kv.matmul_had_cuda(gpu(x), torch.float16).cpu().numpy()
    q, s, z = q.cpu().numpy(), s.cpu().numpy(), z.cpu().numpy()
    assert np.all(np.isinf(xh[40])) and np.isposinf(s[40, 0]) and np.isposinf(z[40, 0]) and np.all(q[40] == 0)
    keep = [i for i in range(70) if i != 40]
    wq, ws, wz = o.kv_asym_quant(xh[keep])
    assert np.array_equal(q[keep], wq) and np.array_equal(bits(s[keep]), bits(ws)) and np.array_equal(bits(z[keep]), bits(wz))
    # in place, as qr_hadamard allows
    t = gpu(x[:50].copy())
    rc = _lib.lib().qr_hadamard(t.data_ptr(), t.data_ptr(), 50, 128, 1, None, 0, 1.0 / np.sqrt(128.0),
                                torch.cuda.current_stream().cuda_stream)
    assert rc == 0 and np.array_equal(bits(t.cpu().numpy()), bits(xh[:50]))


def test_kv_full_size_round_trip():
    """The benchmark tensor [32, 4096, 8, 128]: codes in range, extremes hit, error bound, and a
    strided sample against the oracle."""
    g = torch.Generator().manual_seed(4)
    x = torch.randn(32, 4096, 8, 128, generator=g)
    mask = torch.rand(x.shape, generator=torch.Generator().manual_seed(5)) < 0.005
    x[mask] *= 15
    x = x.half()
    xd = x.to(dev())
    q, s, z = kv.asym_quantize_and_pack_i4(xd)
    y = kv.unpack_i4_and_asym_dequantize(q, s, z)
    assert bool(((y.float() - xd.float()).abs() <= s.float() / 2 + 0.004 * (15 * s.float() + z.float().abs()) + 1e-3).all())
    lo, hi = q & 0xF, q >> 4
    assert int(torch.minimum(lo.amin(-1), hi.amin(-1)).max()) == 0 and int(torch.maximum(lo.amax(-1), hi.amax(-1)).min()) == 15
    sub = x[::7, ::211].numpy()
    wq, ws, wz = o.kv_asym_quant(sub)
    assert np.array_equal(q[::7, ::211].cpu().numpy(), wq) and np.array_equal(bits(s[::7, ::211].cpu().numpy()), bits(ws))


# ------------------------------------------------------------------------------ benchmark-size configs

def check_rows_against_oracle(y, a, sa, w, sw, rows):
    want = o.linear4bit(a[rows], sa[rows], w, sw)
    assert np.array_equal(bits(y[rows].cpu().numpy()), bits(want))


def test_config_down_proj_2048x11008x4096_end_to_end():
    """Config 2 at full size: fused Hadamard+quantise then fused GEMM+dequant.  Codes are checked
    against the oracle quantiser on the kernel's Hadamard output for every row; the linear output
    is checked bit-exactly on a strided sample of rows (all 4096 columns)."""
    m, k, n = 2048, 11008, 4096
    x = gpu(synth_x(m, k, seed=0))
    w, sw = synth_w(n, k, seed=1)
    fused = quarot_amd.nn.OnlineHadamardQuantizer(k).cuda()
    p, y_h = quarot_amd.hadamard_quantize(x, fused.had_rem_dim, fused.rem_dim, return_transformed=True)
    wq, ws = o.quantizer(y_h.cpu().numpy())
    assert np.array_equal(p.quantized_x.cpu().numpy(), wq) and np.array_equal(p.scales_x.cpu().numpy().reshape(-1), ws)
    rows = np.arange(0, m, 37)
    assert close(y_h[rows].cpu().numpy(), o.online_hadamard(x[rows].cpu().numpy()))
    lin = quarot_amd.nn.Linear4bit(k, n).half().cuda()
    lin.weight.copy_(gpu(w))
    lin.weight_scales.copy_(gpu(sw))
    y = lin(p)
    check_rows_against_oracle(y, wq, ws, w, sw.reshape(-1), rows)


@pytest.mark.parametrize("m,k,n", [(32768, 4096, 4096), (8192, 4096, 12288), (4096, 11008, 4096)])
def test_prefill_shapes_sampled_rows(m, k, n):
    rng = np.random.default_rng(m + n)
    a = rng.integers(0, 256, (m, k // 2), dtype=np.uint8)
    w = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    sa = (np.abs(rng.standard_normal(m)) * 0.2).astype(F16)
    sw = (np.abs(rng.standard_normal(n)) * 0.01).astype(F16)
    y = quarot_amd.linear_i4(gpu(a), gpu(sa), gpu(w), gpu(sw))
    rows = np.concatenate([np.arange(0, m, 509), [m - 1]])
    check_rows_against_oracle(y, a, sa, w, sw, rows)
    c = quarot_amd.matmul(gpu(a), gpu(w))
    assert np.array_equal(c[rows].cpu().numpy(), o.int4_matmul(a[rows], w))


@pytest.mark.parametrize("m", [1, 8, 32, 64])
@pytest.mark.parametrize("k,n", [(8192, 57344), (28672, 8192)])
def test_decode_shapes_bit_exact(m, k, n):
    rng = np.random.default_rng(m + n)
    a = rng.integers(0, 256, (m, k // 2), dtype=np.uint8)
    w = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    sa = (np.abs(rng.standard_normal(m)) * 0.2).astype(F16)
    sw = (np.abs(rng.standard_normal(n)) * 0.01).astype(F16)
    y = quarot_amd.linear_i4(gpu(a), gpu(sa), gpu(w), gpu(sw))
    cols = np.arange(0, n, 3)
    want = o.linear4bit(a, sa, w[cols], sw[cols])
    assert np.array_equal(bits(y[:, cols].cpu().numpy()), bits(want))


@pytest.mark.parametrize("m,k,n", [(40, 28672, 8192), (53, 28672, 8192), (64, 28672, 8192), (48, 16384, 8192), (64, 16384, 8160),
                                   (40, 28608, 8192), (64, 8192, 8192), (39, 28672, 8192)])
def test_decode_many_tokens_against_a_narrow_weight_with_and_without_scratch(m, k, n):
    """40..64 tokens against a weight with few rows and a long K (70B down_proj): with scratch from the caller the
    shared-token kernel runs with K sliced across workgroups and a second kernel adds the slices' int32 slabs; without
    it the barrier-free kernel runs.  Both bit-exact against the oracle and each other -- whole and ragged K stages,
    a last block of rows that is partial, and shapes just outside the rule (a shorter K, one token fewer), with and
    without bias."""
    rng = np.random.default_rng(m + n + k)
    a = rng.integers(0, 256, (m, k // 2), dtype=np.uint8)
    w = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    a[0, :], w[0, :] = 0x88, 0x88                                  # the largest possible sum: 64 k
    sa = (np.abs(rng.standard_normal(m)) * 0.2 + 0.01).astype(F16)
    sw = (np.abs(rng.standard_normal(n)) * 0.01 + 0.001).astype(F16)
    bias = rng.standard_normal(n).astype(F16)
    ga, gw, gsa, gsw, gb = gpu(a), gpu(w), gpu(sa), gpu(sw), gpu(bias)
    L, st = _lib.lib(), torch.cuda.current_stream().cuda_stream
    ws_bytes = L.qr_workspace_bytes(m, n, k)
    assert (ws_bytes > 0) == (k >= 16384 and m >= 40)
    cols = np.concatenate([np.arange(0, n, 7), [n - 1]])
    for b, nb in ((gb, bias), (None, None)):
        y = quarot_amd.linear_i4(ga, gsa, gw, gsw, b)              # passes the scratch the library asks for
        plain = torch.empty_like(y)
        _lib.check(L.qr_linear_i4_f16(ga.data_ptr(), gsa.data_ptr(), gw.data_ptr(), gsw.data_ptr(),
                                      0 if b is None else b.data_ptr(), m, n, k, plain.data_ptr(), st))
        assert torch.equal(y, plain)
        want = o.linear4bit(a, sa, w[cols], sw[cols], None if nb is None else nb[cols])
        assert np.array_equal(bits(y[:, cols].cpu().numpy()), bits(want))


def test_linear4bit_sequential_is_one_call_with_the_same_results_and_state_dict():
    """Linear4bitSequential against torch.nn.Sequential of the same modules: identical output bits
    (the same two kernels run), identical state-dict keys, and the oracle on a small case; chains
    and inputs it does not recognise run module by module."""
    rng = np.random.default_rng(77)
    nn_ = quarot_amd.nn

    def make(k, n, bias, had, clip=1.0, fp32=False):
        lin = nn_.Linear4bit(k, n, bias=bias).half().cuda()
        lin.weight.copy_(gpu(rng.integers(0, 256, (n, k // 2), dtype=np.uint8)))
        lin.weight_scales.copy_(gpu((np.abs(rng.standard_normal((n, 1))) * 0.01 + 0.001).astype(F16)))
        if bias:
            lin.bias.copy_(gpu(rng.standard_normal(n).astype(F16)))
        front = ([nn_.OnlineHadamard(k, force_fp32=fp32).cuda()] if had else []) + [nn_.Quantizer(clip)]
        return torch.nn.Sequential(*front, lin), nn_.Linear4bitSequential(*front, lin)

    for (m, k, n, bias, had, clip, fp32) in [(37, 11008, 256, True, True, 0.9, False), (1, 28672, 512, False, True, 1.0, False),
                                             (5, 4096, 512, False, False, 1.0, False), (64, 4096, 128, True, True, 1.0, True),
                                             (200, 8192, 320, False, False, 0.95, False)]:
        ref, fused = make(k, n, bias, had, clip, fp32)
        x = gpu(synth_x(m, k, seed=m + k))
        assert torch.equal(fused(x), ref(x)), (m, k, n)
        assert list(fused.state_dict().keys()) == list(ref.state_dict().keys())
    ref, fused = make(4096, 256, True, False)
    x3 = gpu(synth_x(6, 4096, seed=1)).view(2, 3, 4096)
    y3 = fused(x3)
    assert y3.shape == (2, 3, 256) and torch.equal(y3, ref(x3))
    lin = fused[1]
    wq, ws = o.quantizer(x3.view(6, 4096).cpu().numpy())
    want = o.linear4bit(wq, ws, lin.weight.cpu().numpy(), lin.weight_scales.cpu().numpy().reshape(-1), lin.bias.cpu().numpy())
    assert np.array_equal(bits(y3.view(6, 256).cpu().numpy()), bits(want))
    # not one of the two chains, or not a contiguous fp16 tensor: module by module
    plain = nn_.Linear4bitSequential(nn_.Quantizer())
    p = plain(x3.view(6, 4096))
    assert isinstance(p, quarot_amd.PackedQuantizedTensor) and np.array_equal(p.quantized_x.cpu().numpy(), wq)
    xs = gpu(synth_x(6, 8192, seed=2))[:, ::2]
    with pytest.raises(RuntimeError):
        fused(xs)                                            # the reference's modules reject a strided input as well
    fused2 = nn_.Linear4bitSequential(*list(ref))
    fused2.load_state_dict(ref.state_dict())
    assert torch.equal(fused2(x3), y3)


def test_runs_on_the_current_stream():
    s = torch.cuda.Stream()
    x = gpu(synth_x(64, 4096, seed=8))
    with torch.cuda.stream(s):
        q, sc = quarot_amd.quantize_rows(x)
    s.synchronize()
    wq, ws = o.quantizer(x.cpu().numpy())
    assert np.array_equal(q.cpu().numpy(), wq)


@pytest.mark.parametrize("M", [1, 2])
@pytest.mark.parametrize("n", [12288, 20480, 28672])
def test_one_token_hadamard_linear_in_one_launch(n, M):
    """One or two tokens behind a 1024-point factor and a table of order 12, 20 or 28: qr_quantized_linear_f16 runs the front
    and the dot products in ONE kernel in which every workgroup transforms the rows itself.  Its output must carry the
    bits of the two-launch chain (same codes, same scale, same sums, same epilogue) for any number of weight rows
    (odd, one, more than one pass per wave), with and without bias, with a clip that lets the clamp act, and on rows
    holding zeros only, an infinity, a NaN or values that overflow the transform; the oracle's Quantizer + Linear4bit on
    the kernel's own transformed row (itself within rtol / atol 1e-3 of the oracle's transform) closes the chain."""
    rng = np.random.default_rng(n + M)
    hadK, K = quarot_amd.functional.hadamard.get_hadK(n)
    hadK = hadK.to(dev()).half()
    had = quarot_amd.nn.OnlineHadamard(n).to(dev())
    for N, bias, clip in [(1, False, 1.0), (2, True, 1.0), (130, False, 0.9), (4097, True, 1.0), (8192, False, 1.0),
                          (9001, True, 0.8), (20000, False, 1.0)]:
        w = gpu(rng.integers(0, 256, (N, n // 2), dtype=np.uint8))
        sw = gpu((np.abs(rng.standard_normal((N, 1))) * 0.01 + 0.001).astype(F16))
        b = gpu(rng.standard_normal(N).astype(F16)) if bias else None
        xn = synth_x(M, n, seed=N + n, outliers=N % 2 == 1)
        if M == 2:
            xn[1] *= F16(0.21)
        x = gpu(xn)
        got = quarot_amd.quantized_linear(x, w, sw, b, hadK, K, clip_ratio=clip)
        p = quarot_amd.hadamard_quantize(x, hadK, K, clip_ratio=clip)
        want = quarot_amd.linear_i4(p.quantized_x, p.scales_x, w, sw, b)
        assert got.shape == (M, N) and torch.equal(got, want), (n, N)
        if N <= 4097:
            xh = had(x).cpu().numpy()
            ref = o.online_hadamard(x.cpu().numpy()).astype(np.float64)
            assert np.all(np.abs(xh.astype(np.float64) - ref) <= ATOL + RTOL * np.abs(ref))
            xq, xs = o.quantizer(xh, clip)
            ref_y = o.linear4bit(xq, xs, w.cpu().numpy(), sw.cpu().numpy(), None if b is None else b.cpu().numpy())
            assert np.array_equal(bits(got.cpu().numpy()), bits(ref_y)), (n, N)
    N = 777
    w = gpu(rng.integers(0, 256, (N, n // 2), dtype=np.uint8))
    sw = gpu((np.abs(rng.standard_normal((N, 1))) * 0.01 + 0.001).astype(F16))
    for case in ("zeros", "inf", "nan", "overflow", "tiny"):
        x = synth_x(M, n, seed=5)
        if case == "zeros":
            x[M - 1] = 0
        elif case == "inf":
            x[M - 1, 5] = np.inf
        elif case == "nan":
            x[M - 1, n - 3] = np.nan
        elif case == "overflow":
            with np.errstate(over="ignore"):
                x = (x.astype(F32) * F32(900)).astype(F16)          # infinities where the product leaves the fp16 range
        else:
            x *= F16(1e-4)
        xg = gpu(x)
        got = quarot_amd.quantized_linear(xg, w, sw, None, hadK, K)
        p = quarot_amd.hadamard_quantize(xg, hadK, K)
        want = quarot_amd.linear_i4(p.quantized_x, p.scales_x, w, sw, None)
        assert np.array_equal(bits(got.cpu().numpy()), bits(want.cpu().numpy())), (n, case)


@pytest.mark.parametrize("M", [1, 2])
def test_one_or_two_tokens_quantizer_linear_in_one_launch(M):
    """One or two tokens through Quantizer -> Linear4bit: qr_quantized_linear_f16 (had_K = 0) runs ONE kernel in which
    every workgroup quantises the rows itself.  Bit for bit the two-launch chain, on rows of 64 to 32768 columns (short
    last segments of the weight rows included), one to 57344 weight rows, with bias, with a clip that lets the clamp
    act, on rows of zeros and rows holding an infinity or a NaN (with two tokens: in the second row, beside a finite
    first one); and the oracle's Quantizer + Linear4bit on the smaller shapes."""
    rng = np.random.default_rng(4 + M)
    for K, N, bias, clip in [(8192, 57344, False, 1.0), (4096, 4097, True, 1.0), (4096, 11008, False, 0.9), (5120, 300, True, 1.0),
                             (64, 7, False, 1.0), (11008, 4096, False, 1.0), (32768, 33, True, 1.0), (8192, 1, False, 1.0),
                             (2112, 513, True, 0.8), (16448, 64, False, 1.0)]:
        w = gpu(rng.integers(0, 256, (N, K // 2), dtype=np.uint8))
        sw = gpu((np.abs(rng.standard_normal((N, 1))) * 0.01 + 0.001).astype(F16))
        b = gpu(rng.standard_normal(N).astype(F16)) if bias else None
        for case in ("plain", "outliers", "zeros", "inf", "nan"):
            x = synth_x(M, K, seed=K + N, outliers=case == "outliers")
            if M == 2:
                x[1] *= F16(0.37)
            if case == "zeros":
                x[M - 1] = 0
            elif case == "inf":
                x[M - 1, K // 2] = -np.inf
            elif case == "nan":
                x[M - 1, K - 1] = np.nan
            xg = gpu(x)
            got = quarot_amd.quantized_linear(xg, w, sw, b, None, 0, clip_ratio=clip)
            q, s = quarot_amd.quantize_rows(xg, clip)
            want = quarot_amd.linear_i4(q, s, w, sw, b)
            assert got.shape == (M, N) and np.array_equal(bits(got.cpu().numpy()), bits(want.cpu().numpy())), (K, N, case)
            if N <= 4097 and case in ("plain", "outliers"):
                xq, xs = o.quantizer(x, clip)
                ref_y = o.linear4bit(xq, xs, w.cpu().numpy(), sw.cpu().numpy(), None if b is None else b.cpu().numpy())
                assert np.array_equal(bits(got.cpu().numpy()), bits(ref_y)), (K, N, case)
