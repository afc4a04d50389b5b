"""Benchmark configurations at their full sizes on the GPU: the four linear layers of a Llama-2-7B
decoder layer at 32768 tokens through the real module chains, and the K cache (Hadamard over the head
dimension + asymmetric int4) on [32, 4096, 8, 128].  Also the offline weight-side Hadamard helpers.

Bars: codes, scales, int32 accumulators and fp16 outputs BIT-EXACT against the oracle; Hadamard rows
within rtol 1e-3 / atol 1e-3."""
import numpy as np
import pytest
import torch

import quarot_amd
from oracle import quarot_oracle as o
from quarot_amd.transformers import kv_cache as kv

pytestmark = pytest.mark.gpu
F16, F32 = np.float16, np.float32
RTOL = ATOL = 1e-3
M3 = 32768


def gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


def bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


def close(got, want):
    g, w = got.astype(np.float64), want.astype(np.float64)
    return np.all(np.abs(g - w) <= ATOL + RTOL * np.abs(w))


def synth_x(m, k, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g)
    idx = torch.randperm(k, generator=g)[: -(-k // 100)]
    x[:, idx] *= 20
    return x.half()


def synth_w(n, k, seed):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(n, k, generator=g) * 0.02).half()
    s = (w.abs().amax(dim=1, keepdim=True) / 7).half()
    return w, s


def tile_sample_rows(m, block=128):
    """One row in EVERY block of `block` rows, at an in-block offset that walks through all residues
    (so every lane/wave position of a row tile is hit somewhere), plus the last three rows."""
    b = np.arange(m // block)
    rows = b * block + (b * 37 + 5) % block
    return np.unique(np.concatenate([rows, [m - 3, m - 2, m - 1]]))


def oracle_quantizer_all_rows(y_gpu, q_gpu, s_gpu, clip=1.0, chunk=4096):
    """Every row of the quantiser's output against the oracle, in chunks to bound host memory."""
    m = y_gpu.shape[0]
    for r0 in range(0, m, chunk):
        wq, ws = o.quantizer(y_gpu[r0:r0 + chunk].cpu().numpy(), clip)
        assert np.array_equal(q_gpu[r0:r0 + chunk].cpu().numpy(), wq), f"codes differ in rows {r0}..{r0 + chunk}"
        assert np.array_equal(bits(s_gpu.reshape(-1)[r0:r0 + chunk].cpu().numpy()), bits(ws)), f"scales differ from row {r0}"


def whole_output_equals_row_slices(y, p, lin, step=64):
    """The whole [32768, N] output against the same rows pushed through the library in slices of 64
    rows: those take the decode-shaped kernels, which the parity tests check against the oracle on
    their own.  Compared on the GPU, every element."""
    codes, scales = p.quantized_x, p.scales_x.reshape(-1)
    for r0 in range(0, codes.shape[0], step):
        part = quarot_amd.linear_i4(codes[r0:r0 + step], scales[r0:r0 + step], lin.weight, lin.weight_scales, lin.bias)
        assert torch.equal(part, y[r0:r0 + step]), f"rows {r0}..{r0 + step} differ from the sliced launch"


@pytest.fixture(scope="module")
def x4096():
    x = synth_x(M3, 4096, seed=0).cuda()
    p = quarot_amd.nn.Quantizer()(x)
    oracle_quantizer_all_rows(x, p.quantized_x, p.scales_x)              # all 32768 rows
    return x, p


@pytest.mark.parametrize("name,n,seed", [("qkv", 12288, 10), ("o", 4096, 11), ("gate_up", 22016, 12)])
def test_config3_linears_from_4096_at_32768_tokens(x4096, name, n, seed):
    """qkv 4096->12288, o 4096->4096 and gate_up 4096->22016 (86 column tiles, the last one ragged) at
    M = 32768 through Quantizer -> Linear4bit (e2e/quantized_llama/modeling_llama.py:40-44,99-115).
    fp16 outputs and int32 accumulators bit-exact against the oracle on a row of every 128-row block
    (all columns), and the whole output equal to the 64-row-slice launches."""
    x, p = x4096
    w, sw = synth_w(n, 4096, seed)
    base = torch.nn.Linear(4096, n, bias=False).half()
    base.weight.data = w
    lin = quarot_amd.nn.Linear4bit.from_float(base, weight_scales=sw).cuda()
    wq = lin.weight.cpu().numpy()
    assert np.array_equal(wq, o.weight_codes_from_float(w.numpy(), sw.numpy()))
    chain = torch.nn.Sequential(quarot_amd.nn.Quantizer(), lin)
    y = chain(x)
    assert y.shape == (M3, n) and y.dtype == torch.float16
    rows = tile_sample_rows(M3)
    xq, xs = p.quantized_x[rows].cpu().numpy(), p.scales_x.reshape(-1)[rows].cpu().numpy()
    acc = o.int4_matmul(xq, wq)
    assert np.array_equal(bits(y[rows].cpu().numpy()), bits(o.sym_dequant(acc, xs, sw.numpy())))
    c = quarot_amd.matmul(p.quantized_x, lin.weight)
    assert c.dtype == torch.int32 and np.array_equal(c[rows].cpu().numpy(), acc)
    whole_output_equals_row_slices(y, p, lin)
    # the accumulators of the whole output, on the GPU: dequantised by the staged call they give y again
    assert torch.equal(quarot_amd.sym_dequant(c, p.scales_x.reshape(-1), lin.weight_scales), y)
    seq = quarot_amd.nn.Linear4bitSequential(quarot_amd.nn.Quantizer(), lin)
    assert torch.equal(seq(x), y)


def test_config3_down_proj_with_online_hadamard_at_32768_tokens():
    """down 11008->4096 behind OnlineHadamard(11008) = FWHT(64) (x) had_172 at M = 32768: the fused
    Hadamard+quantise kernel's codes and scales against the oracle quantiser on its own transformed
    rows, EVERY row; transformed rows against the oracle's Hadamard on the tile sample; fp16 outputs and
    int32 accumulators bit-exact on the tile sample; whole output equal to the 64-row-slice launches."""
    k, n = 11008, 4096
    x = synth_x(M3, k, seed=0).cuda()
    w, sw = synth_w(n, k, 13)
    base = torch.nn.Linear(k, n, bias=False).half()
    base.weight.data = w
    lin = quarot_amd.nn.Linear4bit.from_float(base, weight_scales=sw).cuda()
    wq = lin.weight.cpu().numpy()
    front = quarot_amd.nn.OnlineHadamardQuantizer(k).cuda()
    p, y_h = quarot_amd.hadamard_quantize(x, front.had_rem_dim, front.rem_dim, return_transformed=True)
    oracle_quantizer_all_rows(y_h, p.quantized_x, p.scales_x)
    p_plain = front(x)                                                   # without the extra output: same codes
    assert torch.equal(p_plain.quantized_x, p.quantized_x) and torch.equal(p_plain.scales_x, p.scales_x)
    staged = quarot_amd.nn.OnlineHadamard(k).cuda()(x)                   # the reference's two-module form
    assert torch.equal(staged, y_h)
    rows = tile_sample_rows(M3)
    assert close(y_h[rows].cpu().numpy(), o.online_hadamard(x[rows].cpu().numpy()))
    nx, ny = x.float().norm(dim=1), y_h.float().norm(dim=1)
    assert torch.allclose(nx, ny, rtol=2e-3)
    del staged, x
    y = lin(p)
    xq, xs = p.quantized_x[rows].cpu().numpy(), p.scales_x.reshape(-1)[rows].cpu().numpy()
    acc = o.int4_matmul(xq, wq)
    assert np.array_equal(bits(y[rows].cpu().numpy()), bits(o.sym_dequant(acc, xs, sw.numpy())))
    c = quarot_amd.matmul(p.quantized_x, lin.weight)
    assert np.array_equal(c[rows].cpu().numpy(), acc)
    assert torch.equal(quarot_amd.sym_dequant(c, p.scales_x.reshape(-1), lin.weight_scales), y)
    whole_output_equals_row_slices(y, p, lin)


def test_config5_k_cache_with_hadamard_full_size():
    """K cache of config 5, [32, 4096, 8, 128] with 0.5 % outliers: the fused kernel (Hadamard over the
    head dimension on the matrix cores + asymmetric int4) against the oracle on a strided sample of
    vectors, EVERY vector against the plain quantiser applied to the plain transform (compared on the
    GPU), the error bound of the round trip and the extreme codes (kv_cache.py:10-33,188-198)."""
    g = torch.Generator().manual_seed(4)
    x = torch.randn(32, 4096, 8, 128, generator=g)
    mask = torch.rand(x.shape, generator=torch.Generator().manual_seed(5)) < 0.005
    x[mask] *= 15
    x = x.half()
    xd = x.cuda()
    q, s, z = kv.asym_quantize_and_pack_i4(xd, hadamard=True)
    assert q.shape == (32, 4096, 8, 64) and s.shape == z.shape == (32, 4096, 8, 1)
    xh = kv.matmul_had_cuda(xd, torch.float16)
    q2, s2, z2 = kv.asym_quantize_and_pack_i4(xh, hadamard=False)        # every vector, on the GPU
    assert torch.equal(q, q2) and torch.equal(s, s2) and torch.equal(z, z2)
    sub_x = x[::5, 3::157].numpy()                                       # 7 x 27 x 8 vectors from all over the tensor
    sub_h = xh[::5, 3::157].cpu().numpy()
    assert close(sub_h, o.kv_hadamard(sub_x))
    wq, ws, wz = o.kv_asym_quant(sub_h)
    assert np.array_equal(q[::5, 3::157].cpu().numpy(), wq)
    assert np.array_equal(bits(s[::5, 3::157].cpu().numpy()), bits(ws)) and np.array_equal(bits(z[::5, 3::157].cpu().numpy()), bits(wz))
    tail = (slice(31, 32), slice(4090, 4096))                            # the last vectors of the tensor
    wq, ws, wz = o.kv_asym_quant(xh[tail].cpu().numpy())
    assert np.array_equal(q[tail].cpu().numpy(), wq) and np.array_equal(bits(s[tail].cpu().numpy()), bits(ws))
    y = kv.unpack_i4_and_asym_dequantize(q, s, z)
    assert bool(((y.float() - xh.float()).abs() <= s.float() / 2 + 0.004 * (15 * s.float() + z.float().abs()) + 1e-3).all())
    lo, hi = q & 0xF, q >> 4
    assert int(torch.minimum(lo.amin(-1), hi.amin(-1)).max()) == 0 and int(torch.maximum(lo.amax(-1), hi.amax(-1)).min()) == 15
    assert torch.allclose(xh.float().norm(dim=-1), xd.float().norm(dim=-1), rtol=3e-3, atol=1e-2)


# ------------------------------------------------------------------------------ offline weight-side helpers

def _closed_form_matrix(n):
    hadk, k = o.get_hadK(n)
    hm = o.sylvester(n // k).astype(np.float64)
    return (hm if k == 1 else np.kron(hadk, hm)) / np.sqrt(np.float64(n))


@pytest.mark.parametrize("fin,fout", [(11008, 96), (4096, 200), (28672, 40), (13824, 24)])
def test_apply_exact_had_to_linear_input_side(fin, fout):
    """W <- W . H^T with H = kron(hadK, H_m) / sqrt(n) on the input side (functional/hadamard.py:109-125),
    fp32 on the GPU, stored back in W's dtype and device: against the float64 closed form."""
    g = torch.Generator().manual_seed(fin)
    lin = torch.nn.Linear(fin, fout, bias=False)
    lin.weight.data = torch.randn(fout, fin, generator=g) * 0.02
    w0 = lin.weight.data.double().numpy()
    quarot_amd.functional.apply_exact_had_to_linear(lin, had_dim=-1, output=False)
    assert lin.weight.dtype == torch.float32 and lin.weight.device.type == "cpu"
    want = w0 @ _closed_form_matrix(fin).T
    assert np.allclose(lin.weight.data.numpy(), want, rtol=1e-4, atol=2e-6)
    half = torch.nn.Linear(fin, fout, bias=False).half().cuda()
    half.weight.data = torch.from_numpy(w0).half().cuda()
    quarot_amd.functional.apply_exact_had_to_linear(half)
    assert half.weight.dtype == torch.float16 and half.weight.is_cuda
    want16 = torch.from_numpy(w0).half().double().numpy() @ _closed_form_matrix(fin).T
    assert close(half.weight.data.cpu().numpy(), want16)


@pytest.mark.parametrize("fin,fout", [(72, 11008), (130, 4096), (33, 5120)])
def test_apply_exact_had_to_linear_output_side(fin, fout):
    """W <- H . W on the output side (functional/hadamard.py:121-123: the transform of W^T's rows)."""
    g = torch.Generator().manual_seed(fout)
    lin = torch.nn.Linear(fin, fout, bias=False)
    lin.weight.data = torch.randn(fout, fin, generator=g) * 0.02
    w0 = lin.weight.data.double().numpy()
    quarot_amd.functional.apply_exact_had_to_linear(lin, had_dim=-1, output=True)
    want = _closed_form_matrix(fout) @ w0
    assert np.allclose(lin.weight.data.numpy(), want, rtol=1e-4, atol=2e-6)


def test_apply_exact_had_to_linear_per_head_output_and_errors():
    """had_dim = 128 on the output side: each block of 128 output features (one attention head of
    v_proj) is transformed on its own (functional/hadamard.py:127-134); the input side with had_dim is
    the reference's NotImplementedError; a had_dim that is no power of two its AssertionError."""
    fin, fout, hd = 96, 4096, 128
    lin = torch.nn.Linear(fin, fout, bias=False)
    lin.weight.data = torch.randn(fout, fin, generator=torch.Generator().manual_seed(1)) * 0.02
    w0 = lin.weight.data.double().numpy()
    quarot_amd.functional.apply_exact_had_to_linear(lin, had_dim=hd, output=True)
    h = o.sylvester(hd).astype(np.float64) / np.sqrt(hd)
    want = np.einsum("gh,bhi->bgi", h, w0.reshape(fout // hd, hd, fin)).reshape(fout, fin)
    assert np.allclose(lin.weight.data.numpy(), want, rtol=1e-4, atol=2e-6)
    with pytest.raises(NotImplementedError):
        quarot_amd.functional.apply_exact_had_to_linear(lin, had_dim=hd, output=False)
    with pytest.raises(AssertionError):
        quarot_amd.functional.apply_exact_had_to_linear(lin, had_dim=96, output=True)
    with pytest.raises(AssertionError):
        quarot_amd.functional.apply_exact_had_to_linear(torch.nn.Identity())


@pytest.mark.parametrize("n", [11008, 5120, 4096])
def test_matmul_hadUt_cuda_is_the_inverse_transform(n):
    """matmul_hadUt_cuda applies kron(hadK^T, H_m) / sqrt(n): the inverse of matmul_hadU_cuda (the
    matrix is orthogonal), and equal to the float64 closed form with the transposed table."""
    fh = quarot_amd.functional.hadamard
    hadk, k = fh.get_hadK(n)
    x = torch.randn(5, n, generator=torch.Generator().manual_seed(n)).cuda()
    hk = None if hadk is None else hadk.cuda()
    y = fh.matmul_hadU_cuda(x, hk, k)
    back = fh.matmul_hadUt_cuda(y, hk, k)
    assert torch.allclose(back, x, rtol=1e-4, atol=1e-5)
    yt = fh.matmul_hadUt_cuda(x, hk, k).cpu().numpy()
    assert np.allclose(yt, o.hadamard_closed_form(x.cpu().double().numpy(), transpose=True), rtol=1e-4, atol=1e-5)
    assert np.allclose(yt, fh.matmul_hadUt(x.cpu()).numpy(), rtol=1e-4, atol=1e-5)      # the torch butterfly statement


def test_random_hadamard_matrix_rotates_a_linear_exactly():
    """random_hadamard_matrix (functional/hadamard.py:85-90) is orthogonal in float64; rotating a
    layer's input side by Q and its input by Q leaves the product unchanged."""
    torch.manual_seed(3)
    qm = quarot_amd.functional.random_hadamard_matrix(344, "cuda")       # 172 * 2
    assert qm.dtype == torch.float64 and qm.is_cuda
    eye = torch.eye(344, dtype=torch.float64, device="cuda")
    assert torch.allclose(qm @ qm.T, eye, atol=1e-12)
    assert torch.allclose(qm.abs(), torch.full_like(qm, 1 / np.sqrt(344)), atol=1e-12)
