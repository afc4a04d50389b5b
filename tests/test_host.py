"""Host-side mirror of the reference interface: names, buffers, assertions, the torch-only
helpers.  Runs without a GPU."""
import numpy as np
import pytest
import torch

import quarot_amd
from oracle import quarot_oracle as o
from quarot_amd.functional import hadamard as fh
from quarot_amd.functional import quantization as fq


def test_public_names_match_reference_layout():
    for name in ("matmul", "sym_quant", "sym_dequant", "PackedQuantizedTensor"):
        assert hasattr(quarot_amd, name)
    for name in ("Linear4bit", "RMSNorm", "Quantizer", "OnlineHadamard"):
        assert hasattr(quarot_amd.nn, name)
    for name in ("pack_i4", "unpack_i4", "asym_quant_dequant", "sym_quant_dequant", "matmul_hadU_cuda",
                 "random_hadamard_matrix", "apply_exact_had_to_linear"):
        assert hasattr(quarot_amd.functional, name)
    for name in ("get_hadK", "matmul_hadU", "is_pow2", "get_had172", "get_had12"):
        assert hasattr(quarot_amd.functional.hadamard, name)


@pytest.mark.parametrize("n", [32, 64, 128, 4096, 8192, 11008, 28672, 13824, 5120, 6656, 17920, 14336, 12288, 72, 80, 20])
def test_get_hadK_matches_oracle(n):
    h, k = fh.get_hadK(n)
    ho, ko = o.get_hadK(n)
    assert k == ko
    if ho is None:
        assert h is None
    else:
        assert h.dtype == torch.float32 and np.array_equal(h.numpy(), ho)
        assert np.array_equal(fh.get_hadK(n, transpose=True)[0].numpy(), ho.T)


def test_get_hadK_asserts_like_reference():
    for n in (324, 100, 3 * 172):
        with pytest.raises(AssertionError):
            fh.get_hadK(n)


def test_pack_unpack_torch_matches_oracle():
    rng = np.random.default_rng(0)
    q = rng.integers(-8, 8, (9, 40))
    p = fq.pack_i4(torch.from_numpy(q))
    assert p.dtype == torch.uint8 and np.array_equal(p.numpy(), o.pack_i4(q))
    u = fq.unpack_i4(p)
    assert u.dtype == torch.int32 and np.array_equal(u.numpy(), q)
    b = torch.arange(256, dtype=torch.uint8).reshape(16, 16)
    assert torch.equal(fq.pack_i4(fq.unpack_i4(b)), b)
    with pytest.raises(AssertionError):
        fq.pack_i4(torch.tensor([[8, 0]]))
    with pytest.raises(AssertionError):
        fq.pack_i4(torch.tensor([[1, 0]], dtype=torch.uint8))
    with pytest.raises(AssertionError):
        fq.unpack_i4(torch.zeros(2, 2, dtype=torch.int8))


def test_torch_quant_primitives():
    x = torch.tensor([[0.26, -1.9, 0.74, 3.0]])
    s = torch.tensor([[0.5]])
    q, _ = fq.sym_quant(x, s, torch.tensor(7))
    assert q.tolist() == [[1.0, -4.0, 1.0, 6.0]]
    assert torch.allclose(fq.sym_quant_dequant(x, s, torch.tensor(7)), q * s)
    mn, mx = fq.get_minq_maxq(4, True)
    assert (int(mn), int(mx)) == (-8, 7)
    mn, mx = fq.get_minq_maxq(4, False)
    assert (int(mn), int(mx)) == (0, 15)
    assert fq.two_compl(torch.tensor([-1, 3]), 4).tolist() == [15, 3]


@pytest.mark.parametrize("n", [16, 64, 24, 344, 224])
def test_matmul_hadU_torch_matches_closed_form(n):
    g = torch.Generator().manual_seed(n)
    x = torch.randn(3, n, generator=g, dtype=torch.float64)
    got = fh.matmul_hadU(x).numpy()
    np.testing.assert_allclose(got, o.hadamard_closed_form(x.numpy()), rtol=2e-7, atol=1e-9)
    np.testing.assert_allclose(fh.matmul_hadUt(fh.matmul_hadU(x)).numpy(), x.numpy(), rtol=1e-6, atol=1e-6)


def test_random_hadamard_matrix_is_orthogonal():
    torch.manual_seed(0)
    q = fh.random_hadamard_matrix(48, "cpu")
    assert q.dtype == torch.float64
    np.testing.assert_allclose((q @ q.T).numpy(), np.eye(48), atol=1e-6)


def test_module_buffers_and_state_dict_keys():
    lin = quarot_amd.nn.Linear4bit(128, 64, bias=True)
    sd = lin.state_dict()
    assert set(sd) == {"weight", "weight_scales", "bias"}
    assert sd["weight"].shape == (64, 64) and sd["weight"].dtype == torch.uint8
    assert sd["weight_scales"].shape == (64, 1)
    assert sd["bias"].shape == (64,) and sd["bias"].dtype == torch.float16
    assert quarot_amd.nn.Linear4bit(128, 64).bias is None
    had = quarot_amd.nn.OnlineHadamard(11008)
    assert had.rem_dim == 172 and had.had_rem_dim.dtype == torch.float16 and "had_rem_dim" in had.state_dict()
    had32 = quarot_amd.nn.OnlineHadamard(28672, force_fp32=True)
    assert had32.rem_dim == 28 and had32.had_rem_dim.dtype == torch.float32
    assert quarot_amd.nn.OnlineHadamard(4096).had_rem_dim is None
    fused = quarot_amd.nn.OnlineHadamardQuantizer(11008)
    fused.load_state_dict(had.state_dict())


def test_reference_assertions_and_errors_without_gpu():
    a = torch.zeros(4, 24, dtype=torch.uint8)
    with pytest.raises(AssertionError, match="must be multiplication of 32"):
        quarot_amd.matmul(a, a)
    with pytest.raises(AssertionError):
        quarot_amd.sym_quant(torch.zeros(2, 8), torch.zeros(2, dtype=torch.float16))
    with pytest.raises(AssertionError):
        quarot_amd.sym_dequant(torch.zeros(2, 2), torch.zeros(2, dtype=torch.float16), torch.zeros(2, dtype=torch.float16))
    with pytest.raises(AssertionError):
        quarot_amd.nn.Linear4bit(64, 32)(torch.zeros(2, 64, dtype=torch.float16))
    # CPU tensors are rejected (torch::checkDeviceType in the reference), never silently computed
    b = torch.zeros(4, 32, dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="GPU"):
        quarot_amd.matmul(b, b)
    with pytest.raises(RuntimeError, match="GPU"):
        quarot_amd.sym_quant(torch.zeros(2, 8, dtype=torch.float16), torch.zeros(2, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="GPU"):
        quarot_amd.nn.Quantizer()(torch.zeros(2, 8, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="GPU"):
        quarot_amd.nn.OnlineHadamard(64)(torch.zeros(2, 64, dtype=torch.float16))


def test_rmsnorm_matches_formula():
    x = torch.randn(4, 32, dtype=torch.float16)
    y = quarot_amd.nn.RMSNorm(32)(x)
    xf = x.float()
    want = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).half()
    assert y.dtype == torch.float16 and torch.allclose(y.float(), want.float(), atol=1e-3)


def test_packed_tensor_carrier():
    p = quarot_amd.PackedQuantizedTensor(torch.zeros(3, 4, dtype=torch.uint8), torch.ones(3, 1, dtype=torch.float16))
    assert p.size() == (3, 4) and p.dtype == torch.uint8 and p.device.type == "cpu"
