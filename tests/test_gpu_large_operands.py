"""Operands of 4 GiB and more: the pipelined GEMM kernels address their operands through 32-bit buffer offsets, so
such shapes are routed to the kernels with 64-bit addressing (and Linear4bit's opt-in FP6 route must step aside).
Both routes, oracle on sampled rows and columns, bit-exact."""
import numpy as np
import pytest
import torch

import quarot_amd
from oracle import quarot_oracle as o

pytestmark = pytest.mark.gpu
F16 = np.float16


def bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


@pytest.mark.parametrize("m,n,k", [(70000, 256, 131008),      # activations' codes 4.6 GB: 192/256-row tiles step aside
                                   (128, 65600, 131008)])     # weights 4.3 GB: 128-row tiles step aside
def test_linear_with_an_operand_of_four_gib_and_more(m, n, k):
    assert max(m, n) * (k // 2) >= 1 << 32
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(m + n)
    a = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, device=dev, generator=g)
    lin = quarot_amd.nn.Linear4bit(k, n, bias=True).half().to(dev)
    lin.weight.copy_(torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=dev, generator=g))
    lin.weight_scales.copy_((torch.rand(n, 1, device=dev, generator=g) * 0.01 + 0.001).half())
    lin.bias.copy_(torch.randn(n, device=dev, generator=g).half())
    sa = (torch.rand(m, 1, device=dev, generator=g) * 0.2 + 0.01).half()
    # extreme rows at both ends: the largest possible sums, 64 k
    a[0].fill_(0x88)
    a[m - 1].fill_(0x88)
    lin.weight[0].fill_(0x88)
    lin.weight[n - 1].fill_(0x77)
    packed = quarot_amd.PackedQuantizedTensor(a, sa)
    y = lin(packed)
    assert y.shape == (m, n) and y.dtype == torch.float16
    lin.prefill_fp6, lin.fp6_min_rows = True, 64               # the FP6 route does not take operands this large
    y6 = lin(packed)
    assert not hasattr(lin, "_f6_cache") and torch.equal(y6, y)
    rng = np.random.default_rng(m)
    rows = sorted(set([0, m - 1] + [int(v) for v in rng.integers(0, m, 4)]))
    cols = sorted(set([0, n - 1] + [int(v) for v in rng.integers(0, n, 30)]))
    want = o.linear4bit(a[rows].cpu().numpy(), sa.view(-1)[rows].cpu().numpy(), lin.weight[cols].cpu().numpy(),
                        lin.weight_scales[cols].cpu().numpy(), lin.bias[cols].cpu().numpy())
    assert np.array_equal(bits(y[rows][:, cols].cpu().numpy()), bits(want))
    # int32 sums of the same shape through quarot.matmul
    c = quarot_amd.matmul(a, lin.weight)
    assert int(c[0, 0]) == 64 * k and int(c[m - 1, n - 1]) == -56 * k
    ref = o.int4_matmul(a[rows].cpu().numpy(), lin.weight[cols].cpu().numpy())
    assert np.array_equal(c[rows][:, cols].cpu().numpy(), ref)
