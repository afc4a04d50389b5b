"""The call that bench.py times, at bench size, under the oracle: LinearWorkload.step() -- one library call per
step (qr_quantized_linear_f16), decode weights rotating among their copies -- must equal the two-call chain
(front kernel, then linear_i4) bit for bit on every rotation, and the oracle's Quantizer + Linear4bit on sampled
rows and output columns (for the Hadamard workloads: applied to the kernel's own transformed rows, which are
themselves held to rtol / atol 1e-3 against the oracle's transform)."""
import numpy as np
import pytest
import torch

import bench
import quarot_amd
from oracle import quarot_oracle as o

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-3


def bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


@pytest.mark.parametrize("name", ["c1", "c2", "c2_fp32had", "c4m1", "c4m64", "c4g1", "c4g64"])
def test_bench_step_equals_the_two_call_chain_and_the_oracle(name):
    dev = torch.device("cuda:0")
    wl = bench.LinearWorkload(name, dev, on_gpu_data=True)
    assert wl.one_call
    if wl.decode:
        assert len(wl.copies) >= 3 and sum(c.numel() for c in wl.copies) >= 640 * 1024 * 1024
    # every rotation of the weight copies, and once around again
    p = wl.front(wl.x)
    want = quarot_amd.linear_i4(p.quantized_x, p.scales_x, wl.lin.weight, wl.lin.weight_scales, wl.lin.bias)
    for _ in range(len(wl.copies) + 1):
        got = wl.step()
        assert got.shape == (wl.m, wl.n) and got.dtype == torch.float16
        assert torch.equal(got, want)
    # the oracle on sampled rows x sampled output columns
    rng = np.random.default_rng(len(name) + wl.m)
    rows = sorted(set([0, wl.m - 1] + [int(v) for v in rng.integers(0, wl.m, 6)]))
    cols = sorted(set([0, wl.n - 1] + [int(v) for v in rng.integers(0, wl.n, 254)]))
    x = wl.x.reshape(wl.m, wl.k)[rows]
    if wl.front_kind in ("had", "had32"):
        had = quarot_amd.nn.OnlineHadamard(wl.k, force_fp32=wl.fp32_had).to(dev)
        xh = had(x).cpu().numpy()                                            # the kernel's own transformed rows
        ref = o.online_hadamard(x.cpu().numpy(), force_fp32=wl.fp32_had).astype(np.float64)
        assert np.all(np.abs(xh.astype(np.float64) - ref) <= ATOL + RTOL * np.abs(ref))
    else:
        xh = x.cpu().numpy()
    xq, xs = o.quantizer(xh)
    assert np.array_equal(p.quantized_x.reshape(wl.m, -1)[rows].cpu().numpy(), xq)
    assert np.array_equal(bits(p.scales_x.reshape(-1)[rows].cpu().numpy()), bits(xs))
    w = wl.lin.weight[cols].cpu().numpy()
    sw = wl.lin.weight_scales[cols].cpu().numpy()
    ref_y = o.linear4bit(xq, xs, w, sw, None)
    assert np.array_equal(bits(got[rows][:, cols].cpu().numpy()), bits(ref_y))
