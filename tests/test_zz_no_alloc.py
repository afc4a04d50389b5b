"""The entry point that allocates nothing (qr_linear_i4_f16_static): through the C ABI, against
qr_linear_i4_f16_ws with a caller-provided workspace, bit for bit, on calls in a row that share the
library's built-in scratch buffer (the later ones with smaller inputs), plus the size limit."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import quarot_oracle as o
from quarot_amd import _lib

pytestmark = pytest.mark.gpu
F16 = np.float16


def gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


def operands(m, n, k, seed):
    rng = np.random.default_rng(seed)
    a = o.pack_i4(rng.integers(-8, 8, (m, k)))
    w = o.pack_i4(rng.integers(-8, 8, (n, k)))
    sa = (np.abs(rng.standard_normal(m)) * 0.2 + 0.01).astype(F16)
    sw = (np.abs(rng.standard_normal(n)) * 0.01 + 0.001).astype(F16)
    bias = rng.standard_normal(n).astype(F16)
    return a, w, sa, sw, bias


def run_both(L, m, n, k, seed, with_bias):
    a, w, sa, sw, bias = operands(m, n, k, seed)
    ga, gw, gsa, gsw, gb = gpu(a), gpu(w), gpu(sa), gpu(sw), gpu(bias)
    bptr = gb.data_ptr() if with_bias else None
    st = torch.cuda.current_stream().cuda_stream
    ws_bytes = L.qr_workspace_bytes(m, n, k)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=ga.device)
    y_ws = torch.full((m, n), float("nan"), dtype=torch.float16, device=ga.device)
    y_st = torch.full((m, n), float("nan"), dtype=torch.float16, device=ga.device)
    assert L.qr_linear_i4_f16_ws(ga.data_ptr(), gsa.data_ptr(), gw.data_ptr(), gsw.data_ptr(), bptr, m, n, k,
                                 y_ws.data_ptr(), ws.data_ptr() if ws_bytes else None, ws_bytes, st) == 0
    free_before = torch.cuda.mem_get_info()[0]
    rc = L.qr_linear_i4_f16_static(ga.data_ptr(), gsa.data_ptr(), gw.data_ptr(), gsw.data_ptr(), bptr, m, n, k,
                                   y_st.data_ptr(), st)
    assert rc == 0, L.qr_strerror(rc)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before          # the call took no device memory
    assert torch.equal(y_st, y_ws), (m, n, k)
    want = o.linear4bit(a, sa, w, sw, bias if with_bias else None)
    assert np.array_equal(y_st.cpu().numpy().view(np.uint16), want.view(np.uint16)), (m, n, k)
    return ws_bytes


def test_static_scratch_entry_point_matches_the_workspace_form_on_consecutive_calls():
    L = _lib.lib()
    # a split-K shape, then smaller ones that reuse (part of) the same scratch with its old contents,
    # then a shape that needs no scratch, then the first one again
    used = [run_both(L, 256, 4096, 11008, 1, False),
            run_both(L, 130, 520, 4160, 2, True),
            run_both(L, 96, 512, 8192, 3, False),
            run_both(L, 37, 300, 1024, 4, True),
            run_both(L, 2048, 4096, 512, 5, False),
            run_both(L, 256, 4096, 11008, 6, True)]
    assert used[0] > 0 and used[1] > 0 and used[2] > 0 and used[3] == 0 and used[4] == 0
    assert max(used) <= 32 << 20


def test_static_scratch_limit_and_argument_errors():
    L = _lib.lib()
    one = ctypes.c_void_p(256)
    big = None
    for shape in ((768, 3072, 65536), (192, 12288, 130944)):
        if L.qr_workspace_bytes(*shape) > (32 << 20):
            big = shape
            break
    assert big is not None
    assert L.qr_linear_i4_f16_static(one, one, one, one, None, *big, one, None) == -7     # nothing is launched
    assert b"scratch" in L.qr_strerror(-7)
    assert L.qr_linear_i4_f16_static(one, one, one, one, None, 128, 4096, 100, one, None) == -2
    assert L.qr_linear_i4_f16_static(one, None, one, one, None, 128, 4096, 4096, one, None) == -1
    assert L.qr_linear_i4_f16_static(one, one, one, one, None, 0, 4096, 4096, None, None) == 0
