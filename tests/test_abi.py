"""The C ABI: the shared library loads and exports exactly what include/quarot_hip.h declares.
No kernel is launched here; argument errors are returned before any launch."""
import ctypes
import pathlib
import re

import pytest

from quarot_amd import _lib

ROOT = pathlib.Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "quarot_hip.h"


@pytest.fixture(scope="module")
def lib():
    if not _lib.LIB_PATH.exists():          # built beforehand normally; build only if nothing is there
        from quarot_amd import build
        build.build(verbose=False)
    return _lib.lib()


def declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(qr_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_expected_entry_points():
    syms = declared_symbols()
    for must in ("qr_hadamard", "qr_sym_quant_f16_i4", "qr_quantize_rows_f16_i4", "qr_hadamard_quantize_f16_i4",
                 "qr_matmul_i4_i32", "qr_sym_dequant_i32_f16", "qr_linear_i4_f16", "qr_kv_quant_f16_i4",
                 "qr_kv_dequant_i4_f16", "qr_version", "qr_strerror", "qr_rmsnorm_quantize_f16_i4", "qr_heads_hadamard_quantize_f16_i4", "qr_quantized_linear_workspace_bytes", "qr_quantized_linear_f16", "qr_kv_quant_append_batch_decode_f16_i4", "qr_kv_append_f16", "qr_batch_decode_f16",
                 "qr_workspace_bytes", "qr_linear_i4_f16_ws", "qr_linear_i4_f16_static", "qr_f6_bytes", "qr_convert_i4_f6",
                 "qr_linear_f6_f16"):
        assert must in syms


def test_library_exports_every_declared_symbol(lib):
    raw = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in declared_symbols():
        assert hasattr(raw, name), name
    assert sorted(_lib.SIGNATURES) == declared_symbols()


def test_version_and_error_text(lib):
    assert lib.qr_version() >= 100
    assert lib.qr_strerror(0) == b"success"
    for code in (-1, -2, -3, -4, -5, -6, -7):
        assert len(lib.qr_strerror(code)) > 5
    assert b"unknown" in lib.qr_strerror(-99)


def test_argument_errors_are_returned_before_any_launch(lib):
    one = ctypes.c_void_p(16)       # never dereferenced: every call below must fail validation first
    assert lib.qr_matmul_i4_i32(one, one, 4, 4, 100, one, None) == -2          # K % 64 != 0
    assert lib.qr_matmul_i4_i32(one, one, 4, 4, 1 << 18, one, None) == -2      # accumulator would overflow
    assert lib.qr_matmul_i4_i32(None, one, 4, 4, 64, one, None) == -1
    assert lib.qr_matmul_i4_i32(ctypes.c_void_p(8), one, 4, 4, 64, one, None) == -4
    assert lib.qr_matmul_i4_i32(one, one, 0, 4, 64, None, None) == 0           # empty: nothing to do
    assert lib.qr_matmul_i4_i32(one, one, -1, 4, 64, one, None) == -2
    assert lib.qr_linear_i4_f16(one, None, one, one, None, 4, 4, 64, one, None) == -1
    assert lib.qr_sym_quant_f16_i4(None, one, 3, 8, one, None) == -1
    assert lib.qr_sym_quant_f16_i4(one, one, 0, 8, one, None) == 0
    assert lib.qr_quantize_rows_f16_i4(one, 1.0, 3, 0, one, one, None) == -2   # max over an empty axis
    assert lib.qr_sym_dequant_i32_f16(one, one, None, 2, 2, one, None) == -1
    assert lib.qr_hadamard(one, one, 2, 100, 1, None, 0, 1.0, None) == -2      # not a power of two
    assert lib.qr_hadamard(one, one, 2, 172 * 3, 172, one, 0, 1.0, None) == -2
    assert lib.qr_hadamard(one, one, 2, 1 << 16, 1, None, 0, 1.0, None) == -3  # longer than one workgroup's LDS
    assert lib.qr_hadamard(one, one, 2, 64, 1, None, 7, 1.0, None) == -5
    assert lib.qr_hadamard(one, one, 2, 11008, 172, None, 0, 1.0, None) == -1  # hadK missing
    assert lib.qr_hadamard_quantize_f16_i4(one, 2, 64, 1, None, 0, 1.0, 1.0, None, one, None, None) == -1
    assert lib.qr_hadamard_quantize_f16_i4(one, 2, 64, 1, None, 0, 1.0, 1.0, ctypes.c_void_p(20), one, None, None) == -4  # codes: 8-byte aligned
    assert lib.qr_kv_quant_f16_i4(one, 4, 100, 0, one, one, one, None) == -3
    assert lib.qr_kv_quant_f16_i4(one, 4, 128, 3, one, one, one, None) == -5
    assert lib.qr_kv_dequant_i4_f16(one, one, one, 0, 128, one, None) == 0
    # the entry point with the built-in scratch buffer: a shape beyond the buffer is refused by size alone
    assert lib.qr_workspace_bytes(768, 3072, 65536) > (32 << 20)
    assert lib.qr_linear_i4_f16_static(one, one, one, one, None, 768, 3072, 65536, one, None) == -7
    assert lib.qr_linear_i4_f16_static(one, one, one, one, None, 128, 4096, 100, one, None) == -2


def test_workspace_query_needs_no_gpu(lib):
    """qr_workspace_bytes is pure host arithmetic: non-zero exactly for prompts of a few hundred tokens
    whose tiles would leave most CUs idle, a whole number of [M, N] int32 slabs."""
    assert lib.qr_workspace_bytes(2048, 4096, 11008) == 0          # enough tiles
    assert lib.qr_workspace_bytes(8, 8192, 28672) == 0             # decode batches use the decode kernel
    assert lib.qr_workspace_bytes(512, 11008, 4096) == 0           # short K: nothing to split
    for m, n, k in ((256, 4096, 11008), (128, 4096, 4096), (96, 8192, 8192), (256, 8192, 28672)):
        ws = lib.qr_workspace_bytes(m, n, k)
        assert ws > 0 and ws % (m * n * 4) == 0 and 2 <= ws // (m * n * 4) <= 16
    assert lib.qr_workspace_bytes(0, 4096, 4096) == 0 and lib.qr_workspace_bytes(256, 4096, 100) == 0
    one = ctypes.c_void_p(16)
    assert lib.qr_linear_i4_f16_ws(one, None, one, one, None, 4, 4, 64, one, None, 0, None) == -1
    assert lib.qr_linear_i4_f16_ws(one, one, one, one, None, 4, 4, 100, one, None, 0, None) == -2


def test_fp6_path_sizes_and_argument_errors_need_no_gpu(lib):
    """The FP6 matrix path: a converted operand is 6 bits per value; argument errors come back before any launch."""
    assert lib.qr_f6_bytes(2048, 11008) == 2048 * 11008 * 3 // 4
    assert lib.qr_f6_bytes(0, 4096) == 0 and lib.qr_f6_bytes(16, 100) == 0
    one = ctypes.c_void_p(16)
    assert lib.qr_convert_i4_f6(one, 4, 100, one, None) == -2                   # K % 64 != 0
    assert lib.qr_convert_i4_f6(None, 4, 64, one, None) == -1
    assert lib.qr_convert_i4_f6(ctypes.c_void_p(8), 4, 64, one, None) == -4
    assert lib.qr_convert_i4_f6(one, 0, 64, one, None) == 0
    assert lib.qr_linear_f6_f16(one, one, one, one, None, 4, 4, 100, one, None) == -2
    assert lib.qr_linear_f6_f16(one, None, one, one, None, 4, 4, 64, one, None) == -1
    assert lib.qr_linear_f6_f16(ctypes.c_void_p(8), one, one, one, None, 4, 4, 64, one, None) == -4
    assert lib.qr_linear_f6_f16(one, one, one, one, None, 1 << 20, 4, 8192, one, None) == -3   # operand beyond 32-bit offsets
    assert lib.qr_linear_f6_f16(one, one, one, one, None, 0, 4, 64, one, None) == 0


def test_quantized_linear_workspace_and_argument_errors_need_no_gpu(lib):
    """The single-call layer entry point: its workspace holds the codes (M K / 2 bytes), the scales
    (2 M bytes), each rounded up to 16 bytes, and the GEMM's own scratch; argument errors are
    reported before anything is launched."""
    assert lib.qr_quantized_linear_workspace_bytes(1, 8192, 28672) == 14336 + 16
    assert lib.qr_quantized_linear_workspace_bytes(2048, 4096, 11008) == 2048 * 5504 + 4096
    m, n, k = 256, 4096, 11008
    assert lib.qr_quantized_linear_workspace_bytes(m, n, k) == m * k // 2 + 512 + lib.qr_workspace_bytes(m, n, k)
    assert lib.qr_quantized_linear_workspace_bytes(0, n, k) == 0
    one = ctypes.c_void_p(16)
    args = (one, 4, 64, 0, None, 0, 1.0, 1.0, one, one, None, 4, one)
    assert lib.qr_quantized_linear_f16(*args, None, 0, None) == -6                 # no workspace
    assert lib.qr_quantized_linear_f16(*args, one, 100, None) == -6                # too small (needs 128 + 16)
    assert lib.qr_quantized_linear_f16(*args, ctypes.c_void_p(24), 4096, None) == -6   # misaligned
    assert lib.qr_quantized_linear_f16(one, 4, 100, 0, None, 0, 1.0, 1.0, one, one, None, 4, one, one, 4096, None) == -2
    assert lib.qr_quantized_linear_f16(None, 4, 64, 0, None, 0, 1.0, 1.0, one, one, None, 4, one, one, 4096, None) == -1
    assert lib.qr_quantized_linear_f16(one, 0, 64, 0, None, 0, 1.0, 1.0, one, one, None, 4, one, None, 0, None) == 0
    assert b"workspace" in lib.qr_strerror(-6)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _lib.lib()
