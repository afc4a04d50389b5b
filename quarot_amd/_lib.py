"""ctypes binding of libquarot_hip.so (the C ABI declared in include/quarot_hip.h).

There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes
import pathlib

_PKG = pathlib.Path(__file__).resolve().parent
LIB_PATH = _PKG / "libquarot_hip.so"

_c = ctypes
_i64, _int, _f32, _ptr = _c.c_int64, _c.c_int, _c.c_float, _c.c_void_p

# name -> (restype, argtypes); mirrors include/quarot_hip.h one to one
SIGNATURES = {
    "qr_version": (_int, ()),
    "qr_strerror": (_c.c_char_p, (_int,)),
    "qr_hadamard": (_int, (_ptr, _ptr, _i64, _int, _int, _ptr, _int, _f32, _ptr)),
    "qr_sym_quant_f16_i4": (_int, (_ptr, _ptr, _i64, _i64, _ptr, _ptr)),
    "qr_quantize_rows_f16_i4": (_int, (_ptr, _f32, _i64, _i64, _ptr, _ptr, _ptr)),
    "qr_hadamard_quantize_f16_i4": (_int, (_ptr, _i64, _int, _int, _ptr, _int, _f32, _f32, _ptr, _ptr, _ptr, _ptr)),
    "qr_rmsnorm_quantize_f16_i4": (_int, (_ptr, _i64, _i64, _int, _f32, _f32, _ptr, _ptr, _ptr, _ptr)),
    "qr_heads_hadamard_quantize_f16_i4": (_int, (_ptr, _i64, _int, _int, _ptr, _f32, _ptr, _ptr, _ptr, _ptr)),
    "qr_matmul_i4_i32": (_int, (_ptr, _ptr, _i64, _i64, _i64, _ptr, _ptr)),
    "qr_sym_dequant_i32_f16": (_int, (_ptr, _ptr, _ptr, _i64, _i64, _ptr, _ptr)),
    "qr_linear_i4_f16": (_int, (_ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _ptr, _ptr)),
    "qr_workspace_bytes": (_c.c_size_t, (_i64, _i64, _i64)),
    "qr_quantized_linear_workspace_bytes": (_c.c_size_t, (_i64, _i64, _i64)),
    "qr_quantized_linear_f16": (_int, (_ptr, _i64, _i64, _int, _ptr, _int, _f32, _f32, _ptr, _ptr, _ptr, _i64, _ptr, _ptr,
                                       _c.c_size_t, _ptr)),
    "qr_linear_i4_f16_ws": (_int, (_ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _ptr, _ptr, _c.c_size_t, _ptr)),
    "qr_linear_i4_f16_static": (_int, (_ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _ptr, _ptr)),
    "qr_f6_bytes": (_c.c_size_t, (_i64, _i64)),
    "qr_convert_i4_f6": (_int, (_ptr, _i64, _i64, _ptr, _ptr)),
    "qr_linear_f6_f16": (_int, (_ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _ptr, _ptr)),
    "qr_kv_quant_f16_i4": (_int, (_ptr, _i64, _int, _int, _ptr, _ptr, _ptr, _ptr)),
    "qr_kv_dequant_i4_f16": (_int, (_ptr, _ptr, _ptr, _i64, _int, _ptr, _ptr)),
    "qr_kv_append_i4": (_int, (_ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _int, _int, _int, _int, _int,
                               _i64, _ptr)),
    "qr_kv_quant_append_f16_i4": (_int, (_ptr, _ptr, _i64, _ptr, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _int, _int, _int, _int,
                                         _int, _i64, _ptr)),
    "qr_batch_decode_workspace_bytes": (_c.c_size_t, (_i64, _int, _i64)),
    "qr_batch_decode_i4": (_int, (_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _int, _int, _int, _int, _int, _i64, _i64, _ptr,
                                  _c.c_size_t, _ptr)),
    "qr_batch_decode_qhad_i4": (_int, (_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _int, _int, _int, _int, _int, _i64, _i64, _ptr,
                                       _c.c_size_t, _ptr)),
    "qr_kv_quant_append_batch_decode_f16_i4": (_int, (_ptr, _ptr, _int, _ptr, _ptr, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _int,
                                                      _int, _int, _int, _int, _i64, _i64, _ptr, _c.c_size_t, _ptr)),
    "qr_kv_append_f16": (_int, (_ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _int, _int, _int, _int, _int,
                                _i64, _ptr)),
    "qr_batch_decode_f16": (_int, (_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _int, _int, _int, _int, _int, _i64, _ptr)),
    "qr_calib_mfma_i8": (_int, (_int, _int, _int, _ptr, _ptr)),
    "qr_calib_copy": (_int, (_ptr, _ptr, _i64, _ptr)),
}

QR_DTYPE_F16, QR_DTYPE_F32 = 0, 1
QR_HADK_SIGNS = 0x100          # or-ed into a `mode`: hadK is passed as sign words (include/quarot_hip.h)
QR_E_NULL, QR_E_SHAPE, QR_E_UNSUPPORTED = -1, -2, -3

_lib = None


def lib():
    """The loaded library (loads on first use).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m quarot_amd.build` "
                "(this package has no CPU or PyTorch fallback)")
        handle = ctypes.CDLL(str(LIB_PATH))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, list(args)
        _lib = handle
    return _lib


def check(code):
    """Raise RuntimeError with the library's message for a non-zero return code."""
    if code != 0:
        raise RuntimeError(f"libquarot_hip: {lib().qr_strerror(code).decode()} (code {code})")


def stream_ptr(device):
    """Raw handle of torch's current stream on `device` (the library launches there)."""
    import torch
    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if raw is not None and device.index is not None:
        return raw(device.index)                 # same value, without building a Stream object
    return torch.cuda.current_stream(device).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def on_device(device):
    """Context that makes `device` current for the launch; nothing to do (and nothing to pay) when
    it already is."""
    import torch
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(device)
