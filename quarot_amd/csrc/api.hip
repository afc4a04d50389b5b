// Version and error text of libquarot_hip.so, and the entry point that chains the front kernel and
// the GEMM of one quantised linear layer.
#include "qr_common.h"

extern "C" int qr_version(void) { return 100; }

extern "C" const char* qr_strerror(int code) {
    switch (code) {
        case QR_OK: return "success";
        case QR_E_NULL: return "a required pointer is NULL";
        case QR_E_SHAPE: return "invalid size (negative, zero, too large, or violating a divisibility rule)";
        case QR_E_UNSUPPORTED: return "valid for the reference but not implemented by this build";
        case QR_E_ALIGN: return "pointer not aligned as required";
        case QR_E_DTYPE: return "unknown dtype or mode code";
        case QR_E_WORKSPACE: return "workspace missing, misaligned or too small";
        case QR_E_SCRATCH_LIMIT: return "the shape needs more scratch than the library's built-in buffer (QR_STATIC_SCRATCH_BYTES) holds";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error code";
}

namespace {
inline size_t align16(size_t v) { return (v + 15) & ~(size_t)15; }
}  // namespace

extern "C" size_t qr_quantized_linear_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    // (rows of 128: room for the transformed rows, which the fused front of that length writes and reads back)
    return align16((size_t)M * (size_t)((K + 1) / 2)) + align16((size_t)M * 2) + (K == 128 ? align16((size_t)M * 256) : 0) +
           qr_workspace_bytes(M, N, K);
}

extern "C" int qr_quantized_linear_f16(const void* x, int64_t M, int64_t K, int had_K, const void* hadK, int mode,
                                       float scale, float clip, const void* W, const void* sW, const void* bias_or_null,
                                       int64_t N, void* y, void* workspace, size_t workspace_bytes, void* stream) {
    if (M < 0 || N < 0 || K <= 0 || had_K < 0) return QR_E_SHAPE;
    if (M == 0 || N == 0) return QR_OK;
    if (K % 64 != 0 || K > 131008) return QR_E_SHAPE;      // the GEMM's rules, checked before anything is launched
    if (!x || !W || !sW || !y) return QR_E_NULL;
    const size_t codes_bytes = align16((size_t)M * (size_t)(K / 2)), scales_bytes = align16((size_t)M * 2);
    if (!workspace || ((uintptr_t)workspace & 15) || workspace_bytes < codes_bytes + scales_bytes) return QR_E_WORKSPACE;
    uint8_t* codes = (uint8_t*)workspace;
    uint8_t* scales = codes + codes_bytes;
    uint8_t* rest = scales + scales_bytes;
    size_t rest_bytes = workspace_bytes - codes_bytes - scales_bytes;
    void* transformed = nullptr;                            // rows of 128 behind a Hadamard: see qr_hadamard_quantize_f16_i4
    if (K == 128 && had_K == 1 && mode == QR_DTYPE_F16) {
        const size_t t_bytes = align16((size_t)M * 256);
        if (rest_bytes < t_bytes) return QR_E_WORKSPACE;
        transformed = rest;
        rest += t_bytes, rest_bytes -= t_bytes;
    }
    // one token behind a long power-of-two factor: the front and the dot products in one launch (same codes, same sums)
    if (M <= 2 && had_K > 1 && mode == QR_DTYPE_F16 && hadK && ((uintptr_t)y & 1) == 0) {
        const int rc1 = qr_internal_token_hadamard_linear(x, M, (int)K, had_K, hadK, scale, clip, W, sW, bias_or_null, N, y,
                                                          (hipStream_t)stream);
        if (rc1 != QR_E_UNSUPPORTED) return rc1;
    }
    if (M <= 2 && had_K == 0 && ((uintptr_t)y & 1) == 0) {
        const int rc1 = qr_internal_token_quant_linear(x, M, K, clip, W, sW, bias_or_null, N, y, (hipStream_t)stream);
        if (rc1 != QR_E_UNSUPPORTED) return rc1;
    }
    int rc = had_K == 0 ? qr_quantize_rows_f16_i4(x, clip, M, K, codes, scales, stream)
                        : qr_hadamard_quantize_f16_i4(x, M, (int)K, had_K, hadK, mode, scale, clip, codes, scales,
                                                      transformed, stream);
    if (rc != QR_OK) return rc;
    return qr_linear_i4_f16_ws(codes, scales, W, sW, bias_or_null, M, N, K, y, rest_bytes ? rest : nullptr, rest_bytes,
                               stream);
}
