// Version and error text of libquarot_hip.so.
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
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error code";
}
