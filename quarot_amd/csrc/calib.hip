// Measurement aids of libquarot_hip.so: kernels whose work is known exactly, for calibrating the two
// rooflines the library's kernels are priced against.  They have no counterpart in the reference and
// no caller in the product path; bench.py runs them next to the workloads.
//   qr_calib_mfma_i8   a register-only loop of v_mfma_i32_32x32x32_i8 (the int4 GEMMs' instruction):
//                      what the matrix pipe sustains on this part with nothing else going on, for
//                      all-zero operands and for operands with the GEMMs' bit statistics
//   qr_calib_copy      a plain copy of known size (16-byte loads and stores): what the profiler's
//                      FETCH_SIZE / WRITE_SIZE counters read for known traffic, and what HBM streams
#include "qr_common.h"

namespace {

// One workgroup = four waves (one per SIMD); a wave keeps four independent accumulator chains going,
// which is how the GEMM kernels issue the instruction (no chain waits for its own previous result).
// Operands: pattern 0 = zeros; 1 = bytes 16 * (code in -8..7), random codes -- exactly what the int4
// kernels feed (nibbles moved to the high half of each byte); 2 = random int8 bytes; 3 = random codes -8..7 as
// sign-extended int8 (what a kernel that unpacked to true int8 would feed).
__global__ __launch_bounds__(256, 1) void calib_mfma_i8_kernel(int pattern, int iters, int store, int* __restrict__ out) {
    u32 seed = (u32)(blockIdx.x * 256 + threadIdx.x) * 2654435761u + 12345u;
    auto next = [&]() {
        seed ^= seed << 13;
        seed ^= seed >> 17;
        seed ^= seed << 5;
        return seed;
    };
    i32x4 a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const u32 ra = next(), rb = next();
            auto sext = [](u32 r) {                       // every byte: its low nibble as a two's-complement int4, sign-extended
                const u32 n = r & 0x0F0F0F0Fu;
                return n | (((n >> 3) & 0x01010101u) * 0xF0u);
            };
            a[i][w] = pattern == 0 ? 0 : pattern == 1 ? (int)(ra & 0xF0F0F0F0u) : pattern == 2 ? (int)ra : (int)sext(ra);
            b[i][w] = pattern == 0 ? 0 : pattern == 1 ? (int)(rb & 0xF0F0F0F0u) : pattern == 2 ? (int)rb : (int)sext(rb);
        }
    i32x16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 4; ++u)                       // 16 instructions per turn
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[(i + u) & 3], b[i], acc[i], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += acc[i][r];
    if (store) out[blockIdx.x * 256 + threadIdx.x] = s;   // (the host passes store = 0: the sums only keep the loop alive)
}

__global__ __launch_bounds__(256) void calib_copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t pieces) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < pieces; i += stride)
        __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

}  // namespace

// ops per launch = workgroups * 4 waves * iters * 16 instructions * 2 * 32 * 32 * 32
extern "C" int qr_calib_mfma_i8(int pattern, int iters, int workgroups, void* out, void* stream) {
    if (pattern < 0 || pattern > 3) return QR_E_DTYPE;
    if (iters <= 0 || workgroups <= 0 || workgroups > (1 << 20)) return QR_E_SHAPE;
    if (!out) return QR_E_NULL;
    calib_mfma_i8_kernel<<<dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream>>>(pattern, iters, 0, (int*)out);
    return qr_launch_status();
}

extern "C" int qr_calib_copy(const void* src, void* dst, int64_t bytes, void* stream) {
    if (bytes < 0 || (bytes & 15)) return QR_E_SHAPE;
    if (bytes == 0) return QR_OK;
    if (!src || !dst) return QR_E_NULL;
    if (((uintptr_t)src & 15) || ((uintptr_t)dst & 15)) return QR_E_ALIGN;
    const int64_t pieces = bytes >> 4;
    const int64_t want = (pieces + 255) / 256, cap = (int64_t)qr_device().cus * 16;
    calib_copy_kernel<<<dim3((unsigned)(want < cap ? want : cap)), dim3(256), 0, (hipStream_t)stream>>>(
        (const u32x4*)src, (u32x4*)dst, pieces);
    return qr_launch_status();
}
