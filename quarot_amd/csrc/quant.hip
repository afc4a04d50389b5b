// Symmetric per-token int4 quantiser and the int32 -> fp16 dequantiser (HBM-bound kernels).
#include "qr_common.h"

namespace {

constexpr int QT = 256;           // threads per workgroup

// One workgroup per row.  NV = 16-byte chunks (8 halves) each thread keeps in registers, so a row
// of up to 256 * 8 * NV columns is read from HBM exactly once.  GIVEN_SCALE: scale[row] is an
// input (sym_quant); otherwise it is derived from the row abs-max and written out (Quantizer).
template <int NV, bool GIVEN_SCALE>
__global__ __launch_bounds__(QT) void quant_rows_kernel(const u32x4* __restrict__ x, const f16* __restrict__ scale_in,
                                                        float clip, int cols8, u32* __restrict__ q,
                                                        f16* __restrict__ scale_out) {
    __shared__ u32 red[QT / QR_WAVE];
    const int64_t row = blockIdx.x;
    const u32x4* xr = x + row * (int64_t)cols8;
    u32x4 v[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        int c = threadIdx.x + i * QT;
        v[i] = c < cols8 ? __builtin_nontemporal_load(xr + c) : u32x4{0, 0, 0, 0};
    }
    // the row's largest magnitude: it gives the scale, and (also with a given scale) tells whether the row is all
    // finite, i.e. whether the lean codes apply
    float s;
    u32 m = 0;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        u32 mi = absmax_bits8(v[i]);
        m = m > mi ? m : mi;
    }
    m = wave_max_u32(m);
    if ((threadIdx.x & (QR_WAVE - 1)) == 0) red[threadIdx.x / QR_WAVE] = m;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < QT / QR_WAVE; ++w) m = m > red[w] ? m : red[w];
    if (GIVEN_SCALE) {
        s = (float)scale_in[row];
    } else {
        f16 sh = quantizer_scale(f16_from_bits((unsigned short)m), clip);
        if (threadIdx.x == 0) scale_out[row] = sh;
        s = (float)sh;
    }
    u32* qr = q + row * (int64_t)cols8;
    if (fast_quant_ok(m, s)) {       // workgroup-uniform
        const FastRecip fr = make_fast_recip(s);
        // (codes are written through the L2: the GEMM that follows still finds them there, and they are not left to
        // be written back in a burst when the kernel ends -- 2048 x 4096: 4.5 -> 4.35 us, the step 33.8 -> 33.5 us)
        if (!GIVEN_SCALE && clamp_cannot_act(clip, s)) {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                int c = threadIdx.x + i * QT;
                if (c < cols8) store_through(&qr[c], sym_codes8_fast<false>(v[i], fr));
            }
        } else {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                int c = threadIdx.x + i * QT;
                if (c < cols8) store_through(&qr[c], sym_codes8_fast<true>(v[i], fr));
            }
        }
        return;
    }
    const bool fast = scale_fast_ok(s);
    const float rs = fast ? 1.0f / s : 0.0f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        int c = threadIdx.x + i * QT;
        if (c < cols8) qr[c] = sym_codes8(v[i], s, rs, fast);
    }
}

// Wave-wide fp32 sum without LDS: four DPP steps reduce each row of 16 lanes, four lane reads combine
// the rows.  The result is wave-uniform; the association order is fixed.
__device__ __forceinline__ float wave_sum_f32_dpp(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return (r0 + r1) + (r2 + r3);
}

// RMSNorm (no gain) followed by the per-token quantiser, one pass over x: the row stays in
// registers between the two reductions.  The normalised value is rounded to fp16 exactly where
// the unfused chain stores it -- fp16( float(x) * rsqrt(sum(x^2) / mean_dim + eps) ), all in fp32 --
// and the quantiser runs on those fp16 values.  Only the association order of the fp32 sum of
// squares is this kernel's own.
template <int NV>
__global__ __launch_bounds__(QT) void rmsnorm_quant_rows_kernel(const u32x4* __restrict__ x, float mean_dim, float eps,
                                                                float clip, int cols8, u32* __restrict__ q,
                                                                f16* __restrict__ scale_out, u32x4* __restrict__ y) {
    __shared__ float redf[QT / QR_WAVE];
    __shared__ u32 red[QT / QR_WAVE];
    const int64_t row = blockIdx.x;
    const int lane = threadIdx.x & (QR_WAVE - 1), wave = threadIdx.x / QR_WAVE;
    const u32x4* xr = x + row * (int64_t)cols8;
    u32x4 v[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = threadIdx.x + i * QT;
        v[i] = c < cols8 ? xr[c] : u32x4{0, 0, 0, 0};
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const f16x2 h = as_f16x2(v[i][w]);
            const float a = (float)h[0], b = (float)h[1];
            ss = __builtin_fmaf(a, a, ss);          // a * a is exact in fp32 (22 bits)
            ss = __builtin_fmaf(b, b, ss);
        }
    ss = wave_sum_f32_dpp(ss);
    if (lane == 0) redf[wave] = ss;
    __syncthreads();
    const float total = (redf[0] + redf[1]) + (redf[2] + redf[3]);
    const float r = 1.0f / __builtin_sqrtf(total / mean_dim + eps);
    u32 m = 0;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const f16x2 h = as_f16x2(v[i][w]);
            v[i][w] = narrow_f16x2((float)h[0] * r, (float)h[1] * r);
        }
        const u32 mi = absmax_bits8(v[i]);
        m = m > mi ? m : mi;
    }
    m = wave_max_u32_dpp(m);
    if (lane == 0) red[wave] = m;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < QT / QR_WAVE; ++w) m = m > red[w] ? m : red[w];
    const f16 sh = quantizer_scale(f16_from_bits((unsigned short)m), clip);
    if (threadIdx.x == 0) scale_out[row] = sh;
    const float s = (float)sh;
    u32* qr = q + row * (int64_t)cols8;
    if (y) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = threadIdx.x + i * QT;
            if (c < cols8) y[row * (int64_t)cols8 + c] = v[i];
        }
    }
    if (fast_quant_ok(m, s)) {       // workgroup-uniform
        const FastRecip fr = make_fast_recip(s);
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = threadIdx.x + i * QT;
            if (c < cols8) store_through(&qr[c], sym_codes8_fast(v[i], fr));      // (through the L2, as in quant_rows_kernel)
        }
        return;
    }
    const bool fast = scale_fast_ok(s);
    const float rs = fast ? 1.0f / s : 0.0f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = threadIdx.x + i * QT;
        if (c < cols8) qr[c] = sym_codes8(v[i], s, rs, fast);
    }
}

// Hadamard across the heads of an attention output row, then the quantiser, in one pass
// (e2e/quantized_llama/modeling_llama.py:108-110: OnlineHadamard(num_heads) on the transposed view,
// transpose back, reshape, then o_proj's Quantizer).  A row is [H, 128] fp16, H = 4 NC heads; the
// transform is the Walsh-Hadamard transform of size H over the head index for each of the 128
// positions, scaled by 1/sqrt(H) and rounded to fp16 once (quarot/nn/hadamard.py:17-23 with K = 1).
// One WAVE per row, four rows per workgroup, no LDS and no barrier: lane l holds the 16-byte chunks
// l + 64 i, i.e. heads (l >> 4) + 4 i at positions 8 (l & 15) ...: head bits 2.. are the chunk index
// i (butterflies in the lane), bits 0 and 1 are lane bits 4 and 5 (v_permlane16_swap /
// v_permlane32_swap, one swap per butterfly).  The row maximum is a wave reduction.
template <int NC>
__global__ __launch_bounds__(QT) void heads_hadamard_quant_rows_kernel(const u32x4* __restrict__ x, int64_t rows,
                                                                       float hscale, float clip, u32* __restrict__ q,
                                                                       f16* __restrict__ scale_out,
                                                                       u32x4* __restrict__ y) {
    constexpr int cols8 = NC * QR_WAVE;
    const int lane = threadIdx.x & (QR_WAVE - 1), wave = threadIdx.x / QR_WAVE;
    const int64_t row = (int64_t)blockIdx.x * (QT / QR_WAVE) + wave;
    if (row >= rows) return;                                // a whole wave: nothing below synchronises waves
    const u32x4* xr = x + row * (int64_t)cols8;
    u32x4 raw[NC];
#pragma unroll
    for (int i = 0; i < NC; ++i) raw[i] = xr[lane + i * QR_WAVE];
    // head bits 2..: pairs of chunks of this lane.  The first stage reads the fp16 pairs directly
    // (fused multiply-adds by +-1 with fp16 sources: one instruction converts and adds).
    float f[NC][8];
    float one = 1.0f, minus_one = -1.0f;
    asm volatile("" : "+v"(one), "+v"(minus_one));           // opaque, or the compiler splits the fma into convert + add
#pragma unroll
    for (int i = 0; i < NC; i += 2)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const f16x2 lo = as_f16x2(raw[i][w]), hi = as_f16x2(raw[i + 1][w]);
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                f[i][2 * w + k] = __builtin_fmaf((float)hi[k], one, (float)lo[k]);
                f[i + 1][2 * w + k] = __builtin_fmaf((float)hi[k], minus_one, (float)lo[k]);
            }
        }
#pragma unroll
    for (int b = 2; b < NC; b <<= 1)
#pragma unroll
        for (int i = 0; i < NC; ++i)
            if ((i & b) == 0) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float lo = f[i][e], hi = f[i | b][e];
                    f[i][e] = lo + hi;
                    f[i | b][e] = lo - hi;
                }
            }
    // head bits 0 and 1: lanes 16 and 32 apart.  Two values A, B of a lane go through a stage together:
    // swapping A with B across the lane pair leaves (A_lower, A_upper) in the lower lane and
    // (B_lower, B_upper) in the upper one; each forms sum and difference of what it holds, and a second
    // swap hands the lower lane both sums and the upper lane both differences -- two swaps, one add
    // and one subtract for two butterflies.  Then scale and round to fp16.
    u32x4 v[NC];
    u32 m = 0;
#pragma unroll
    for (int i = 0; i < NC; ++i) {
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
            u32 a = __builtin_bit_cast(u32, f[i][e]), c = __builtin_bit_cast(u32, f[i][e + 1]);
            {
                const auto s1 = __builtin_amdgcn_permlane16_swap(a, c, false, false);
                const float lo = __builtin_bit_cast(float, (u32)s1[0]), hi = __builtin_bit_cast(float, (u32)s1[1]);
                const auto s2 = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(u32, lo + hi),
                                                                 __builtin_bit_cast(u32, lo - hi), false, false);
                a = s2[0];
                c = s2[1];
            }
            {
                const auto s1 = __builtin_amdgcn_permlane32_swap(a, c, false, false);
                const float lo = __builtin_bit_cast(float, (u32)s1[0]), hi = __builtin_bit_cast(float, (u32)s1[1]);
                const auto s2 = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(u32, lo + hi),
                                                                 __builtin_bit_cast(u32, lo - hi), false, false);
                a = s2[0];
                c = s2[1];
            }
            f[i][e] = __builtin_bit_cast(float, a);
            f[i][e + 1] = __builtin_bit_cast(float, c);
        }
#pragma unroll
        for (int w = 0; w < 4; ++w) v[i][w] = narrow_f16x2(f[i][2 * w] * hscale, f[i][2 * w + 1] * hscale);
        const u32 mi = absmax_bits8(v[i]);
        m = m > mi ? m : mi;
    }
    m = wave_max_u32_dpp(m);
    const f16 sh = quantizer_scale(f16_from_bits((unsigned short)m), clip);
    if (lane == 0) scale_out[row] = sh;
    const float s = (float)sh;
    u32* qr = q + row * (int64_t)cols8;
    if (y) {
#pragma unroll
        for (int i = 0; i < NC; ++i) y[row * (int64_t)cols8 + lane + i * QR_WAVE] = v[i];
    }
    if (fast_quant_ok(m, s)) {       // wave-uniform
        const FastRecip fr = make_fast_recip(s);
#pragma unroll
        for (int i = 0; i < NC; ++i) store_through(&qr[lane + i * QR_WAVE], sym_codes8_fast(v[i], fr));   // (through the L2, as in quant_rows_kernel)
        return;
    }
    const bool fast = scale_fast_ok(s);
    const float rs = fast ? 1.0f / s : 0.0f;
#pragma unroll
    for (int i = 0; i < NC; ++i) qr[lane + i * QR_WAVE] = sym_codes8(v[i], s, rs, fast);
}

// Any column count (odd included), any alignment: one workgroup per row, scalar accesses, the row
// is read twice when the scale has to be derived.  Used only when the vector kernel's
// preconditions (cols % 8 == 0, cols <= 32768, 16-byte aligned x, 4-byte aligned q) do not hold.
template <bool GIVEN_SCALE>
__global__ __launch_bounds__(QT) void quant_rows_generic_kernel(const f16* __restrict__ x, const f16* __restrict__ scale_in,
                                                                float clip, int64_t cols, uint8_t* __restrict__ q,
                                                                f16* __restrict__ scale_out) {
    __shared__ u32 red[QT / QR_WAVE];
    const int64_t row = blockIdx.x;
    const f16* xr = x + row * cols;
    const int64_t cols_dst = (cols + 1) / 2;
    float s;
    if (GIVEN_SCALE) {
        s = (float)scale_in[row];
    } else {
        u32 m = 0;
        for (int64_t c = threadIdx.x; c < cols; c += QT) {
            u32 b = f16_bits(xr[c]) & 0x7fffu;
            m = m > b ? m : b;
        }
        m = wave_max_u32(m);
        if ((threadIdx.x & (QR_WAVE - 1)) == 0) red[threadIdx.x / QR_WAVE] = m;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < QT / QR_WAVE; ++w) m = m > red[w] ? m : red[w];
        f16 sh = quantizer_scale(f16_from_bits((unsigned short)m), clip);
        if (threadIdx.x == 0) scale_out[row] = sh;
        s = (float)sh;
    }
    const bool fast = scale_fast_ok(s);
    const float rs = fast ? 1.0f / s : 0.0f;
    for (int64_t j = threadIdx.x; j < cols_dst; j += QT) {
        u32 lo = (u32)sym_code(xr[2 * j], s, rs, fast) & 0xfu;
        u32 hi = (2 * j + 1 < cols) ? ((u32)sym_code(xr[2 * j + 1], s, rs, fast) & 0xfu) : 0u;
        q[row * cols_dst + j] = (uint8_t)(lo | (hi << 4));
    }
}

// y = fp16(fp16(sr * sc) * fp16_rn(q)): 8 columns per thread (two 16-byte loads, one 16-byte store).
__global__ __launch_bounds__(QT) void dequant_i32_f16_kernel(const int32_t* __restrict__ q, const f16* __restrict__ sr,
                                                             const f16* __restrict__ sc, int64_t rows, int64_t cols,
                                                             f16* __restrict__ y, bool vec_ok) {
    const int64_t cols8 = (cols + 7) / 8;
    const int64_t total = rows * cols8;
    for (int64_t idx = (int64_t)blockIdx.x * QT + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * QT) {
        const int64_t r = idx / cols8;
        const int64_t c0 = (idx - r * cols8) * 8;
        const f16 a = sr[r];
        const int32_t* qp = q + r * cols + c0;
        f16* yp = y + r * cols + c0;
        if (vec_ok && c0 + 8 <= cols) {
            i32x4 q0 = __builtin_nontemporal_load((const i32x4*)qp);
            i32x4 q1 = __builtin_nontemporal_load((const i32x4*)qp + 1);
            f16x8 b = *(const f16x8*)(sc + c0);
            f16x8 o;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                o[i] = (f16)(a * b[i]) * (f16)(float)q0[i];
                o[i + 4] = (f16)(a * b[i + 4]) * (f16)(float)q1[i];
            }
            __builtin_nontemporal_store(o, (f16x8*)yp);
        } else {
            for (int i = 0; i < 8 && c0 + i < cols; ++i) yp[i] = (f16)(a * sc[c0 + i]) * (f16)(float)qp[i];
        }
    }
}

template <bool GIVEN>
int launch_quant(const void* x, const void* scale_in, float clip, int64_t rows, int64_t cols, void* q, void* scale_out,
                 hipStream_t st) {
    if (rows == 0 || cols == 0) return QR_OK;
    const bool vec = (cols % 8 == 0) && cols <= 32768 && (((uintptr_t)x & 15) == 0) && (((uintptr_t)q & 3) == 0);
    dim3 grid((unsigned)rows), block(QT);
    if (rows > 0x7fffffffLL) return QR_E_SHAPE;
    if (!vec) {
        quant_rows_generic_kernel<GIVEN><<<grid, block, 0, st>>>((const f16*)x, (const f16*)scale_in, clip, cols,
                                                                  (uint8_t*)q, (f16*)scale_out);
        return qr_launch_status();
    }
    const int cols8 = (int)(cols / 8);
    const int nv = (cols8 + QT - 1) / QT;
#define QR_LAUNCH(NV)                                                                                                  \
    quant_rows_kernel<NV, GIVEN><<<grid, block, 0, st>>>((const u32x4*)x, (const f16*)scale_in, clip, cols8, (u32*)q, \
                                                         (f16*)scale_out)
    if (nv <= 1) QR_LAUNCH(1);
    else if (nv <= 2) QR_LAUNCH(2);
    else if (nv <= 4) QR_LAUNCH(4);
    else if (nv <= 6) QR_LAUNCH(6);
    else if (nv <= 8) QR_LAUNCH(8);
    else QR_LAUNCH(16);
#undef QR_LAUNCH
    return qr_launch_status();
}

}  // namespace

extern "C" int qr_sym_quant_f16_i4(const void* x, const void* scale, int64_t rows, int64_t cols, void* q, void* stream) {
    if (rows < 0 || cols < 0) return QR_E_SHAPE;
    if (rows == 0 || cols == 0) return QR_OK;
    if (!x || !scale || !q) return QR_E_NULL;
    return launch_quant<true>(x, scale, 1.0f, rows, cols, q, nullptr, (hipStream_t)stream);
}

extern "C" int qr_quantize_rows_f16_i4(const void* x, float clip, int64_t rows, int64_t cols, void* q, void* scales,
                                       void* stream) {
    if (rows < 0 || cols < 0) return QR_E_SHAPE;
    if (rows == 0) return QR_OK;
    if (cols == 0) return QR_E_SHAPE;   // torch.max over an empty axis raises in the reference
    if (!x || !q || !scales) return QR_E_NULL;
    return launch_quant<false>(x, nullptr, clip, rows, cols, q, scales, (hipStream_t)stream);
}

extern "C" int qr_rmsnorm_quantize_f16_i4(const void* x, int64_t rows, int64_t cols, int mean_dim, float eps, float clip,
                                          void* q, void* scales, void* y_or_null, void* stream) {
    if (rows < 0 || cols <= 0 || mean_dim <= 0) return QR_E_SHAPE;
    if (rows == 0) return QR_OK;
    if (rows > 0x7fffffffLL) return QR_E_SHAPE;
    if (!x || !q || !scales) return QR_E_NULL;
    if (cols % 8 != 0 || cols > 32768) return QR_E_UNSUPPORTED;
    if (((uintptr_t)x & 15) || ((uintptr_t)y_or_null & 15) || ((uintptr_t)q & 3)) return QR_E_ALIGN;
    const int cols8 = (int)(cols / 8);
    const int nv = (cols8 + QT - 1) / QT;
    dim3 grid((unsigned)rows), block(QT);
    hipStream_t st = (hipStream_t)stream;
#define QR_LAUNCH(NV)                                                                                                 \
    rmsnorm_quant_rows_kernel<NV><<<grid, block, 0, st>>>((const u32x4*)x, (float)mean_dim, eps, clip, cols8, (u32*)q, \
                                                          (f16*)scales, (u32x4*)y_or_null)
    if (nv <= 1) QR_LAUNCH(1);
    else if (nv <= 2) QR_LAUNCH(2);
    else if (nv <= 4) QR_LAUNCH(4);
    else if (nv <= 6) QR_LAUNCH(6);
    else if (nv <= 8) QR_LAUNCH(8);
    else QR_LAUNCH(16);
#undef QR_LAUNCH
    return qr_launch_status();
}

extern "C" int qr_heads_hadamard_quantize_f16_i4(const void* x, int64_t rows, int heads, int head_dim,
                                                 const void* hadK_or_null, float clip, void* q, void* scales,
                                                 void* y_or_null, void* stream) {
    if (rows < 0 || heads <= 0 || head_dim <= 0) return QR_E_SHAPE;
    if (rows == 0) return QR_OK;
    if (rows > 0x7fffffffLL) return QR_E_SHAPE;
    if (!x || !q || !scales) return QR_E_NULL;
    const bool pow2 = heads == 16 || heads == 32 || heads == 64;
    const bool table = hadK_or_null && heads % 4 == 0 && heads <= 64 && !pow2;
    if (head_dim != 128 || !(pow2 || table)) return QR_E_UNSUPPORTED;
    if (((uintptr_t)x & 15) || ((uintptr_t)y_or_null & 15) || ((uintptr_t)q & 3)) return QR_E_ALIGN;
    if (table)
        return qr_internal_heads_matrix_quantize(x, rows, heads, hadK_or_null, clip, q, scales, y_or_null,
                                                 (hipStream_t)stream);
    dim3 grid((unsigned)((rows + QT / QR_WAVE - 1) / (QT / QR_WAVE))), block(QT);
    hipStream_t st = (hipStream_t)stream;
    const float hscale = 1.0f / __builtin_sqrtf((float)heads);
#define QR_LAUNCH(NC)                                                                                                 \
    heads_hadamard_quant_rows_kernel<NC><<<grid, block, 0, st>>>((const u32x4*)x, rows, hscale, clip, (u32*)q,        \
                                                                 (f16*)scales, (u32x4*)y_or_null)
    if (heads == 16) QR_LAUNCH(4);
    else if (heads == 32) QR_LAUNCH(8);
    else QR_LAUNCH(16);
#undef QR_LAUNCH
    return qr_launch_status();
}

extern "C" int qr_sym_dequant_i32_f16(const void* q, const void* scale_row, const void* scale_col, int64_t rows,
                                      int64_t cols, void* y, void* stream) {
    if (rows < 0 || cols < 0) return QR_E_SHAPE;
    if (rows == 0 || cols == 0) return QR_OK;
    if (!q || !scale_row || !scale_col || !y) return QR_E_NULL;
    const bool vec_ok = (cols % 8 == 0) && (((uintptr_t)q & 15) == 0) && (((uintptr_t)y & 15) == 0) &&
                        (((uintptr_t)scale_col & 15) == 0);
    const int64_t total = rows * ((cols + 7) / 8);
    int64_t blocks = (total + QT - 1) / QT;
    if (blocks > 256 * 64) blocks = 256 * 64;
    dequant_i32_f16_kernel<<<dim3((unsigned)blocks), dim3(QT), 0, (hipStream_t)stream>>>(
        (const int32_t*)q, (const f16*)scale_row, (const f16*)scale_col, rows, cols, (f16*)y, vec_ok);
    return qr_launch_status();
}
