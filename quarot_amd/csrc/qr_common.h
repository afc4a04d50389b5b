// Shared device helpers for the gfx950 kernels of libquarot_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <mutex>
#include <vector>
#include <stdint.h>
#include "../../include/quarot_hip.h"

typedef _Float16 f16;
typedef f16 f16x2 __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef f16 f16x4 __attribute__((ext_vector_type(4)));
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32;
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));

#define QR_WAVE 64

// Raise a kernel's dynamic-LDS limit, once per (kernel, device, size): the runtime call costs host
// time on every launch otherwise.  A benign race at first use only repeats the call.
static inline hipError_t qr_allow_dynamic_lds(const void* kernel, size_t bytes) {
    struct Entry {
        const void* fn;
        int dev;
        size_t bytes;
    };
    static std::vector<Entry> table;            // grows with the kernel instantiations in use (never shrinks)
    static std::mutex guard;                    // entry points may be called from several host threads
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    std::lock_guard<std::mutex> lock(guard);
    for (Entry& t : table)
        if (t.fn == kernel && t.dev == dev) {
            if (t.bytes >= bytes) return hipSuccess;
            e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
            if (e == hipSuccess) t.bytes = bytes;
            return e;
        }
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e == hipSuccess) table.push_back(Entry{kernel, dev, bytes});
    return e;
}

// Compute units of the current device and the number of XCDs (L2 domains) they form: workgroups are
// dealt round-robin to the XCDs, 32 CUs each on gfx950 (256 CUs = 8 XCDs; a partitioned device has
// fewer of both).  Cached per device; {256, 8} if the query fails.
struct QrDevice {
    int cus, xcds;
};
static inline QrDevice qr_device() {
    constexpr int kMax = 64;
    static QrDevice table[kMax];
    static std::mutex guard;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMax) return QrDevice{256, 8};
    std::lock_guard<std::mutex> lock(guard);
    if (table[dev].cus == 0) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) cus = 256;
        table[dev] = QrDevice{cus, cus >= 64 ? cus / 32 : 1};
    }
    return table[dev];
}

// Resident workgroups per CU for a kernel at a given block size and dynamic LDS size (cached; used
// to size the grid of persistent kernels so that every workgroup is resident at once).
static inline int qr_blocks_per_cu(const void* kernel, int threads, size_t lds) {
    struct Entry {
        const void* fn;
        int dev, threads;
        size_t lds;
        int blocks;
    };
    static std::vector<Entry> table;
    static std::mutex guard;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 1;
    std::lock_guard<std::mutex> lock(guard);
    for (const Entry& t : table)
        if (t.fn == kernel && t.dev == dev && t.threads == threads && t.lds == lds) return t.blocks;
    int blocks = 1;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, kernel, threads, lds) != hipSuccess || blocks < 1) blocks = 1;
    table.push_back(Entry{kernel, dev, threads, lds, blocks});
    return blocks;
}

// kv.hip: y = x . H_128 * scale on rows of 128 halves (matrix-core kernel shared with the K-cache quantiser)
int qr_internal_hadamard128_f16(const void* x, void* y, int64_t rows, float scale, hipStream_t st);

// hadamard.hip: y = x . (hadK (x) I_128)^T / sqrt(heads) on rows of heads * 128 halves, then the quantiser
int qr_internal_heads_matrix_quantize(const void* x, int64_t rows, int heads, const void* hadK, float clip, void* q,
                                      void* scales, void* y_or_null, hipStream_t st);

// decode_fused.hip: Hadamard + quantiser + linear layer of one or two tokens in one launch (rows of 1024 K halves,
// K <= 32); QR_E_UNSUPPORTED, with nothing launched, for any other shape
int qr_internal_token_hadamard_linear(const void* x, int64_t M, int n, int K, const void* hadK, float scale, float clip,
                                      const void* W, const void* sW, const void* bias, int64_t N, void* y, hipStream_t st);

// decode_fused.hip: quantiser + linear layer of one or two tokens in one launch; QR_E_UNSUPPORTED, with nothing
// launched, for anything else
int qr_internal_token_quant_linear(const void* x, int64_t M, int64_t K, float clip, const void* W, const void* sW,
                                   const void* bias, int64_t N, void* y, hipStream_t st);

static inline int qr_launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? QR_OK : (int)e;
}

// fp16 bit helpers ---------------------------------------------------------------------------
__device__ __forceinline__ f16 f16_from_bits(unsigned short b) { return __builtin_bit_cast(f16, b); }
__device__ __forceinline__ unsigned short f16_bits(f16 h) { return __builtin_bit_cast(unsigned short, h); }

// Narrow a value that must FIRST be rounded to fp32 (the reference multiplies in fp32, then casts).
// The empty asm hides the producer from the optimiser, which otherwise folds "multiply, then
// convert" into v_fma_mixlo_f16: that instruction rounds the exact product once, and differs from
// the two-step result in rare double-rounding cases.
__device__ __forceinline__ f16 narrow_f16(float v) {
    asm("" : "+v"(v));
    return (f16)v;
}

// Two floats -> two fp16 (round to nearest even) packed in one word, `a` in the low half
// (v_cvt_pk_f16_f32).  The empty asm keeps a producing multiply from being folded into a
// single-rounding mixed-precision instruction, as in narrow_f16.
__device__ __forceinline__ u32 narrow_f16x2(float a, float b) {
    asm("" : "+v"(a), "+v"(b));
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {a, b};
    const f16x2 h = __builtin_convertvector(v, f16x2);
    return __builtin_bit_cast(u32, h);
}

// Two floats -> two fp16 (round to nearest even) where nothing can be folded into the conversion (the
// operands are matrix-instruction results, not products): no empty asm, so no copies of the operands.
__device__ __forceinline__ u32 cvt_f16x2(float a, float b) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {a, b};
    return __builtin_bit_cast(u32, __builtin_convertvector(v, f16x2));
}

// An 8-byte store that is written through the L2 to memory at once (device scope) instead of staying dirty in the
// L2 until the kernel ends; the line remains in the L2 for readers on the same XCD.
__device__ __forceinline__ void store_through(u32x2* dst, u32x2 v) {
    __hip_atomic_store((unsigned long long*)dst, ((unsigned long long)v[1] << 32) | v[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void store_through(u32* dst, u32 v) {
    __hip_atomic_store(dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Reinterpret one 32-bit word as two halves.  Always go through this by-value helper: applying
// __builtin_bit_cast directly to an element of an ext-vector (v[i]) was seen to read element 0
// whatever the index.
__device__ __forceinline__ f16x2 as_f16x2(u32 w) { return __builtin_bit_cast(f16x2, w); }

// max over |x| for the 8 halves held in a uint4, as raw magnitudes (sign bit cleared).  Comparing
// magnitudes as unsigned integers orders finite values and inf correctly and lets a NaN win, which
// is how torch.max propagates it.
__device__ __forceinline__ u32 absmax_bits8(u32x4 v) {
    u32 m = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        u32 w = v[i] & 0x7fff7fffu;
        u32 lo = w & 0xffffu, hi = w >> 16;
        m = m > lo ? m : lo;
        m = m > hi ? m : hi;
    }
    return m;
}

__device__ __forceinline__ u32 wave_max_u32(u32 v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        u32 o = (u32)__shfl_xor((int)v, off, QR_WAVE);
        v = v > o ? v : o;
    }
    return v;
}

// The same maximum without LDS round trips: four DPP steps reduce each row of 16 lanes (every lane
// of a row ends with the row's maximum), four lane reads and scalar maxima combine the rows.  The
// result is wave-uniform.
__device__ __forceinline__ u32 wave_max_u32_dpp(u32 v) {
    int o;
    o = __builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true);     // quad_perm [1,0,3,2]
    v = v > (u32)o ? v : (u32)o;
    o = __builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true);     // quad_perm [2,3,0,1]
    v = v > (u32)o ? v : (u32)o;
    o = __builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xF, 0xF, true);    // row_half_mirror
    v = v > (u32)o ? v : (u32)o;
    o = __builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xF, 0xF, true);    // row_mirror
    v = v > (u32)o ? v : (u32)o;
    const u32 r0 = (u32)__builtin_amdgcn_readlane((int)v, 0), r1 = (u32)__builtin_amdgcn_readlane((int)v, 16);
    const u32 r2 = (u32)__builtin_amdgcn_readlane((int)v, 32), r3 = (u32)__builtin_amdgcn_readlane((int)v, 48);
    const u32 a = r0 > r1 ? r0 : r1, b = r2 > r3 ? r2 : r3;
    return a > b ? a : b;
}

// Quantiser scale: fp16( float(fp16(amax / 7)) * clip ), each step correctly rounded.  amax / 7
// never lies on (or within 2^-14 relative of) an fp16 rounding boundary: a boundary (i + 1/2) ulp
// would need amax = 7 i + 3.5 units of its own grid.  So the fp32 product with the rounded
// constant 1/7 (relative error < 2^-23) rounds to the same fp16 as the exact quotient (checked for
// every finite fp16 amax).
__device__ __forceinline__ f16 quantizer_scale(f16 amax, float clip) {
    const f16 s = narrow_f16((float)amax * (1.0f / 7.0f));
    return narrow_f16((float)s * clip);
}

// One code: clamp(round_half_even(fp16(x / s)), -8, 7) with x / s a single correctly rounded fp16
// division.  `rs` = 1.0f / s (IEEE).  q1 below is x / s to within a fraction of a float ulp
// (reciprocal, one Newton correction with exact residual); the exact quotient of two fp16 numbers
// is either an fp16 rounding boundary itself (then q1 is exact, the quotient having <= 12
// significant bits) or at least 2^-23 away from one in relative terms, more than q1's error, so
// rounding q1 to fp16 gives the correctly rounded quotient.  s == 0 and non-finite cases take the
// IEEE division directly.  NaN converts to 0, +-inf saturates and is clamped.
__device__ __forceinline__ int sym_code(f16 x, float s, float rs, bool fast_ok) {
    float xf = (float)x;
    float q;
    if (fast_ok) {
        float q0 = xf * rs;
        float e = __builtin_fmaf(-q0, s, xf);
        float q1 = __builtin_fmaf(e, rs, q0);
        q = __builtin_fabsf(q0) < __builtin_inff() ? q1 : q0;   // x = +-inf: keep the infinity
    } else {
        q = xf / s;
    }
    f16 d = (f16)q;
    float r = __builtin_rintf((float)d);
    int c = (int)r;              // v_cvt_i32_f32: NaN -> 0, saturating
    c = c < -8 ? -8 : c;
    c = c > 7 ? 7 : c;
    return (r != r) ? 0 : c;
}

// 8 fp16 (one 16-byte chunk) -> 8 nibbles in one 32-bit word, element 0 in the lowest nibble.
__device__ __forceinline__ u32 sym_codes8(u32x4 v, float s, float rs, bool fast_ok) {
    u32 out = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f16 a = f16_from_bits((unsigned short)(v[i] & 0xffffu));
        f16 b = f16_from_bits((unsigned short)(v[i] >> 16));
        u32 ca = (u32)sym_code(a, s, rs, fast_ok) & 0xfu;
        u32 cb = (u32)sym_code(b, s, rs, fast_ok) & 0xfu;
        out |= (ca | (cb << 4)) << (8 * i);
    }
    return out;
}

// ---- lean quantiser for rows known to be all-finite with a finite non-zero scale ------------------
// q = x * r with r the CORRECTLY ROUNDED fp32 reciprocal of the scale: one multiplication per value.
// That (f16)q is the correctly rounded fp16 division wherever a code depends on it (quotients in
// [0.25, 32): below, every candidate rounds to code 0; above, the clamp decides) was checked by brute
// force over every pair of a finite fp16 value and a positive finite fp16 scale (31744 x 31743 pairs:
// no difference; with r one ulp off in either direction a few thousand pairs differ, so the
// reciprocal must be the correctly rounded one).  Why it works: a quotient of two fp16 numbers keeps
// a relative distance above 2^-23 from every fp16 rounding boundary (see sym_code), and the two
// roundings here (r, then the product) stay within 2^-23.
// Adding 1536 (ulp 1 in [1024, 2048)) in fp16 rounds to the nearest integer, ties to even, and leaves the
// two's-complement code in the low four mantissa bits; the clamp to [-8, 7] follows on the bit patterns
// (sym_pair_fast), which commutes with the rounding (monotone, and -8, 7 are representable).
struct FastRecip {
    float r;
};
// s: a finite non-zero fp16 value as float.  v_rcp_f32 is good to one ulp; a Newton step in fma form
// brings r1 within 2^-24 (1 + 2^-22) of 1 / s; in the second step e = 1 - s r1 is EXACT (s has 11
// significant bits, the product 35, and all but 12 cancel), so fma(e, r1, r1) rounds
// (1 / s) (1 - e^2) once: the correctly rounded reciprocal, because 1 / s for an 11-bit s keeps a
// relative distance of at least 2^-36 from every fp32 rounding boundary and e^2 < 2^-46.
__device__ __forceinline__ FastRecip make_fast_recip(float s) {
    const float r0 = __builtin_amdgcn_rcpf(s);
    const float r1 = __builtin_fmaf(__builtin_fmaf(-s, r0, 1.0f), r0, r0);
    FastRecip f;
    f.r = __builtin_fmaf(__builtin_fmaf(-s, r1, 1.0f), r1, r1);
    return f;
}
// w[i] holds two fp16 values 1536 + code (codes in the low four bits of each half, element 2 i in
// the low half): gather the eight nibbles into one word, element 0 lowest.  Two byte permutes bring
// the low bytes of all eight halves together, two more split them into the bytes of the even and of
// the odd elements, a shift and a bit-select merge them: six instructions.
__device__ __forceinline__ u32 pack_nibbles8(const u32 (&w)[4]) {
    const u32 p01 = __builtin_amdgcn_perm(w[1], w[0], 0x06020400u);     // w0.b0 w1.b0 w0.b2 w1.b2
    const u32 p23 = __builtin_amdgcn_perm(w[3], w[2], 0x06020400u);
    const u32 even = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
    const u32 odd = __builtin_amdgcn_perm(p23, p01, 0x07060302u);
    return (even & 0x0F0F0F0Fu) | ((odd << 4) & 0xF0F0F0F0u);
}
// Two codes from one packed word, as the fp16 pair (1536 + code, 1536 + code).  The quotient is formed as
// fp16(fma(x, r, 0)) -- the halves go into the mixed-precision multiply as they are, and where the compiler
// takes the form that rounds the exact product once (v_fma_mixlo/hi_f16) the result is still the correctly
// rounded fp16 quotient: x r lies within 2^-24 (relative) of x / s and a quotient of two fp16 numbers keeps more
// than 2^-23 from every rounding boundary it is not exactly on.  The clamp acts on the bit patterns AFTER the
// addition: 1536 + code in [1528, 1543] is 0x65f8 .. 0x6607, patterns of positive halves order like signed
// 16-bit integers, every negative sum (quotients below -1536) is a negative integer and an overflow to +inf
// (0x7c00) lies above: two packed integer instructions instead of two fp32 clamps and a conversion.
template <bool CLAMP>
__device__ __forceinline__ u32 sym_pair_fast(u32 w, FastRecip f) {
    const f16x2 h2 = as_f16x2(w);
    f16x2 qh = {(f16)__builtin_fmaf((float)h2[0], f.r, 0.0f), (f16)__builtin_fmaf((float)h2[1], f.r, 0.0f)};
    qh = qh + f16x2{(f16)1536.0f, (f16)1536.0f};
    if (!CLAMP) return __builtin_bit_cast(u32, qh);
    typedef short i16x2 __attribute__((ext_vector_type(2)));
    i16x2 b = __builtin_bit_cast(i16x2, qh);
    b = __builtin_elementwise_max(b, i16x2{0x65f8, 0x65f8});
    b = __builtin_elementwise_min(b, i16x2{0x6607, 0x6607});
    return __builtin_bit_cast(u32, b);
}
// 8 fp16 (one 16-byte chunk) -> 8 nibbles, element 0 lowest: four sym_pair_fast and the gather.  CLAMP = false only
// where clamp_cannot_act() holds for the row.
template <bool CLAMP = true>
__device__ __forceinline__ u32 sym_codes8_fast(u32x4 v, FastRecip f) {
    u32 b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) b[i] = sym_pair_fast<CLAMP>(v[i], f);
    return pack_nibbles8(b);
}
// A scale that the quantiser itself derived from the row's largest magnitude with clip >= 1 keeps every quotient
// inside the code range when it is a normal fp16 number: |x| <= amax and s >= (amax / 7) (1 - 2^-11)^2 give
// |x / s| < 7.5, which rounds to at most 7 (a subnormal scale can be several per cent off: it keeps the clamp).
__device__ __forceinline__ bool clamp_cannot_act(float clip, float s) { return clip >= 1.0f && s >= 6.103515625e-05f; }
// amax bits below 0x7c00 <=> every element of the row is finite
__device__ __forceinline__ bool fast_quant_ok(u32 amax_bits, float s) {
    const float a = __builtin_fabsf(s);
    return amax_bits < 0x7c00u && a > 0.0f && a < __builtin_inff();
}

// The reciprocal path is valid when s is a finite non-zero fp16 (then 1/s is a finite float).
__device__ __forceinline__ bool scale_fast_ok(float s) {
    float a = __builtin_fabsf(s);
    return a > 0.0f && a < __builtin_inff();
}
