// Asymmetric int4 quantiser of the KV cache (quarot/transformers/kv_cache.py:10-33): the code forms shared by kv.hip
// and attn.hip, and the quantiser of ONE 128-wide vector by one wave, for kernels that quantise the vector they are
// about to use.
#pragma once
#include "qr_paged.h"

// Eight codes clamp(round_half_even(fp16(fp16(x + zero) / scale)), 0, 15) for all-finite input: the
// add is one packed fp16 add, the division the one-multiplication form of sym_codes8_fast (the
// shifted value is an fp16 number like any other), the rounding the +1536 trick.
// CLAMP = false leaves the clamp out: the shifted values lie in [0, range] by construction, so with a
// scale that is a NORMAL fp16 number (relative rounding error <= 2^-11: range >= 2^-10 is enough) the
// quotient is at most 15 (1 + 2^-11) and rounds to 15 at most.  A subnormal scale can be off by several
// per cent and needs the clamp (range / 15 = 10.5 units of 2^-24 -> scale 10 units -> quotient 15.75).
template <bool CLAMP = true>
__device__ __forceinline__ u32 asym_codes8_fast(u32x4 v, f16 zero, FastRecip f) {
    const f16x2 z2 = {zero, zero};
    u32 b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const f16x2 sh = as_f16x2(v[i]) + z2;
        // the quotient straight from the packed pair to the packed fp16 quotient (one mixed-precision instruction per
        // value; see sym_pair_fast for why its single rounding is still the correctly rounded division), then + 1536
        f16x2 h = {(f16)__builtin_fmaf((float)sh[0], f.r, 0.0f), (f16)__builtin_fmaf((float)sh[1], f.r, 0.0f)};
        h = h + f16x2{(f16)1536.0f, (f16)1536.0f};
        if (CLAMP) {
            // on the bit patterns: 1536 + code in [1536, 1551] is 0x6600 .. 0x660f; patterns of positive halves order
            // like signed 16-bit integers, negative sums are negative integers, +inf (0x7c00) lies above
            typedef short i16x2 __attribute__((ext_vector_type(2)));
            i16x2 c = __builtin_bit_cast(i16x2, h);
            c = __builtin_elementwise_max(c, i16x2{0x6600, 0x6600});
            c = __builtin_elementwise_min(c, i16x2{0x660f, 0x660f});
            b[i] = __builtin_bit_cast(u32, c);
        } else {
            b[i] = __builtin_bit_cast(u32, h);
        }
    }
    return pack_nibbles8(b);
}
// A vector's minimum decides the sign of a zero `zero` (= -min): a vector that holds both zeros must give the same one in
// every kernel, whatever the order of its reduction.  All minima of the quantisers are therefore taken with the
// hardware's minimum instructions, for which -0 is below +0 (a comparison and a selection returns whichever of two
// zeros stands second): -0.0 if the vector holds one, and +0.0 -- hence zero = -0.0, as -min gives -- if all its zeros are +0.0.
__device__ __forceinline__ f16 min_of_pair(f16x2 v) { return __builtin_fminf16(v[0], v[1]); }
// ranges from which the clamp-free form is exact (see above)
__device__ __forceinline__ bool asym_range_normal(f16 rng) { return rng >= (f16)0.0009765625f; }

// One fp16 vector of 128 values through (HAD) H_128 * hscale and the asymmetric int4 quantiser, by ONE wave, with the
// arithmetic of kv_had128_kernel operation for operation: the same matrix instructions on the same operand layout
// (all 32 columns of the second operand hold this one vector, where that kernel holds 32 vectors), the same rounding
// to fp16, the same minimum / maximum, scale, zero and code forms -- so codes and parameters are the bits that
// kernel writes for the vector.  `piece`: the vector's 16-byte piece number lane % 16 (the caller's load, so that it can
// be in flight early); `stage`: 256 bytes of LDS private to the wave.
// Result, in every lane: W = the 32 code bytes [32 h, 32 h + 32) of the vector for h = lane / 32; sc, zp.
template <bool HAD>
__device__ __forceinline__ void kv_quant_one_vector(u32x4 piece, u32x4* stage, float hscale, u32 (&W)[8], f16& sc, f16& zp) {
    const int lane = threadIdx.x & 63, v = lane & 31, h = lane >> 5;
    if (lane < 16) stage[lane] = piece;
    __builtin_amdgcn_wave_barrier();                               // (LDS operations of one wave execute in order)
    u32 yw[4][4][2];
    if (!HAD) {
#pragma unroll
        for (int jt = 0; jt < 4; ++jt)
#pragma unroll
            for (int qq = 0; qq < 4; ++qq) {
                const u32x2 t = ((const u32x2*)stage)[(4 * jt + qq) * 2 + h];
                yw[jt][qq][0] = t[0];
                yw[jt][qq][1] = t[1];
            }
    } else {
        f16x8 hb[2], hn[2];
#pragma unroll
        for (int o = 0; o < 2; ++o)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const bool neg = (__builtin_popcount(v & (16 * o + 8 * h + e)) & 1) != 0;
                hb[o][e] = neg ? (f16)-1.0f : (f16)1.0f;
                hn[o][e] = neg ? (f16)1.0f : (f16)-1.0f;
            }
        u32x4 xf[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) xf[ks] = stage[2 * ks + h];
        f32x16 acc[4];
#pragma unroll
        for (int jt = 0; jt < 4; ++jt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[jt][r] = 0.f;
#pragma unroll
        for (int jt = 0; jt < 4; ++jt)
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                const bool neg = (__builtin_popcount(jt & (ks >> 1)) & 1) != 0;
                acc[jt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(neg ? hn[ks & 1] : hb[ks & 1], __builtin_bit_cast(f16x8, xf[ks]),
                                                                 acc[jt], 0, 0, 0);
            }
#pragma unroll
        for (int jt = 0; jt < 4; ++jt)
#pragma unroll
            for (int qq = 0; qq < 4; ++qq) {
                yw[jt][qq][0] = narrow_f16x2(acc[jt][4 * qq] * hscale, acc[jt][4 * qq + 1] * hscale);
                yw[jt][qq][1] = narrow_f16x2(acc[jt][4 * qq + 2] * hscale, acc[jt][4 * qq + 3] * hscale);
            }
    }
    __builtin_amdgcn_wave_barrier();
    f16x2 mn2 = as_f16x2(yw[0][0][0]), mx2 = mn2;
    u16x2 am2 = {0, 0};
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
#pragma unroll
        for (int qq = 0; qq < 4; ++qq)
#pragma unroll
            for (int w = 0; w < 2; ++w) {
                mn2 = __builtin_elementwise_min(mn2, as_f16x2(yw[jt][qq][w]));
                mx2 = __builtin_elementwise_max(mx2, as_f16x2(yw[jt][qq][w]));
                am2 = __builtin_elementwise_max(am2, __builtin_bit_cast(u16x2, yw[jt][qq][w] & 0x7fff7fffu));
            }
    const f16 mn0 = min_of_pair(mn2);
    const f16 mx0 = mx2[0] > mx2[1] ? mx2[0] : mx2[1];
    f16x2 pr = {mn0, -mx0};
    const f16x2 other = as_f16x2((u32)__shfl_xor((int)__builtin_bit_cast(u32, pr), 32, 64));
    pr = __builtin_elementwise_min(pr, other);
    const f16 mn = pr[0], mx = -pr[1];
    const bool bad = (am2[0] > am2[1] ? am2[0] : am2[1]) >= 0x7c00u;
    const bool finite = __builtin_amdgcn_ballot_w64(bad) == 0;
    u32 U[8];
    if (finite) {
        f16 rng = narrow_f16((float)mx - (float)mn);
        const f16 floor_ = (f16)1e-5f;
        rng = rng < floor_ ? floor_ : rng;
        sc = narrow_f16((float)rng * (1.0f / 15.0f));
        zp = -mn;
        const FastRecip fr = make_fast_recip((float)sc);
        if (__builtin_amdgcn_ballot_w64(!asym_range_normal(rng)) == 0) {
#pragma unroll
            for (int m = 0; m < 8; ++m) {
                const int jt = m >> 1, q0 = (m & 1) * 2;
                U[m] = asym_codes8_fast<false>(u32x4{yw[jt][q0][0], yw[jt][q0][1], yw[jt][q0 + 1][0], yw[jt][q0 + 1][1]}, zp, fr);
            }
        } else {
#pragma unroll
            for (int m = 0; m < 8; ++m) {
                const int jt = m >> 1, q0 = (m & 1) * 2;
                U[m] = asym_codes8_fast<true>(u32x4{yw[jt][q0][0], yw[jt][q0][1], yw[jt][q0 + 1][0], yw[jt][q0 + 1][1]}, zp, fr);
            }
        }
    } else {
        // a NaN anywhere in the vector makes its range, scale and zero NaN and every code 0; infinities follow the
        // IEEE operations of the reference
        float fmn = __builtin_inff(), fmx = -__builtin_inff();
        bool has_nan = false;
#pragma unroll
        for (int jt = 0; jt < 4; ++jt)
#pragma unroll
            for (int qq = 0; qq < 4; ++qq)
#pragma unroll
                for (int w = 0; w < 2; ++w) {
                    const f16x2 p = as_f16x2(yw[jt][qq][w]);
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        const float t = (float)p[e];
                        has_nan = has_nan || (t != t);
                        fmn = __builtin_fminf(t, fmn);
                        fmx = t > fmx ? t : fmx;
                    }
                }
        const float omn = __shfl_xor(fmn, 32, 64), omx = __shfl_xor(fmx, 32, 64);
        const int other_nan = __shfl_xor((int)has_nan, 32, 64);
        has_nan = has_nan || other_nan != 0;
        fmn = __builtin_fminf(omn, fmn);
        fmx = omx > fmx ? omx : fmx;
        if (has_nan) fmn = fmx = __builtin_nanf("");
        f16 rng = (f16)(fmx - fmn);
        const f16 floor_ = (f16)1e-5f;
        rng = rng < floor_ ? floor_ : rng;
        sc = (f16)(float)((double)(float)rng / 15.0);
        zp = (f16)(-fmn);
        const float s = (float)sc, z = (float)zp;
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            const int jt = m >> 1, q0 = (m & 1) * 2;
            u32 word = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const f16x2 p = as_f16x2(yw[jt][q0 + (i >> 1)][i & 1]);
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const float sh = (float)(f16)((float)p[e] + z);
                    const float r = __builtin_rintf((float)(f16)(sh / s));
                    int code = (int)r;
                    code = code < 0 ? 0 : (code > 15 ? 15 : code);
                    code = (r != r) ? 0 : code;
                    word |= (u32)code << (4 * (2 * i + e));
                }
            }
            U[m] = word;
        }
    }
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        const auto sw = __builtin_amdgcn_permlane32_swap(U[m], U[m + 4], false, false);
        W[2 * m] = __builtin_amdgcn_perm(sw[1], sw[0], 0x05040100u);
        W[2 * m + 1] = __builtin_amdgcn_perm(sw[1], sw[0], 0x07060302u);
    }
}
