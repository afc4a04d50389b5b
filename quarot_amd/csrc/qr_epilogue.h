// Epilogue pieces shared by the GEMM kernels: the row-contiguous store of a wave's output slab and the
// fp16 dequantisation of four accumulators of one token.
#pragma once
#include "qr_common.h"

namespace {

// Row-contiguous output of one wave's 32 x (32 NJ) fp16 slab.  In the accumulator layout a lane owns
// 4 consecutive columns of one row, so a direct store instruction would write 16-byte pieces of 32
// different rows and leave every 128-byte line to be assembled from eight partial writes in L2
// (measured: 2.6x the output bytes written to memory on outputs larger than L2).  Instead the slab
// goes through a wave-private LDS region and leaves as 16 bytes per lane with NJ*4 consecutive lanes
// covering one row segment, i.e. whole lines per instruction.
//   o[jj][gq] = this lane's columns jj*32 + gq*8 + (lane/32)*4 .. +3 of row lane%32.
//   region: 32 * NJ * 8 slots of 8 bytes; the 8-byte slot index within a row is XORed with a key made
//   from the row so that the 32 rows written by one instruction spread over all banks.
//   rows: how many of the slab's 32 rows exist in the output (the last row tile of a token count that
//   is no multiple of the tile height); the others are computed on clamped inputs and not stored.
template <int NJ>
__device__ __forceinline__ void store_slab_rows(u32x2* region, const f16x4 (&o)[NJ][4], int lane, f16* ybase, int N,
                                                int rows = 32) {
    constexpr int U = NJ * 8;                   // 8-byte slots per row
    constexpr int LPR = U / 2;                  // lanes (16 bytes each) per row on the way out
    constexpr int RPP = 64 / LPR;               // rows per store instruction
    const int r = lane & 31, khalf = lane >> 5;
#pragma unroll
    for (int jj = 0; jj < NJ; ++jj)
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
            const int u = jj * 8 + gq * 2 + khalf;
            region[r * U + (u ^ ((r * U / 32) & (U - 1)))] = __builtin_bit_cast(u32x2, o[jj][gq]);
        }
    const u32x4* region16 = (const u32x4*)region;
    const int s = lane % LPR;
#pragma unroll
    for (int pass = 0; pass < 32 / RPP; ++pass) {
        const int rr = lane / LPR + pass * RPP;
        const int key = (rr * U / 32) & (U - 1);
        u32x4 v = region16[rr * LPR + (s ^ (key >> 1))];
        if (key & 1) v = u32x4{v[2], v[3], v[0], v[1]};
        // (nontemporal: the output is not read again by this launch, and written this way it disturbs the operands
        // in L2 less -- measured 1-4 % off whole GEMM launches at 2048 and 32768 tokens, int8 and FP6 kernels alike)
        if (rr < rows) __builtin_nontemporal_store(v, (u32x4*)(ybase + (int64_t)rr * N + s * 8));
    }
}

// Four dequantised outputs of one row: fp16( fp16(sa * sb) * fp16(acc >> 8) ) (+ bias), the three
// (four) fp16 operations as packed instructions on column pairs -- each lane of a packed fp16
// multiply or add rounds exactly like the scalar instruction.
__device__ __forceinline__ f16x4 dequant4(int a0, int a1, int a2, int a3, f16 sa, f16x4 sb, f16x4 bi, bool with_bias) {
    const f16x2 s2 = {sa, sa};
    const f16x2 q01 = as_f16x2(narrow_f16x2((float)(a0 >> 8), (float)(a1 >> 8)));
    const f16x2 q23 = as_f16x2(narrow_f16x2((float)(a2 >> 8), (float)(a3 >> 8)));
    f16x2 y01 = (s2 * f16x2{sb[0], sb[1]}) * q01;
    f16x2 y23 = (s2 * f16x2{sb[2], sb[3]}) * q23;
    if (with_bias) {
        y01 = y01 + f16x2{bi[0], bi[1]};
        y23 = y23 + f16x2{bi[2], bi[3]};
    }
    return f16x4{y01[0], y01[1], y23[0], y23[1]};
}

// the same for accumulators that are exact integers held as fp32 (the FP6 matrix path)
__device__ __forceinline__ f16x4 dequant4_f32(float a0, float a1, float a2, float a3, f16 sa, f16x4 sb, f16x4 bi, bool with_bias) {
    const f16x2 s2 = {sa, sa};
    const f16x2 q01 = as_f16x2(narrow_f16x2(a0, a1));
    const f16x2 q23 = as_f16x2(narrow_f16x2(a2, a3));
    f16x2 y01 = (s2 * f16x2{sb[0], sb[1]}) * q01;
    f16x2 y23 = (s2 * f16x2{sb[2], sb[3]}) * q23;
    if (with_bias) {
        y01 = y01 + f16x2{bi[0], bi[1]};
        y23 = y23 + f16x2{bi[2], bi[3]};
    }
    return f16x4{y01[0], y01[1], y23[0], y23[1]};
}

}  // namespace
