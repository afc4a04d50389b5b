// KV-cache path: per-head Hadamard (optional) + per-vector asymmetric int4 quantise/pack, and the
// inverse dequantiser.  A vector of `dim` halves is spread over dim/8 adjacent lanes, 16 bytes each;
// a wave handles 512/dim vectors, so all global accesses are full-width and coalesced.
#include "qr_kvq.h"

namespace {

constexpr int KT = 256;

template <int MASK>
__device__ __forceinline__ float kv_lane_xor(float v) {
    int i = __builtin_bit_cast(int, v);
    int r;
    if constexpr (MASK == 1) r = __builtin_amdgcn_mov_dpp(i, 0xB1, 0xF, 0xF, true);
    else if constexpr (MASK == 2) r = __builtin_amdgcn_mov_dpp(i, 0x4E, 0xF, 0xF, true);
    else if constexpr (MASK == 4) r = __builtin_amdgcn_ds_swizzle(i, 0x101F);
    else if constexpr (MASK == 8) r = __builtin_amdgcn_mov_dpp(i, 0x128, 0xF, 0xF, true);
    else r = __builtin_amdgcn_ds_swizzle(i, 0x401F);   // MASK == 16
    return __builtin_bit_cast(float, r);
}

template <int MASK>
__device__ __forceinline__ void kv_butterfly(float (&v)[8], int lane) {
    const float sgn = (lane & MASK) != 0 ? -1.0f : 1.0f;     // upper lane of a pair: partner - own
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float p = kv_lane_xor<MASK>(v[e]);
        v[e] = __builtin_fmaf(v[e], sgn, p);
    }
}

template <int MASK>
__device__ __forceinline__ void kv_minmax(float& mn, float& mx) {
    float a = kv_lane_xor<MASK>(mn), b = kv_lane_xor<MASK>(mx);
    mn = __builtin_fminf(a, mn);                                   // (the instruction's minimum: see min_of_pair)
    mx = b > mx ? b : mx;
}

// (min, -max) of a vector as one packed pair, reduced across the vector's lanes with one packed min
template <int MASK>
__device__ __forceinline__ f16x2 kv_pair_min(f16x2 p) {
    int i = __builtin_bit_cast(int, p);
    int r;
    if constexpr (MASK == 1) r = __builtin_amdgcn_mov_dpp(i, 0xB1, 0xF, 0xF, true);
    else if constexpr (MASK == 2) r = __builtin_amdgcn_mov_dpp(i, 0x4E, 0xF, 0xF, true);
    else if constexpr (MASK == 4) r = __builtin_amdgcn_ds_swizzle(i, 0x101F);
    else if constexpr (MASK == 8) r = __builtin_amdgcn_mov_dpp(i, 0x128, 0xF, 0xF, true);
    else r = __builtin_amdgcn_ds_swizzle(i, 0x401F);
    return __builtin_elementwise_min(p, __builtin_bit_cast(f16x2, r));
}

// LG = log2(lanes per vector) = log2(dim) - 3, 1..5
// PAGED (head dimension 128 only): codes and {scale, zero} go straight to the vector's place in the paged
// cache instead of dense arrays.
template <int LG, bool HAD, bool PAGED = false>
__global__ __launch_bounds__(KT) void kv_quant_kernel(const u32x4* __restrict__ x, int64_t nchunks, float hscale,
                                                      u32* __restrict__ q, f16* __restrict__ scale,
                                                      f16* __restrict__ zero, PagedDst pd) {
    const int lane = threadIdx.x & 63;
    constexpr int U = 4;                                 // chunks per thread and turn: their loads are all issued first
    const int64_t stride = (int64_t)gridDim.x * KT * U;  // multiple of 64 > lanes per vector
    for (int64_t c0 = (int64_t)blockIdx.x * KT * U; c0 < nchunks; c0 += stride) {
      u32x4 hps[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
          const int64_t c = c0 + u * KT + threadIdx.x;
          hps[u] = c < nchunks ? __builtin_nontemporal_load(x + c) : u32x4{0, 0, 0, 0};
      }
      u32 outws[U];
      f16 scs[U], zps[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        u32x4 hp = hps[u];                               // the 8 fp16 values to quantise, packed
        if (HAD) {
            float v[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[2 * i] = (float)f16_from_bits((unsigned short)(hp[i] & 0xffffu));
                v[2 * i + 1] = (float)f16_from_bits((unsigned short)(hp[i] >> 16));
            }
#pragma unroll
            for (int h = 1; h < 8; h <<= 1)
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if ((i & h) == 0) {
                        float a = v[i], b = v[i | h];
                        v[i] = a + b;
                        v[i | h] = a - b;
                    }
            if (LG > 0) kv_butterfly<1>(v, lane);
            if (LG > 1) kv_butterfly<2>(v, lane);
            if (LG > 2) kv_butterfly<4>(v, lane);
            if (LG > 3) kv_butterfly<8>(v, lane);
            if (LG > 4) kv_butterfly<16>(v, lane);
#pragma unroll
            for (int i = 0; i < 4; ++i)                  // the transform's fp16 output
                hp[i] = narrow_f16x2(v[2 * i] * hscale, v[2 * i + 1] * hscale);
        }
        u32 outw;
        f16 sc, zp;
        const u32 amax = absmax_bits8(hp);
        if (__builtin_amdgcn_ballot_w64(amax >= 0x7c00u) == 0) {
            // every value in the wave is finite: packed min / max, then the lean code path
            f16x2 mn2 = as_f16x2(hp[0]), mx2 = mn2;
#pragma unroll
            for (int i = 1; i < 4; ++i) {
                mn2 = __builtin_elementwise_min(mn2, as_f16x2(hp[i]));
                mx2 = __builtin_elementwise_max(mx2, as_f16x2(hp[i]));
            }
            const f16 mn0 = min_of_pair(mn2);
            const f16 mx0 = mx2[0] > mx2[1] ? mx2[0] : mx2[1];
            f16x2 pr = {mn0, -mx0};
            if (LG > 0) pr = kv_pair_min<1>(pr);
            if (LG > 1) pr = kv_pair_min<2>(pr);
            if (LG > 2) pr = kv_pair_min<4>(pr);
            if (LG > 3) pr = kv_pair_min<8>(pr);
            if (LG > 4) pr = kv_pair_min<16>(pr);
            const f16 mn = pr[0], mx = -pr[1];
            // scale = max(fp16(max - min), fp16(1e-5)) / 15 ; zero = -min   (each step one fp16 rounding).
            // range / 15 is never within 2^-16 (relative) of an fp16 rounding boundary, so the fp32
            // product with the rounded constant rounds like the exact quotient (checked for every fp16).
            f16 rng = narrow_f16((float)mx - (float)mn);
            const f16 floor_ = (f16)1e-5f;
            rng = rng < floor_ ? floor_ : rng;
            sc = narrow_f16((float)rng * (1.0f / 15.0f));
            zp = -mn;
            const FastRecip fr = make_fast_recip((float)sc);
            if (__builtin_amdgcn_ballot_w64(!asym_range_normal(rng)) == 0) outw = asym_codes8_fast<false>(hp, zp, fr);
            else outw = asym_codes8_fast<true>(hp, zp, fr);
        } else {
            float v[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[2 * i] = (float)f16_from_bits((unsigned short)(hp[i] & 0xffffu));
                v[2 * i + 1] = (float)f16_from_bits((unsigned short)(hp[i] >> 16));
            }
            float mn = v[0], mx = v[0];
            float nan_seen = amax > 0x7c00u ? 1.0f : 0.0f;       // magnitude bits above infinity's: a NaN in this lane
#pragma unroll
            for (int e = 1; e < 8; ++e) {
                mn = __builtin_fminf(v[e], mn);
                mx = v[e] > mx ? v[e] : mx;
            }
            float nan_lo = 0.0f;                                 // (unused minimum of the flag; the maximum is the "any")
            if (LG > 0) { kv_minmax<1>(mn, mx); kv_minmax<1>(nan_lo, nan_seen); }
            if (LG > 1) { kv_minmax<2>(mn, mx); kv_minmax<2>(nan_lo, nan_seen); }
            if (LG > 2) { kv_minmax<4>(mn, mx); kv_minmax<4>(nan_lo, nan_seen); }
            if (LG > 3) { kv_minmax<8>(mn, mx); kv_minmax<8>(nan_lo, nan_seen); }
            if (LG > 4) { kv_minmax<16>(mn, mx); kv_minmax<16>(nan_lo, nan_seen); }
            // torch.amax / amin propagate a NaN: range, scale and zero of that vector are NaN, every code 0
            if (nan_seen != 0.0f) mn = mx = __builtin_nanf("");
            f16 rng = (f16)(mx - mn);
            const f16 floor_ = (f16)1e-5f;
            rng = rng < floor_ ? floor_ : rng;                   // NaN < x is false: NaN stays
            sc = (f16)(float)((double)(float)rng / 15.0);
            zp = (f16)(-mn);
            const float s = (float)sc, z = (float)zp;
            const float rs = 1.0f / s;
            outw = 0;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float sh = (float)(f16)(v[e] + z);
                const float q0 = sh * rs;
                const float er = __builtin_fmaf(-q0, s, sh);
                const float q1 = __builtin_fabsf(q0) < __builtin_inff() ? __builtin_fmaf(er, rs, q0) : q0;
                const float r = __builtin_rintf((float)(f16)q1);
                int code = (int)r;
                code = code < 0 ? 0 : (code > 15 ? 15 : code);
                code = (r != r) ? 0 : code;
                outw |= (u32)code << (4 * e);
            }
        }
        outws[u] = outw;
        scs[u] = sc;
        zps[u] = zp;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
          const int64_t c = c0 + u * KT + threadIdx.x;   // nchunks is a multiple of lanes-per-vector: groups are all-live or all-dead
          if (c < nchunks) {
              if (PAGED) {
                  const int64_t vec = c >> LG, token = vec / pd.c.num_heads;
                  int64_t page;
                  int entry;
                  if (paged_locate(pd.c, pd.append_indptr, token, page, entry)) {
                      const int64_t s = paged_slot(pd.c, page, pd.kv, (int)(vec - token * pd.c.num_heads), entry);
                      ((u32*)pd.c.data)[s * (1 << LG) + (c & ((1 << LG) - 1))] = outws[u];
                      if ((lane & ((1 << LG) - 1)) == 0) pd.c.param[s] = pack_scale_zero(scs[u], zps[u]);
                  }
              } else {
                  __builtin_nontemporal_store(outws[u], q + c);
                  if ((lane & ((1 << LG) - 1)) == 0) {
                      scale[c >> LG] = scs[u];
                      zero[c >> LG] = zps[u];
                  }
              }
          }
      }
    }
}

template <int LG>
__global__ __launch_bounds__(KT) void kv_dequant_kernel(const u32* __restrict__ q, const f16* __restrict__ scale,
                                                        const f16* __restrict__ zero, int64_t nchunks,
                                                        u32x4* __restrict__ y) {
    constexpr int U = 4;                                 // chunks per thread and turn: their loads are all issued first
    const int64_t stride = (int64_t)gridDim.x * KT * U;
    for (int64_t c0 = (int64_t)blockIdx.x * KT * U + threadIdx.x; c0 < nchunks; c0 += stride) {
        u32 ws[U];
        f16 scs[U], zps[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t c = c0 + u * KT;
            const int64_t cc = c < nchunks ? c : nchunks - 1;
            ws[u] = *(q + cc);
            scs[u] = scale[cc >> LG];
            zps[u] = zero[cc >> LG];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t c = c0 + u * KT;
            const u32 w = ws[u];
            const f16 sc = scs[u], zp = zps[u];
            u32x4 o;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const f16 a = (f16)((f16)(float)((w >> (8 * i)) & 0xfu) * sc) - zp;
                const f16 b = (f16)((f16)(float)((w >> (8 * i + 4)) & 0xfu) * sc) - zp;
                o[i] = (u32)f16_bits(a) | ((u32)f16_bits(b) << 16);
            }
            if (c < nchunks) __builtin_nontemporal_store(o, y + c);
        }
    }
}

// ---- head dimension 128 with the Hadamard: the transform on the matrix cores ----------------------
// Seven butterfly stages cost 11.5 vector instructions per element (a cross-lane stage is two
// instructions per element however it is written) and bound the kernel above at ~3 TB/s.  Here a
// wave takes 32 vectors at a time and computes Y^T = H_128 . X^T with v_mfma_f32_32x32x16_f16:
//   * first operand: H_128 tiles (32 outputs j x 16 inputs k).  H[j][k] = (-1)^popcount(j & k) factors
//     by index bits: tile (jt, ks) is a base tile that depends on ks & 1 only, times the wave-uniform
//     sign (-1)^popcount(jt & (ks >> 1)).  Two base tiles and their negations: 16 registers.
//   * second operand: X^T, lane (vector v = lane % 32, half h = lane / 32) supplies 8 consecutive
//     inputs of ITS vector: 16 bytes of the vector's row.  The 8 KB block of 32 rows is fetched with
//     coalesced 16-byte loads one block ahead, staged in a wave-private LDS region (pieces XOR-keyed by
//     the row) and read back as fragments: no workgroup barrier anywhere in the kernel.
//   * result: lane (v, h) holds outputs j = 32 jt + 8 q + 4 h + (0..3) of vector v, i.e. 64 of the 128
//     outputs of one vector (lane ^ 32 holds the others).  Scaling, fp16 rounding, min / max (packed,
//     in-lane, then one exchange with lane ^ 32) and the codes stay in the lane; four
//     v_permlane32_swap then give lane h the 32 contiguous output bytes [32 h, 32 h + 32) of its
//     vector, so a wave writes 2 KB of consecutive codes.
// The fp32 sums are formed in the matrix core's order, not the butterflies': the plain transform of a
// 128-wide row (qr_hadamard, used by matmul_had_cuda) runs through the same kernel (QUANT = false),
// so that codes remain those of the quantiser applied to that transform's output, bit for bit.
constexpr int KM_WAVES = 4;

__device__ __forceinline__ int km_slot(int row, int piece) { return row * 16 + (piece ^ (row & 15)); }

template <bool QUANT, bool PAGED = false>
__global__ __launch_bounds__(64 * KM_WAVES, 2) void kv_had128_kernel(const u32x4* __restrict__ x, int64_t vectors,
                                                                     float hscale, u32x4* __restrict__ q,
                                                                     f16* __restrict__ scale, f16* __restrict__ zero,
                                                                     u32x4* __restrict__ y, PagedDst pd,
                                                                     const u32x4* __restrict__ x2, int plain_mask) {
    __shared__ u32x4 km_lds[KM_WAVES * 512];                       // 8 KB per wave
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int v = lane & 31, h = lane >> 5;
    u32x4* stage = km_lds + wave * 512;

    // base tiles of H_128 for ks even / odd: row j = v (jt = 0), inputs k = 16 (ks & 1) + 8 h + e
    f16x8 hb[2], hn[2];
#pragma unroll
    for (int o = 0; o < 2; ++o)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const bool neg = (__builtin_popcount(v & (16 * o + 8 * h + e)) & 1) != 0;
            hb[o][e] = neg ? (f16)-1.0f : (f16)1.0f;
            hn[o][e] = neg ? (f16)1.0f : (f16)-1.0f;
        }

    // PAGED: a part that is quantised WITHOUT the transform -- the values of an append, or keys when the caller
    // wants none -- skips the matrix stage (its bit in plain_mask), so that keys and values of an append are ONE
    // launch: blocks [0, blocks1) take x, blocks [blocks1, 2 blocks1) take x2 into the value slots.
    const int64_t blocks1 = (vectors + 31) >> 5;
    const int64_t blocks = (PAGED && x2) ? 2 * blocks1 : blocks1;
    const int64_t wstride = (int64_t)gridDim.x * KM_WAVES;
    int64_t blk = (int64_t)blockIdx.x * KM_WAVES + wave;
    // block of 32 rows = 512 pieces of 16 bytes; load c takes pieces 64 c + lane: row 4 c + lane / 16
    u32x4 pre[8];
    auto fetch = [&](int64_t b) {
        const bool second = PAGED && b >= blocks1;
        const u32x4* src = second ? x2 : x;
        if (second) b -= blocks1;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            int64_t row = b * 32 + 4 * c + (lane >> 4);
            row = row < vectors ? row : vectors - 1;               // the last block may be short: repeat its last row
            pre[c] = __builtin_nontemporal_load(src + row * 16 + (lane & 15));     // (streamed once: 70 -> 65.5 us on 268 MB in, then 63 us with the codes leaving as nontemporal stores too)
        }
    };
    // The loop is rotated so that every turn issues the same memory operations in the same order, without a
    // branch around any of them: [fragment reads] [transform, quantiser] [stores of block b] [wait for the loads
    // of block b + 1, issued a turn earlier and therefore OLDER than those stores; stage them] [loads of block
    // b + 2].  The wait then counts the stores as still allowed in flight; with a conditional load or store
    // anywhere in the turn the compiler has to wait for everything, i.e. for the stores' round trip, every turn.
    // (Past the end the last block is fetched again, and rows past the end repeat the last row: their lanes
    // compute the last vector's values once more and store them to the last vector's place.)
    auto stage_in = [&]() {                                        // LDS operations of one wave execute in order:
#pragma unroll                                                     // these writes follow the current block's reads
        for (int c = 0; c < 8; ++c) stage[km_slot(4 * c + (lane >> 4), lane & 15)] = pre[c];
    };
    auto turn_end = [&](int64_t b) {                               // b: the block just finished
        stage_in();
        const int64_t nb = b + 2 * wstride;
        fetch(nb < blocks ? nb : blocks - 1);
    };
    if (blk < blocks) {
        fetch(blk);
        stage_in();
        fetch(blk + wstride < blocks ? blk + wstride : blocks - 1);
    }
    for (; blk < blocks; blk += wstride) {
        const bool second = PAGED && blk >= blocks1;               // wave-uniform
        const bool plain = PAGED && ((plain_mask >> (second ? 1 : 0)) & 1);
        // scaled, rounded outputs: yw[jt][qq] = the four outputs j = 32 jt + 8 qq + 4 h + (0..3), two per word
        u32 yw[4][4][2];
        if (plain) {
            // no transform: the lane's outputs are the staged values themselves (half h of piece 4 jt + qq of row v),
            // taken as they are -- an infinity or NaN stays in its own element, as in the separate quantiser
#pragma unroll
            for (int jt = 0; jt < 4; ++jt)
#pragma unroll
                for (int qq = 0; qq < 4; ++qq) {
                    const u32x2 t = ((const u32x2*)stage)[km_slot(v, 4 * jt + qq) * 2 + h];
                    yw[jt][qq][0] = t[0];
                    yw[jt][qq][1] = t[1];
                }
        } else {
            u32x4 xf[8];
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) xf[ks] = stage[km_slot(v, 2 * ks + h)];
            f32x16 acc[4];
#pragma unroll
            for (int jt = 0; jt < 4; ++jt)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[jt][r] = 0.f;
#pragma unroll
            for (int jt = 0; jt < 4; ++jt)
#pragma unroll
                for (int ks = 0; ks < 8; ++ks) {
                    const bool neg = (__builtin_popcount(jt & (ks >> 1)) & 1) != 0;     // compile-time after unrolling
                    acc[jt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(neg ? hn[ks & 1] : hb[ks & 1],
                                                                     __builtin_bit_cast(f16x8, xf[ks]), acc[jt], 0, 0, 0);
                }
#pragma unroll
            for (int jt = 0; jt < 4; ++jt)
#pragma unroll
                for (int qq = 0; qq < 4; ++qq) {
                    yw[jt][qq][0] = narrow_f16x2(acc[jt][4 * qq] * hscale, acc[jt][4 * qq + 1] * hscale);
                    yw[jt][qq][1] = narrow_f16x2(acc[jt][4 * qq + 2] * hscale, acc[jt][4 * qq + 3] * hscale);
                }
        }
        const int64_t blk1 = second ? blk - blocks1 : blk;
        const int64_t vec = blk1 * 32 + v;
        if (!QUANT) {
            // back through the staging region (all fragment reads are done): 8-byte pieces in, rows out
#pragma unroll
            for (int jt = 0; jt < 4; ++jt)
#pragma unroll
                for (int qq = 0; qq < 4; ++qq) {
                    const int piece = 4 * jt + qq;                 // 16-byte piece of the row; this lane's half h of it
                    ((u32x2*)stage)[km_slot(v, piece) * 2 + h] = u32x2{yw[jt][qq][0], yw[jt][qq][1]};
                }
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const int row = 4 * c + (lane >> 4);
                const u32x4 o = stage[km_slot(row, lane & 15)];
                int64_t grow = blk * 32 + row;
                grow = grow < vectors ? grow : vectors - 1;        // (a repeat of the last row: the same values again)
                y[grow * 16 + (lane & 15)] = o;                    // (plain: as a nontemporal store 81 -> 91 us on 2 x 268 MB)
            }
            turn_end(blk);
            continue;
        }
        // ---- quantiser on the lane's 64 values: packed minimum and maximum first
        f16x2 mn2 = as_f16x2(yw[0][0][0]), mx2 = mn2;
#pragma unroll
        for (int jt = 0; jt < 4; ++jt)
#pragma unroll
            for (int qq = 0; qq < 4; ++qq)
#pragma unroll
                for (int w = 0; w < 2; ++w) {
                    mn2 = __builtin_elementwise_min(mn2, as_f16x2(yw[jt][qq][w]));
                    mx2 = __builtin_elementwise_max(mx2, as_f16x2(yw[jt][qq][w]));
                }
        const f16 mn0 = min_of_pair(mn2);
        const f16 mx0 = mx2[0] > mx2[1] ? mx2[0] : mx2[1];
        f16x2 pr = {mn0, -mx0};                                    // (min, -max): one packed min across the two lanes
        const f16x2 other = as_f16x2((u32)__shfl_xor((int)__builtin_bit_cast(u32, pr), 32, 64));
        pr = __builtin_elementwise_min(pr, other);
        const f16 mn = pr[0], mx = -pr[1];
        // Is every value finite?  Behind the transform that needs no pass over the values: an infinity or NaN in
        // a vector reaches EVERY output of that vector (each is a sum of all 128 inputs times +-1), so one output
        // tells; what is left is a finite sum too large for fp16, and that shows in the minimum or maximum.
        // Appends (parts of which skip the transform) are looked at value by value.
        bool bad;
        if (PAGED) {
            u16x2 am2 = {0, 0};                                    // largest magnitude bits: >= 0x7c00 means inf or NaN
#pragma unroll
            for (int jt = 0; jt < 4; ++jt)
#pragma unroll
                for (int qq = 0; qq < 4; ++qq)
#pragma unroll
                    for (int w = 0; w < 2; ++w)
                        am2 = __builtin_elementwise_max(am2, __builtin_bit_cast(u16x2, yw[jt][qq][w] & 0x7fff7fffu));
            bad = (am2[0] > am2[1] ? am2[0] : am2[1]) >= 0x7c00u;
        } else {
            bad = (yw[0][0][0] & 0x7c00u) == 0x7c00u || (f16_bits(mn) & 0x7fffu) >= 0x7c00u || (f16_bits(mx) & 0x7fffu) >= 0x7c00u;
        }
        const bool finite = __builtin_amdgcn_ballot_w64(bad) == 0;
        f16 sc, zp;
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
            // a NaN anywhere in a vector makes its range, scale and zero NaN and every code 0 (torch's
            // min / max propagate it); infinities follow the IEEE operations of the reference
            float mn = __builtin_inff(), mx = -__builtin_inff();
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
                            mn = __builtin_fminf(t, mn);
                            mx = t > mx ? t : mx;
                        }
                    }
            const float omn = __shfl_xor(mn, 32, 64), omx = __shfl_xor(mx, 32, 64);
            const int other_nan = __shfl_xor((int)has_nan, 32, 64);    // (every lane takes part: behind a short-circuit
            has_nan = has_nan || other_nan != 0;                       //  `||` the lanes that hold the NaN would sit the exchange out)
            mn = __builtin_fminf(omn, mn);
            mx = omx > mx ? omx : mx;
            if (has_nan) mn = mx = __builtin_nanf("");
            f16 rng = (f16)(mx - mn);
            const f16 floor_ = (f16)1e-5f;
            rng = rng < floor_ ? floor_ : rng;                     // NaN < x is false: NaN stays
            sc = (f16)(float)((double)(float)rng / 15.0);
            zp = (f16)(-mn);
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
        // U[m] = (piece 2m, piece 2m + 1) of this lane's sixteen 2-byte pieces; pieces of the two lanes
        // of a vector interleave.  After the swaps lane h holds both lanes' pieces of words 8 h .. 8 h + 7.
        u32 W[8];
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            const auto sw = __builtin_amdgcn_permlane32_swap(U[m], U[m + 4], false, false);
            W[2 * m] = __builtin_amdgcn_perm(sw[1], sw[0], 0x05040100u);
            W[2 * m + 1] = __builtin_amdgcn_perm(sw[1], sw[0], 0x07060302u);
        }
        if (!PAGED) {
            const int64_t vc = vec < vectors ? vec : vectors - 1;  // (lanes past the end hold the last vector's values)
            __builtin_nontemporal_store(u32x4{W[0], W[1], W[2], W[3]}, q + vc * 4 + 2 * h);
            __builtin_nontemporal_store(u32x4{W[4], W[5], W[6], W[7]}, q + vc * 4 + 2 * h + 1);
            scale[vc] = sc;                                        // both lanes of a vector: the same two values
            zero[vc] = zp;
        } else if (vec < vectors) {
            {
                const int64_t token = vec / pd.c.num_heads;
                int64_t page;
                int entry;
                if (paged_locate(pd.c, pd.append_indptr, token, page, entry)) {
                    const int64_t s = paged_slot(pd.c, page, second ? 1 : pd.kv, (int)(vec - token * pd.c.num_heads), entry);
                    u32x4* dst = (u32x4*)pd.c.data + s * 4 + 2 * h;
                    dst[0] = u32x4{W[0], W[1], W[2], W[3]};
                    dst[1] = u32x4{W[4], W[5], W[6], W[7]};
                    if (h == 0) pd.c.param[s] = pack_scale_zero(sc, zp);
                }
            }
        }
        turn_end(blk);
    }
}

template <bool QUANT, bool PAGED = false>
int launch_had128(const void* x, int64_t vectors, float hscale, void* q, void* scale, void* zero, void* y, hipStream_t st,
                  const PagedDst& pd = PagedDst{}, const void* x2 = nullptr, int plain_mask = 0) {
    auto kern = kv_had128_kernel<QUANT, PAGED>;
    const int64_t blocks = ((vectors + 31) >> 5) * (x2 ? 2 : 1);
    const int64_t want = (blocks + KM_WAVES - 1) / KM_WAVES;
    const int64_t cap = (int64_t)qr_device().cus * qr_blocks_per_cu((const void*)kern, 64 * KM_WAVES, 0);
    const unsigned grid = (unsigned)(want < cap ? want : cap);
    kern<<<dim3(grid), dim3(64 * KM_WAVES), 0, st>>>((const u32x4*)x, vectors, hscale, (u32x4*)q, (f16*)scale, (f16*)zero,
                                                    (u32x4*)y, pd, (const u32x4*)x2, plain_mask);
    return qr_launch_status();
}

int log2_dim(int dim) {
    for (int l = 4; l <= 8; ++l)
        if ((1 << l) == dim) return l;
    return -1;
}

unsigned grid_for(int64_t nchunks, int per_block = KT) {
    int64_t b = (nchunks + per_block - 1) / per_block;
    const int64_t cap = 256 * 32;
    return (unsigned)(b < cap ? b : cap);
}

}  // namespace

extern "C" int qr_kv_quant_f16_i4(const void* x, int64_t vectors, int dim, int had_mode, void* q, void* scale,
                                  void* zero, void* stream) {
    if (vectors < 0) return QR_E_SHAPE;
    const int l2 = log2_dim(dim);
    if (l2 < 0) return dim > 0 ? QR_E_UNSUPPORTED : QR_E_SHAPE;
    if (had_mode != 0 && had_mode != 1) return QR_E_DTYPE;
    if (vectors == 0) return QR_OK;
    if (!x || !q || !scale || !zero) return QR_E_NULL;
    if (((uintptr_t)x & 15) || ((uintptr_t)q & 3)) return QR_E_ALIGN;
    const int64_t nchunks = vectors * (dim / 8);
    const float hs = (float)(1.0 / __builtin_sqrt((double)dim));
    hipStream_t st = (hipStream_t)stream;
    if (dim == 128 && had_mode == 1 && (((uintptr_t)q & 15) == 0))
        return launch_had128<true>(x, vectors, hs, q, scale, zero, nullptr, st);
    dim3 grid(grid_for(nchunks, 4 * KT)), block(KT);
#define QR_KV(LG)                                                                                                     \
    case LG + 3:                                                                                                      \
        if (had_mode)                                                                                                 \
            kv_quant_kernel<LG, true><<<grid, block, 0, st>>>((const u32x4*)x, nchunks, hs, (u32*)q, (f16*)scale,     \
                                                              (f16*)zero, PagedDst{});                                \
        else                                                                                                          \
            kv_quant_kernel<LG, false><<<grid, block, 0, st>>>((const u32x4*)x, nchunks, hs, (u32*)q, (f16*)scale,    \
                                                               (f16*)zero, PagedDst{});                               \
        break;
    switch (l2) {
        QR_KV(1) QR_KV(2) QR_KV(3) QR_KV(4) QR_KV(5)
    }
#undef QR_KV
    return qr_launch_status();
}

// The plain transform of 128-wide fp16 rows with the arithmetic of the fused kernel (see above).
__attribute__((visibility("hidden"))) int qr_internal_hadamard128_f16(const void* x, void* y, int64_t rows, float scale,
                                                                      hipStream_t st) {
    return launch_had128<false>(x, rows, scale, nullptr, nullptr, nullptr, y, st);
}

extern "C" int qr_kv_dequant_i4_f16(const void* q, const void* scale, const void* zero, int64_t vectors, int dim,
                                    void* y, void* stream) {
    if (vectors < 0) return QR_E_SHAPE;
    const int l2 = log2_dim(dim);
    if (l2 < 0) return dim > 0 ? QR_E_UNSUPPORTED : QR_E_SHAPE;
    if (vectors == 0) return QR_OK;
    if (!q || !scale || !zero || !y) return QR_E_NULL;
    if (((uintptr_t)y & 15) || ((uintptr_t)q & 3)) return QR_E_ALIGN;
    const int64_t nchunks = vectors * (dim / 8);
    hipStream_t st = (hipStream_t)stream;
    dim3 grid(grid_for(nchunks, 4 * KT)), block(KT);
    switch (l2 - 3) {
        case 1: kv_dequant_kernel<1><<<grid, block, 0, st>>>((const u32*)q, (const f16*)scale, (const f16*)zero, nchunks, (u32x4*)y); break;
        case 2: kv_dequant_kernel<2><<<grid, block, 0, st>>>((const u32*)q, (const f16*)scale, (const f16*)zero, nchunks, (u32x4*)y); break;
        case 3: kv_dequant_kernel<3><<<grid, block, 0, st>>>((const u32*)q, (const f16*)scale, (const f16*)zero, nchunks, (u32x4*)y); break;
        case 4: kv_dequant_kernel<4><<<grid, block, 0, st>>>((const u32*)q, (const f16*)scale, (const f16*)zero, nchunks, (u32x4*)y); break;
        case 5: kv_dequant_kernel<5><<<grid, block, 0, st>>>((const u32*)q, (const f16*)scale, (const f16*)zero, nchunks, (u32x4*)y); break;
    }
    return qr_launch_status();
}

// Quantise new K and V vectors and write them straight into their pages: what
// MultiLayerPagedKVCache4Bit.update does with matmul_had_cuda, asym_quantize_and_pack_i4 (twice), two
// torch.cat and init_kv_i4 / append_kv_i4 (quarot/transformers/kv_cache.py:174-251), as one launch.
extern "C" int qr_kv_quant_append_f16_i4(const void* k, const void* v, int64_t tokens, const void* append_indptr_or_null,
                                         int k_had_mode, void* kv_data, void* kv_param, const void* kv_indptr,
                                         const void* kv_indices, const void* last_page_offset, int64_t num_pages,
                                         int num_layers, int layer_idx, int num_heads, int page_size, int head_dim,
                                         int64_t batch_size, void* stream) {
    if (tokens < 0 || num_pages < 0 || num_layers <= 0 || layer_idx < 0 || layer_idx >= num_layers || num_heads <= 0 ||
        page_size <= 0 || batch_size < 0 || batch_size > 0x7fffffff || head_dim <= 0)
        return QR_E_SHAPE;
    if (head_dim != 128) return QR_E_UNSUPPORTED;
    if (k_had_mode != 0 && k_had_mode != 1) return QR_E_DTYPE;
    if (batch_size == 0 || tokens == 0) return QR_OK;
    if (!append_indptr_or_null && tokens != batch_size) return QR_E_SHAPE;
    if (!k || !v || !kv_data || !kv_param || !kv_indptr || !kv_indices || !last_page_offset) return QR_E_NULL;
    if (((uintptr_t)k & 15) || ((uintptr_t)v & 15) || ((uintptr_t)kv_data & 15) || ((uintptr_t)kv_param & 3)) return QR_E_ALIGN;
    PagedDst pd;
    pd.c = qr_internal_paged_kv(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, num_pages, num_layers, layer_idx,
                                num_heads, page_size, batch_size);
    pd.append_indptr = (const int32_t*)append_indptr_or_null;
    const int64_t vectors = tokens * num_heads;
    const float hs = (float)(1.0 / __builtin_sqrt(128.0));
    hipStream_t st = (hipStream_t)stream;
    // keys (through H_128, or as they are when the caller wants them untransformed) and values (as they are) in
    // ONE launch of the matrix-core kernel: bit for bit the codes, scales and zeros of the separate quantisers
    pd.kv = 0;
    return launch_had128<true, true>(k, vectors, hs, nullptr, nullptr, nullptr, nullptr, st, pd, v, k_had_mode ? 2 : 3);
}
