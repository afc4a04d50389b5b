// int4 x int4 -> int32 GEMM on the gfx950 int8 matrix cores, with an optional fused fp16 dequant
// epilogue.  C[M, N] = unpack(A)[M, K] . unpack(B)[N, K]^T, both operands K-contiguous, packed two
// nibbles per byte (even k in the low nibble).
//
// Feeding int4 to an int8 MFMA without sign extension: for a 32-bit word p holding 8 nibbles,
//     lo = (p << 4) & 0xF0F0F0F0   holds 16 * v[even k] in each byte (as a signed int8)
//     hi =  p       & 0xF0F0F0F0   holds 16 * v[odd k]
// Both operands are scaled by 16, so every product is 256 * a * b and the accumulator is exactly
// 256 * (the int4 dot product); an arithmetic shift by 8 at the end restores it.  Even and odd k
// go to different MFMA issues; that permutation of k is the same for A and B, so dot products are
// unchanged.  |acc| <= 256 * 64 * K requires K < 131072.
//
// The MFMA's first operand is the W (B-matrix) fragment and its second the X (A-matrix) fragment,
// so in the 32x32 accumulator a lane owns one token (m = lane % 32) and runs of 4 consecutive
// output features n: stores are 8 bytes (fp16) or 16 bytes (int32) per lane.
//
// Issue budget: a 32x32x32 int8 MFMA occupies the matrix pipe for 32 cycles and a wave's VALU op
// takes 4; measured on MI355X, up to ~5 VALU ops per MFMA are hidden.  Unpacking costs 3 VALU ops per
// packed dword, i.e. 6 (IM + JN) / (IM JN) per MFMA for a wave tile of IM x JN MFMA tiles: 64x128 per
// wave (4.5) is the smallest tile that fits.  To still run two waves per SIMD on a 128x256 workgroup
// tile (one tile per CU at M = 2048, N = 4096), eight waves are arranged as 2 (M) x 2 (N) x 2 (K): the
// two K-groups take alternate 64-k sub-steps of every stage and exchange half of their accumulators
// through LDS at the end.
#include "qr_common.h"
#include "qr_epilogue.h"
#include <type_traits>

namespace {

// LDS holds, per stage, (BM + BN) rows of 64 packed bytes (128 k values) as four 16-byte chunks.
// The chunk position is XOR-swizzled with bits 2..3 of the row so that the 16 rows a quarter-wave
// reads in one ds_read_b128 beat fall in 16 different 16-byte bank groups.
__device__ __forceinline__ int lds_slot(int row, int chunk) { return row * 4 + (chunk ^ ((row >> 2) & 3)); }

template <int BM, int BN, int WAVES_M, int WAVES_N, bool DEQ>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_i4_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, int M, int N, int Kb, int32_t* __restrict__ C,
    f16* __restrict__ Y, const f16* __restrict__ sA, const f16* __restrict__ sB, const f16* __restrict__ bias,
    int tiles_m, int tiles_n, int nxcd) {
    constexpr int NT = 64 * WAVES_M * WAVES_N;              // threads per workgroup
    constexpr int TM = BM / WAVES_M, TN = BN / WAVES_N;     // per-wave output tile
    constexpr int IM = TM / 32, JN = TN / 32;               // 32x32 MFMA tiles per wave
    constexpr int CH = (BM + BN) * 4;                       // 16-byte chunks per stage
    constexpr int NL = (CH + NT - 1) / NT;                  // chunks each thread moves per stage
    static_assert(TM % 32 == 0 && TN % 32 == 0, "tile shape");
    // two stage buffers; the same memory later stages the fp16 output slabs (one per wave)
    constexpr int SLAB = 32 * 64 * 2 / 16;                  // 16-byte units of a 32-row x 64-column fp16 slab
    static_assert(2 * CH >= WAVES_M * WAVES_N * SLAB, "output slabs must fit in the stage buffers");
    __shared__ u32x4 lds_raw[2 * CH];
    u32x4(*lds)[CH] = (u32x4(*)[CH])lds_raw;

    // Workgroups are dealt round-robin to the nxcd XCDs (each with its own L2).  Give every XCD a
    // contiguous range of tile ids, and walk tiles in groups of GROUP_M rows so that the tiles in
    // flight on one XCD share A rows and B rows.
    const int per_xcd = gridDim.x / nxcd;
    int tile = (blockIdx.x % nxcd) * per_xcd + blockIdx.x / nxcd;
    if (tile >= tiles_m * tiles_n) return;
    constexpr int GROUP_M = 8;
    const int group_sz = GROUP_M * tiles_n;
    const int g = tile / group_sz;
    const int gm0 = g * GROUP_M;
    const int gh = (tiles_m - gm0) < GROUP_M ? (tiles_m - gm0) : GROUP_M;
    const int tm = gm0 + (tile - g * group_sz) % gh;
    const int tn = (tile - g * group_sz) / gh;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    // Global -> LDS staging: chunk id = tid + i * NT; 4 consecutive threads fetch one row's 64 bytes.
    // Rows beyond M (or N) are clamped to the last valid row: they are read but never stored.
    const uint8_t* src[NL];
    int dst[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        int qid = tid + i * NT;
        if (qid >= CH) qid = CH - 1;        // CH not a multiple of NT: the tail repeats the last chunk
        const int row = qid >> 2, c = qid & 3;
        if (row < BM) {
            int gr = m0 + row;
            gr = gr < M ? gr : M - 1;
            src[i] = A + (int64_t)gr * Kb + c * 16;
        } else {
            int gr = n0 + row - BM;
            gr = gr < N ? gr : N - 1;
            src[i] = B + (int64_t)gr * Kb + c * 16;
        }
        dst[i] = lds_slot(row, c);
    }

    i32x16 acc[IM][JN];
#pragma unroll
    for (int i = 0; i < IM; ++i)
#pragma unroll
        for (int j = 0; j < JN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

    const int arow = wm * TM + (lane & 31);
    const int brow = BM + wn * TN + (lane & 31);
    const int khalf = lane >> 5;

    // One stage = 64 packed bytes per row = two sub-steps of 64 k values (two MFMA issues each).
    auto compute = [&](const u32x4* buf, int nsub) {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            if (s < nsub) {
                i32x4 alo[IM], ahi[IM], blo[JN], bhi[JN];
#pragma unroll
                for (int i = 0; i < IM; ++i) {
                    u32x4 p = buf[lds_slot(arow + i * 32, s * 2 + khalf)];
                    alo[i] = (i32x4)((p << 4) & 0xF0F0F0F0u);
                    ahi[i] = (i32x4)(p & 0xF0F0F0F0u);
                }
#pragma unroll
                for (int j = 0; j < JN; ++j) {
                    u32x4 p = buf[lds_slot(brow + j * 32, s * 2 + khalf)];
                    blo[j] = (i32x4)((p << 4) & 0xF0F0F0F0u);
                    bhi[j] = (i32x4)(p & 0xF0F0F0F0u);
                }
                // all even-k issues first, then all odd-k ones: consecutive MFMAs never share an accumulator
#pragma unroll
                for (int i = 0; i < IM; ++i)
#pragma unroll
                    for (int j = 0; j < JN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(blo[j], alo[i], acc[i][j], 0, 0, 0);
#pragma unroll
                for (int i = 0; i < IM; ++i)
#pragma unroll
                    for (int j = 0; j < JN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bhi[j], ahi[i], acc[i][j], 0, 0, 0);
            }
        }
    };

    // K % 64 == 0, so a row is a whole number of 32-byte half-stages: `full` whole stages, then
    // possibly one half stage (chunks 0 and 1 only).
    const int full = Kb / 64;
    const bool half_tail = (Kb & 63) != 0;
    // Global loads run TWO stages ahead of the MFMAs (HBM/L2 latency exceeds one stage of compute):
    // stage ks+2 is requested into one register set at the top of iteration ks, while the other
    // set (stage ks+1, requested an iteration earlier) is written to LDS at the bottom.
    u32x4 preA[NL], preB[NL];
    if (full > 0) {
#pragma unroll
        for (int i = 0; i < NL; ++i) preA[i] = *(const u32x4*)(src[i]);
#pragma unroll
        for (int i = 0; i < NL; ++i) lds[0][dst[i]] = preA[i];
    }
    if (full > 1) {
#pragma unroll
        for (int i = 0; i < NL; ++i) preA[i] = *(const u32x4*)(src[i] + 64);      // stage 1
    }
    __syncthreads();
    auto iteration = [&](int ks, u32x4(&cur)[NL], u32x4(&nxt)[NL]) {
        // `cur` holds stage ks+1 (in flight or landed); `nxt` receives stage ks+2
        if (ks + 2 < full) {
#pragma unroll
            for (int i = 0; i < NL; ++i) nxt[i] = *(const u32x4*)(src[i] + (int64_t)(ks + 2) * 64);
        }
        compute(lds[ks & 1], 2);
        if (ks + 1 < full) {
#pragma unroll
            for (int i = 0; i < NL; ++i) lds[(ks + 1) & 1][dst[i]] = cur[i];
        }
        __syncthreads();
    };
    {
        int ks = 0;
        for (; ks + 1 < full; ks += 2) {
            iteration(ks, preA, preB);
            iteration(ks + 1, preB, preA);
        }
        if (ks < full) iteration(ks, preA, preB);
    }
#pragma unroll
    for (int i = 0; i < NL; ++i) src[i] += (int64_t)(full > 0 ? full - 1 : 0) * 64;   // last full stage
    if (half_tail) {
        // chunks 2 and 3 of this last stage lie beyond the row: only chunks 0/1 are fetched and used
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            int qid = tid + i * NT;
            if (qid >= CH) qid = CH - 1;
            if ((qid & 3) < 2) lds[0][dst[i]] = *(const u32x4*)(src[i] + (full > 0 ? 64 : 0));
        }
        __syncthreads();
        compute(lds[0], 1);
    }

    // Epilogue.  Accumulator layout (first operand = W rows, second = X rows): lane l, register v ->
    // n = (v/4)*8 + (l/32)*4 + v%4, m = l%32.
    // Tiles of an fp16 output whose columns all exist leave as full rows through LDS, 64 columns (one
    // line) at a time; a last row tile stores the rows that exist.
    const bool by_rows = DEQ && n0 + BN <= N && (N & 7) == 0 && (((uintptr_t)Y) & 15) == 0;
    if (DEQ && by_rows) {
        constexpr int NJ = JN > 2 ? 2 : JN;                 // MFMA tiles per slab
        __syncthreads();                                    // every wave is done with the stage buffers
#pragma unroll
        for (int jb = 0; jb < JN; jb += NJ) {
            f16x4 sbh[NJ][4], bih[NJ][4];
#pragma unroll
            for (int jj = 0; jj < NJ; ++jj)
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    const int col = n0 + wn * TN + (jb + jj) * 32 + gq * 8 + khalf * 4;
                    sbh[jj][gq] = *(const f16x4*)(sB + col);
                    bih[jj][gq] = bias ? *(const f16x4*)(bias + col) : f16x4{(f16)0, (f16)0, (f16)0, (f16)0};
                }
#pragma unroll
            for (int i = 0; i < IM; ++i) {
                const int row0 = m0 + wm * TM + i * 32;       // (rows past M: computed on a clamped scale, not stored)
                if (row0 >= M) continue;
                const f16 sa = sA[min(row0 + (lane & 31), M - 1)];
                f16x4 o[NJ][4];
#pragma unroll
                for (int jj = 0; jj < NJ; ++jj)
#pragma unroll
                    for (int gq = 0; gq < 4; ++gq)
                        o[jj][gq] = dequant4(acc[i][jb + jj][gq * 4], acc[i][jb + jj][gq * 4 + 1], acc[i][jb + jj][gq * 4 + 2],
                                             acc[i][jb + jj][gq * 4 + 3], sa, sbh[jj][gq], bih[jj][gq], bias != nullptr);
                store_slab_rows<NJ>((u32x2*)(lds_raw + wave * SLAB), o, lane,
                                    Y + (int64_t)row0 * N + n0 + wn * TN + jb * 32, N, M - row0);
            }
        }
        return;
    }
    // column scales (and bias) of this lane's 4-column groups, fetched up front as 8-byte vectors
    f16x4 sb4[JN][4], bi4[JN][4];
    if (DEQ) {
#pragma unroll
        for (int j = 0; j < JN; ++j)
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const int col = n0 + wn * TN + j * 32 + gq * 8 + khalf * 4;
                if (col + 4 <= N && (N & 3) == 0) {
                    sb4[j][gq] = *(const f16x4*)(sB + col);
                    if (bias) bi4[j][gq] = *(const f16x4*)(bias + col);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int cc = col + e < N ? col + e : N - 1;
                        sb4[j][gq][e] = sB[cc];
                        if (bias) bi4[j][gq][e] = bias[cc];
                    }
                }
            }
    }
#pragma unroll
    for (int i = 0; i < IM; ++i) {
        const int row = m0 + wm * TM + i * 32 + (lane & 31);
        if (row >= M) continue;
        f16 sa = (f16)0;
        if (DEQ) sa = sA[row];
#pragma unroll
        for (int j = 0; j < JN; ++j) {
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const int col = n0 + wn * TN + j * 32 + gq * 8 + khalf * 4;
                if (col >= N) continue;
                int v4[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v4[e] = acc[i][j][gq * 4 + e] >> 8;
                const bool whole = (col + 4 <= N) && ((N & 3) == 0);
                if (DEQ) {
                    f16 o[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        f16 yv = (f16)(sa * sb4[j][gq][e]) * (f16)(float)v4[e];
                        if (bias) yv = yv + bi4[j][gq][e];
                        o[e] = yv;
                    }
                    f16* yp = Y + (int64_t)row * N + col;
                    if (whole) {
                        *(f16x4*)yp = f16x4{o[0], o[1], o[2], o[3]};
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (col + e < N) yp[e] = o[e];
                    }
                } else {
                    int32_t* cp = C + (int64_t)row * N + col;
                    if (whole) {
                        *(i32x4*)cp = i32x4{v4[0], v4[1], v4[2], v4[3]};
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (col + e < N) cp[e] = v4[e];
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Compute-bound shapes (M > 64): 128x256 workgroup tile, eight waves as 2 (M) x 2 (N) x 2 (K).
//
// Both K-groups own the same 64x128 wave tiles and split every 128-k stage between them (group g
// takes the 64-k sub-step g); they exchange half of their accumulators through LDS at the end.
// The two waves that share a SIMD belong to different K-groups and run half an iteration out of
// phase: group 0 reads and unpacks its fragments and then multiplies, group 1 first multiplies the
// operands it unpacked during the previous iteration and then reads and unpacks the next ones.  So
// on every SIMD one wave's unpacking (VALU) runs under the other wave's MFMAs instead of both
// unpacking, then both multiplying.  A stage is 256 k (a full 128-byte line per row, so every line
// fetched from L2 is used whole); three LDS stages rotate (group 1 reads one stage ahead of group
// 0), global loads run one more stage ahead through registers, one barrier per stage.
// (A variant in which half the waves only unpacked into int8 planes in LDS for the other half was
// measured LDS-bound: twice the LDS bytes at ~128 B/clk/CU exceed the MFMA time.)
template <int BM, int BN, int WAVES_M, int WAVES_N, bool DEQ>
__global__ __launch_bounds__(128 * WAVES_M * WAVES_N) void gemm_ks_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, int M, int N, int Kb, int32_t* __restrict__ C,
    f16* __restrict__ Y, const f16* __restrict__ sA, const f16* __restrict__ sB, const f16* __restrict__ bias,
    int tiles_m, int tiles_n, int ksplit, int nxcd) {
    constexpr int NT = 128 * WAVES_M * WAVES_N;
    constexpr int TM = BM / WAVES_M, TN = BN / WAVES_N;
    constexpr int IM = TM / 32, JN = TN / 32;
    // ksplit > 1 (int32 output only): the stages of K are divided among ksplit workgroups per tile;
    // slice s writes its partial sums to the s-th [M, N] slab of C, and a second kernel adds the slabs
    // (atomic adds into one slab were measured 3-4x slower than the whole unsplit product).
    // A stage is 128 packed bytes (256 k) per row = one full cache line, eight 16-byte chunks,
    // four 64-k sub-steps; K-group g multiplies sub-steps 2g and 2g+1.
    constexpr int CH = (BM + BN) * 8;
    constexpr int NL = CH / NT;
    constexpr int NBUF = 3;
    constexpr int JH = JN / 2;
    static_assert(CH % NT == 0 && JN % 2 == 0, "tile shape");
    extern __shared__ u32x4 ks_lds[];                       // [NBUF][CH]; later the accumulator exchange

    const int per_xcd = gridDim.x / nxcd;
    const int unit = (blockIdx.x % nxcd) * per_xcd + blockIdx.x / nxcd;
    if (unit >= tiles_m * tiles_n * ksplit) return;
    const int tile = unit / ksplit, split = unit - tile * ksplit;   // the slices of a tile are neighbours in L2
    constexpr int GROUP_M = 8;
    const int group_sz = GROUP_M * tiles_n;
    const int g = tile / group_sz;
    const int gm0 = g * GROUP_M;
    const int gh = (tiles_m - gm0) < GROUP_M ? (tiles_m - gm0) : GROUP_M;
    const int tm = gm0 + (tile - g * group_sz) % gh;
    const int tn = (tile - g * group_sz) / gh;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kg = wave / (WAVES_M * WAVES_N);
    const int wxy = wave % (WAVES_M * WAVES_N);
    const int wm = wxy / WAVES_N, wn = wxy % WAVES_N;
    const int khalf = lane >> 5;
    const int all_stages = (Kb + 127) / 128;
    if (ksplit > 1) C += (int64_t)split * M * N;
    const int s_first = (int)((int64_t)all_stages * split / ksplit);
    const int stages = (int)((int64_t)all_stages * (split + 1) / ksplit) - s_first;   // >= 1: ksplit <= all_stages
    // chunk position within a row is XOR-swizzled with (row >> 1) & 7: the 16 rows a quarter-wave
    // reads at one logical chunk cover all sixteen 16-byte bank groups (row parity picks the half)
    auto slot8 = [](int row, int chunk) { return row * 8 + (chunk ^ ((row >> 1) & 7)); };

    // ---- staging (all threads): chunk id = tid + i * NT, eight consecutive threads fetch one row's line.
    // Thread-invariant parts are kept out of registers: the rows of a thread's chunks differ by
    // multiples of 64 (same swizzle), so LDS slots differ by compile-time constants.
    static_assert(NT == 512 && BM % 64 == 0 && BN % 64 == 0, "staging layout");
    const int srow = tid >> 3;
    const int scoff = (tid & 7) * 16;
    const int dst0 = slot8(srow, tid & 7);
    u32 goff[NL];                                           // byte offset of the row from A (i < BM/64) or B
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int row = srow + i * 64;
        int gr = row < BM ? m0 + row : n0 + row - BM;
        const int lim = row < BM ? M - 1 : N - 1;
        gr = gr < lim ? gr : lim;
        goff[i] = (u32)gr * (u32)Kb;
    }
    // branch-free loads: a stage past the end repeats the last one; chunks beyond the row end of a
    // partly filled last stage re-read the stage's first chunk and are zeroed when written to LDS
    const bool ragged = (Kb & 127) != 0;
    auto fetch = [&](int st, u32x4(&r)[NL]) {
        const int kb = (s_first + (st < stages ? st : stages - 1)) * 128;
        const u32 off = (u32)((kb + scoff < Kb) ? kb + scoff : kb);
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            if (i * 64 < BM) r[i] = *(const u32x4*)(A + (size_t)(goff[i] + off));
            else r[i] = *(const u32x4*)(B + (size_t)(goff[i] + off));
        }
    };
    auto deposit = [&](int st, int buf, u32x4(&r)[NL]) {
        if (st < stages) {
            if (ragged && (s_first + st) * 128 + scoff >= Kb) {
#pragma unroll
                for (int i = 0; i < NL; ++i) r[i] = u32x4{0, 0, 0, 0};
            }
            u32x4* base = ks_lds + buf * CH + dst0;
#pragma unroll
            for (int i = 0; i < NL; ++i) base[i * 64 * 8] = r[i];
        }
    };
    i32x16 acc[IM][JN];
#pragma unroll
    for (int i = 0; i < IM; ++i)
#pragma unroll
        for (int j = 0; j < JN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

    // this wave's fragment slots for its two sub-steps (u = 0, 1): logical chunk (2 kg + u) * 2 + khalf;
    // tile rows differ by multiples of 32 (same swizzle): compile-time offsets
    int aslot[2], bslot[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        aslot[u] = slot8(wm * TM + (lane & 31), (2 * kg + u) * 2 + khalf);
        bslot[u] = slot8(BM + wn * TN + (lane & 31), (2 * kg + u) * 2 + khalf);
    }
    struct Ops {
        i32x4 alo[IM], ahi[IM], blo[JN], bhi[JN];
    };
    auto load_ops = [&](int buf, int u, Ops& o) {
        const u32x4* pa = ks_lds + buf * CH + (u ? aslot[1] : aslot[0]);
        const u32x4* pb = ks_lds + buf * CH + (u ? bslot[1] : bslot[0]);
#pragma unroll
        for (int i = 0; i < IM; ++i) {
            const u32x4 p = pa[i * 32 * 8];
            o.alo[i] = (i32x4)((p << 4) & 0xF0F0F0F0u);
            o.ahi[i] = (i32x4)(p & 0xF0F0F0F0u);
        }
#pragma unroll
        for (int j = 0; j < JN; ++j) {
            const u32x4 p = pb[j * 32 * 8];
            o.blo[j] = (i32x4)((p << 4) & 0xF0F0F0F0u);
            o.bhi[j] = (i32x4)(p & 0xF0F0F0F0u);
        }
    };
    auto multiply = [&](const Ops& o) {
        // all even-k issues first, then all odd-k ones: consecutive MFMAs never share an accumulator
#pragma unroll
        for (int i = 0; i < IM; ++i)
#pragma unroll
            for (int j = 0; j < JN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.blo[j], o.alo[i], acc[i][j], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < IM; ++i)
#pragma unroll
            for (int j = 0; j < JN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.bhi[j], o.ahi[i], acc[i][j], 0, 0, 0);
    };

    Ops ops;
    int bcur = 0;
    // Global loads run one stage ahead of the LDS fill: stage ks+2 is written to LDS during
    // iteration ks from registers requested at the end of iteration ks-1.  The first three stages
    // are requested together: the accumulators are not live yet, so two more register sets are
    // free, and the prologue costs one memory round trip instead of three.
    u32x4 regs[NL];
    {
        u32x4 first[NL], second[NL];
        fetch(0, first);
        fetch(1, second);
        fetch(2, regs);
        deposit(0, 0, first);
        deposit(1, 1, second);
    }
    __syncthreads();                                    // stages 0 and 1 visible
    if (kg == 1) load_ops(0, 0, ops);                   // group 1 starts one unpack ahead
    for (int ks = 0; ks < stages; ++ks) {
        const int bnext = bcur == NBUF - 1 ? 0 : bcur + 1;
        const int bfill = bnext == NBUF - 1 ? 0 : bnext + 1;
        if (kg == 0) {
            load_ops(bcur, 0, ops);
            multiply(ops);
            load_ops(bcur, 1, ops);
            multiply(ops);
        } else {
            multiply(ops);                              // sub-step 2 of this stage (unpacked earlier)
            load_ops(bcur, 1, ops);
            multiply(ops);                              // sub-step 3
            if (ks + 1 < stages) load_ops(bnext, 0, ops);   // next stage's sub-step 2
        }
        deposit(ks + 2, bfill, regs);
        fetch(ks + 3, regs);
        __syncthreads();
        bcur = bnext;
    }

    // K-split: group 0 finalises the lower half of the j tiles and group 1 the upper half; each sends
    // the other half across, one row of MFMA tiles (i) per round, four 16-byte pieces per lane.
    const int j_first = kg * JH;
    {
        u32x4* xbuf = ks_lds;
        const int send0 = (1 - kg) * JH;
        for (int i = 0; i < IM; ++i) {
            __syncthreads();
#pragma unroll
            for (int jj = 0; jj < JH; ++jj)
#pragma unroll
                for (int qv = 0; qv < 4; ++qv) {
                    const int slot = (((wxy * 2 + (1 - kg)) * JH + jj) * 4 + qv) * 64 + lane;
                    i32x4 piece;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        int val = 0;
#pragma unroll
                        for (int ii = 0; ii < IM; ++ii)
#pragma unroll
                            for (int jx = 0; jx < JN; ++jx)
                                if (ii == i && jx == send0 + jj) val = acc[ii][jx][qv * 4 + e];
                        piece[e] = val;
                    }
                    xbuf[slot] = (u32x4)piece;
                }
            __syncthreads();
#pragma unroll
            for (int jj = 0; jj < JH; ++jj)
#pragma unroll
                for (int qv = 0; qv < 4; ++qv) {
                    const int slot = (((wxy * 2 + kg) * JH + jj) * 4 + qv) * 64 + lane;
                    const i32x4 piece = (i32x4)xbuf[slot];
#pragma unroll
                    for (int ii = 0; ii < IM; ++ii)
#pragma unroll
                        for (int jx = 0; jx < JN; ++jx)
                            if (ii == i && jx == j_first + jj) {
#pragma unroll
                                for (int e = 0; e < 4; ++e) acc[ii][jx][qv * 4 + e] += piece[e];
                            }
                }
        }
    }

    // Epilogue: lane l, register v -> n = (v/4)*8 + (l/32)*4 + v%4, m = l%32.
    // column scales (and bias) of this lane's 4-column groups, fetched up front as 8-byte vectors
    f16x4 sb4[JH][4], bi4[JH][4];                          // only the j tiles this K-group stores
    if (DEQ) {
#pragma unroll
        for (int jj = 0; jj < JH; ++jj)
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const int col = n0 + wn * TN + (j_first + jj) * 32 + gq * 8 + khalf * 4;
                if (col + 4 <= N && (N & 3) == 0) {
                    sb4[jj][gq] = *(const f16x4*)(sB + col);
                    if (bias) bi4[jj][gq] = *(const f16x4*)(bias + col);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int cc = col + e < N ? col + e : N - 1;
                        sb4[jj][gq][e] = sB[cc];
                        if (bias) bi4[jj][gq][e] = bias[cc];
                    }
                }
            }
    }
    // tiles of an fp16 output whose columns all exist leave as full rows through LDS (each K-group its 64 columns)
    const bool by_rows = DEQ && n0 + BN <= N && (N & 7) == 0 && (((uintptr_t)Y) & 15) == 0;
    if (DEQ && by_rows) __syncthreads();                    // the exchange buffers are no longer read
#pragma unroll
    for (int i = 0; i < IM; ++i) {
        const int row = m0 + wm * TM + i * 32 + (lane & 31);
        if (DEQ && by_rows) {
            const int row0 = m0 + wm * TM + i * 32;           // (rows past M: computed on a clamped scale, not stored)
            if (row0 >= M) continue;
            const f16 sa = sA[min(row, M - 1)];
            f16x4 o[JH][4];
#pragma unroll
            for (int j = 0; j < JN; ++j) {
                if (j < j_first || j >= j_first + JH) continue;
#pragma unroll
                for (int gq = 0; gq < 4; ++gq)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        f16 yv = (f16)(sa * sb4[j % JH][gq][e]) * (f16)(float)(acc[i][j][gq * 4 + e] >> 8);
                        if (bias) yv = yv + bi4[j % JH][gq][e];
                        o[j % JH][gq][e] = yv;
                    }
            }
            store_slab_rows<JH>((u32x2*)(ks_lds + wave * (32 * JH * 32 * 2 / 16)), o, lane,
                                Y + (int64_t)row0 * N + n0 + wn * TN + j_first * 32, N, M - row0);
            continue;
        }
        if (row >= M) continue;
        f16 sa = (f16)0;
        if (DEQ) sa = sA[row];
#pragma unroll
        for (int j = 0; j < JN; ++j) {
            if (j < j_first || j >= j_first + JH) continue;     // the other K-group stores this tile
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const int col = n0 + wn * TN + j * 32 + gq * 8 + khalf * 4;
                if (col >= N) continue;
                int v4[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v4[e] = acc[i][j][gq * 4 + e] >> 8;
                const bool whole = (col + 4 <= N) && ((N & 3) == 0);
                if (DEQ) {
                    f16 o[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        f16 yv = (f16)(sa * sb4[j % JH][gq][e]) * (f16)(float)v4[e];
                        if (bias) yv = yv + bi4[j % JH][gq][e];
                        o[e] = yv;
                    }
                    f16* yp = Y + (int64_t)row * N + col;
                    if (whole) {
                        *(f16x4*)yp = f16x4{o[0], o[1], o[2], o[3]};
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (col + e < N) yp[e] = o[e];
                    }
                } else {
                    int32_t* cp = C + (int64_t)row * N + col;
                    if (whole) {
                        *(i32x4*)cp = i32x4{v4[0], v4[1], v4[2], v4[3]};
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (col + e < N) cp[e] = v4[e];
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
template <int BM, int BN, int WAVES_M, int WAVES_N>
int launch_ks(const void* A, const void* B, int M, int N, int Kb, void* C, void* Y, const void* sA, const void* sB,
              const void* bias, hipStream_t st, int ksplit = 1) {
    constexpr int NT = 128 * WAVES_M * WAVES_N;
    constexpr size_t STAGES = (size_t)3 * (BM + BN) * 8 * 16;
    constexpr size_t XCH = (size_t)WAVES_M * WAVES_N * 2 * (BN / WAVES_N / 64) * 256 * 16;
    constexpr size_t LDS = STAGES > XCH ? STAGES : XCH;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const int64_t tiles = (int64_t)tiles_m * tiles_n * ksplit;
    if (tiles > 0x3fffffff) return QR_E_SHAPE;
    if (ksplit > 1 && Y) return QR_E_UNSUPPORTED;           // partial sums exist only as int32
    const int nxcd = qr_device().xcds;                      // the grid is a whole number of rounds over the XCDs
    const unsigned grid = (unsigned)((tiles + nxcd - 1) / nxcd * nxcd);
    hipError_t e;
    if (Y) {
        auto kern = gemm_ks_kernel<BM, BN, WAVES_M, WAVES_N, true>;
        e = qr_allow_dynamic_lds((const void*)kern, LDS);
        if (e != hipSuccess) return (int)e;
        kern<<<dim3(grid), dim3(NT), LDS, st>>>((const uint8_t*)A, (const uint8_t*)B, M, N, Kb, nullptr, (f16*)Y,
                                                (const f16*)sA, (const f16*)sB, (const f16*)bias, tiles_m, tiles_n, 1, nxcd);
    } else {
        auto kern = gemm_ks_kernel<BM, BN, WAVES_M, WAVES_N, false>;
        e = qr_allow_dynamic_lds((const void*)kern, LDS);
        if (e != hipSuccess) return (int)e;
        kern<<<dim3(grid), dim3(NT), LDS, st>>>((const uint8_t*)A, (const uint8_t*)B, M, N, Kb, (int32_t*)C, nullptr,
                                                nullptr, nullptr, nullptr, tiles_m, tiles_n, ksplit, nxcd);
    }
    return qr_launch_status();
}

// ------------------------------------------------------------------------------------------------
// Software-pipelined kernels: four waves, ONE per SIMD, each owning a 128x128 wave tile (16 MFMA
// tiles, all 256 AGPRs), so that unpacking costs 3 instructions per MFMA.  A wave hides its own LDS
// latency and unpacking under its own MFMAs: while the 32 MFMAs of a 64-k sub-step run, the packed
// fragments of its next sub-step are read from LDS and unpacked.  The loop is written as explicit
// slots -- one MFMA, up to 4 unpacking instructions, at most one LDS read / LDS write / global
// load -- and a full scheduling barrier after every slot keeps the compiler from regrouping them
// (measured for one wave per SIMD: up to 5 VALU per MFMA cost 9 %, 6 cost 40 %).  A stage is 256 k
// (a 128-byte line per row); two LDS stage buffers; global loads are raw buffer loads (scalar
// descriptor + scalar stage offset + constant 32-bit lane offset: no address arithmetic in the loop)
// running ahead in registers; one workgroup barrier per stage.
//   gemm_sp256_kernel  256x256 tile, waves 2 (M) x 2 (N), whole K per wave: shapes with many tiles.  Also as a
//                      192x256 tile (wave tiles of 96x128: 12 MFMA tiles, 3.5 unpacking instructions per
//                      MFMA) for shapes that 256-row tiles spread over a fraction of the CUs and 128-row
//                      tiles over a round and a bit (2048 tokens against 5120 weight rows: 160 / 220 /
//                      320 tiles of 256 / 192 / 128 rows on 256 CUs).
//   gemm_spk_kernel    128x256 tile (one per CU at M = 2048, N = 4096), waves 2 (N) x 2 (K): the two
//                      K-groups take alternate pairs of sub-steps and exchange half of their
//                      accumulators through LDS at the end.
template <bool DEQ, bool RAGGED, int BM = 256>
__global__ __launch_bounds__(256) void gemm_sp256_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, int M, int N, int Kb, int32_t* __restrict__ C,
    f16* __restrict__ Y, const f16* __restrict__ sA, const f16* __restrict__ sB, const f16* __restrict__ bias,
    int tiles_m, int tiles_n, int nxcd) {
    static_assert(BM == 256 || BM == 192, "wave tiles of 4 or 3 accumulator tiles along M");
    constexpr int BN = 256, NT = 256;
    constexpr int TM = BM / 2, TN = 128, IM = TM / 32, JN = 4;
    constexpr int CH = (BM + BN) * 8;                       // 16-byte chunks per stage
    constexpr int NL = CH / NT;                             // 16 (14) per thread
    constexpr int NF = IM + JN;                             // fragments per sub-step
    constexpr int NMF = 2 * IM * JN;                        // MFMAs (= slots) per sub-step
    constexpr int UNP = NF * 12;                            // unpacking instructions per sub-step
    constexpr int S0 = 4;                                   // first slot that unpacks (LDS reads are issued in slots 0..7, in fragment order)
    constexpr bool DIRECT = !RAGGED;                        // whole stages go straight into LDS (see gemm_spk_kernel)
    extern __shared__ u32x4 sp2_lds[];                       // [2][CH]; later the output slabs

    const int per_xcd = gridDim.x / nxcd;
    int tile = (blockIdx.x % nxcd) * per_xcd + blockIdx.x / nxcd;
    if (tile >= tiles_m * tiles_n) return;
    constexpr int GROUP_M = 8;
    const int group_sz = GROUP_M * tiles_n;
    const int g = tile / group_sz;
    const int gm0 = g * GROUP_M;
    const int gh = (tiles_m - gm0) < GROUP_M ? (tiles_m - gm0) : GROUP_M;
    const int tm = gm0 + (tile - g * group_sz) % gh;
    const int tn = (tile - g * group_sz) / gh;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int khalf = lane >> 5;
    const int stages = (Kb + 127) / 128;
    auto slot8 = [](int row, int chunk) { return row * 8 + (chunk ^ ((row >> 1) & 7)); };

    // staging: chunk id = tid + i * 256: row = tid / 8 + 32 i, piece tid % 8
    const int srow = tid >> 3;
    const int scoff = (tid & 7) * 16;
    const int dst0 = slot8(srow, tid & 7);                  // rows differ by multiples of 32: same swizzle key
    u32 goff[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int row = srow + i * 32;
        int gr = row < BM ? m0 + row : n0 + row - BM;
        const int lim = row < BM ? M - 1 : N - 1;
        gr = gr < lim ? gr : lim;
        goff[i] = (u32)gr * (u32)Kb + (RAGGED ? 0u : DIRECT ? (u32)(((tid & 7) ^ ((srow >> 1) & 7)) * 16) : (u32)scoff);
    }
    u32x4 regs[1][NL];                                      // one set: loads run one (long) stage ahead of their LDS write
    // One 16-byte chunk of stage st (branch-free: stages past the end repeat the last one), as a raw
    // buffer load: scalar descriptor + scalar stage offset + constant 32-bit per-thread offset, so
    // the address costs no vector instruction and half the address traffic of a 64-bit pointer.
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, (int)((u32)M * (u32)Kb), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void*)B, 0, (int)((u32)N * (u32)Kb), 0x00020000);
    auto fetch1 = [&](int st, int set, int i) {
        const int kb = (st < stages ? st : stages - 1) * 128;
        u32 off = goff[i];
        if (RAGGED) off += (u32)((kb + scoff < Kb) ? scoff : 0);
        regs[set][i] = (i * 32 < BM) ? __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, off, kb, 0)
                                     : __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, off, kb, 0);
    };
    auto deposit1 = [&](int st, int buf, int set, int i) {    // st past the end: a repeat of the last stage, never read
        const bool dead = RAGGED && st >= stages - 1 && (stages - 1) * 128 + scoff >= Kb;
        sp2_lds[buf * CH + dst0 + i * 32 * 8] = dead ? u32x4{0, 0, 0, 0} : regs[set][i];
    };

    // direct form: chunk i of stage st into stage buffer buf (a wave's 64 lanes fill 1 KB of consecutive LDS)
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    auto dma1 = [&](int st, int buf, int i) {
        const int kb = (st < stages ? st : stages - 1) * 128;
        __attribute__((address_space(3))) void* dst =
            (__attribute__((address_space(3))) void*)(sp2_lds + buf * CH + i * NT + wave_u * 64);
        // (off: a plain u32 -- goff's bound depends on a template parameter, and with such an operand the
        // host pass silently drops the kernel's stub)
        const u32 off = goff[i];
        if (i * 32 < BM) __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, dst, 16, off, kb, 0, 0);
        else __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, dst, 16, off, kb, 0, 0);
    };

    i32x16 acc[IM][JN];
#pragma unroll
    for (int i = 0; i < IM; ++i)
#pragma unroll
        for (int j = 0; j < JN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

    // fragment slots of sub-step u: logical chunk 2 u + khalf
    int aslot[4], bslot[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        aslot[u] = slot8(wm * TM + (lane & 31), 2 * u + khalf);
        bslot[u] = slot8(BM + wn * TN + (lane & 31), 2 * u + khalf);
    }
    // fragments: index 0..1 = A (32-row tiles of the wave tile), 2..5 = B
    struct Packed {
        u32x4 f[IM + JN];
    };
    struct Ops {
        i32x4 lo[IM + JN], hi[IM + JN];
    };
    auto read1 = [&](int buf, int u, int r, Packed& p) {
        p.f[r] = r < IM ? sp2_lds[buf * CH + aslot[u] + r * 32 * 8] : sp2_lds[buf * CH + bslot[u] + (r - IM) * 32 * 8];
    };
    // unpacking as UNP single instructions: dword d = n / 3 of the packed dwords,
    // n % 3 = 0: lo = p << 4;  1: lo &= mask;  2: hi = p & mask
    auto unpack1 = [&](const Packed& p, Ops& o, int n) {
        const int d = n / 3, f = d >> 2, e = d & 3, kind = n % 3;
        if (kind == 0) o.lo[f][e] = (int)(p.f[f][e] << 4);
        else if (kind == 1) o.lo[f][e] = o.lo[f][e] & (int)0xF0F0F0F0u;
        else o.hi[f][e] = (int)(p.f[f][e] & 0xF0F0F0F0u);
    };
    auto mfma1 = [&](const Ops& o, int q) {
        const int t = q % (IM * JN), i = t / JN, j = t % JN;
        if (q < IM * JN) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.lo[IM + j], o.lo[i], acc[i][j], 0, 0, 0);
        else acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.hi[IM + j], o.hi[i], acc[i][j], 0, 0, 0);
    };
    // One 64-k sub-step = NMF = 32 slots.  Slot q: MFMA q of the current operands; slots 0..7 read
    // the packed fragments of the NEXT sub-step (one fragment buffer), slots S0.. unpack them
    // (UNP / (NMF - S0) = 4 instructions per slot); slots 8.. of sub-step 0 also write one chunk of
    // stage ks+1 to LDS each, slots 8.. of sub-step 1 request the same chunks of stage ks+2 (at most
    // one memory instruction per slot).  A full scheduling barrier after every slot keeps this order.
#define QR_SP2_SUBSTEP(CUR, NXT, RBUF, RU, DEP, FET)                                             \
    _Pragma("unroll") for (int q_ = 0; q_ < NMF; ++q_) {                                         \
        mfma1(CUR, q_);                                                                          \
        if (q_ < NF) read1(RBUF, RU, q_, pk);                                                    \
        if (q_ >= S0) {                                                                          \
            _Pragma("unroll") for (int n_ = ((q_ - S0) * UNP) / (NMF - S0); n_ < ((q_ - S0 + 1) * UNP) / (NMF - S0); ++n_) \
                unpack1(pk, NXT, n_);                                                            \
        }                                                                                        \
        if ((DEP) && q_ >= 8 && q_ < 8 + NL) deposit1(ks + 1, nb, 0, q_ - 8);                    \
        if ((FET) && q_ >= 8 && q_ < 8 + NL) fetch1(ks + 2, 0, q_ - 8);                          \
        __builtin_amdgcn_sched_barrier(0);                                                       \
    }

    Packed pk;
    Ops ops[2];
    if constexpr (DIRECT) {
        // Two stage buffers.  Sub-step 0 of stage s is read during sub-step 3 of stage s - 1, the rest
        // during sub-steps 0..2 of stage s; after the barrier of stage s (before its sub-step 3) nobody
        // reads buffer s % 2 any more, and the loads of stage s + 2 into it are issued in that sub-step 3:
        // they have three sub-steps (~2 us) to land before the next barrier, which waits for all of this
        // wave's loads.
#define QR_SP2D_BARRIER(ALLOWED)                                                                 \
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(ALLOWED) : "memory");
#define QR_SP2D_SUBSTEP(CUR, NXT, RBUF, RU, FET)                                                 \
    _Pragma("unroll") for (int q_ = 0; q_ < NMF; ++q_) {                                         \
        mfma1(CUR, q_);                                                                          \
        if (q_ < NF) read1(RBUF, RU, q_, pk);                                                    \
        if (q_ >= S0) {                                                                          \
            _Pragma("unroll") for (int n_ = ((q_ - S0) * UNP) / (NMF - S0); n_ < ((q_ - S0 + 1) * UNP) / (NMF - S0); ++n_) \
                unpack1(pk, NXT, n_);                                                            \
        }                                                                                        \
        if ((FET) && q_ >= 8 && q_ < 8 + NL) dma1(ks + 2, b, q_ - 8);                            \
        __builtin_amdgcn_sched_barrier(0);                                                       \
    }
#pragma unroll
        for (int i = 0; i < NL; ++i) dma1(0, 0, i);
#pragma unroll
        for (int i = 0; i < NL; ++i) dma1(1, 1, i);
        QR_SP2D_BARRIER(NL)
#pragma unroll
        for (int r = 0; r < NF; ++r) read1(0, 0, r, pk);
#pragma unroll
        for (int n = 0; n < UNP; ++n) unpack1(pk, ops[0], n);
        for (int ks = 0; ks < stages; ++ks) {
            const int b = ks & 1, nb = b ^ 1;
            QR_SP2D_SUBSTEP(ops[0], ops[1], b, 1, false)
            QR_SP2D_SUBSTEP(ops[1], ops[0], b, 2, false)
            QR_SP2D_SUBSTEP(ops[0], ops[1], b, 3, false)
            QR_SP2D_BARRIER(0)                              // stage ks+1 landed; stage ks fully read
            QR_SP2D_SUBSTEP(ops[1], ops[0], nb, 0, true)
        }
#undef QR_SP2D_SUBSTEP
#undef QR_SP2D_BARRIER
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");    // repeats of the last stage still landing
    } else {
    // prologue: stage 0 into LDS, stage 1 requested; sub-step 0 unpacked
#pragma unroll
    for (int i = 0; i < NL; ++i) fetch1(0, 0, i);
#pragma unroll
    for (int i = 0; i < NL; ++i) deposit1(0, 0, 0, i);
#pragma unroll
    for (int i = 0; i < NL; ++i) fetch1(1, 0, i);
    __syncthreads();
#pragma unroll
    for (int r = 0; r < NF; ++r) read1(0, 0, r, pk);
#pragma unroll
    for (int n = 0; n < UNP; ++n) unpack1(pk, ops[0], n);
    for (int ks = 0; ks < stages; ++ks) {
        const int b = ks & 1, nb = b ^ 1;
        // sub-step 0: multiply (ks,0); read + unpack (ks,1); stage ks+1 -> LDS, request ks+2
        QR_SP2_SUBSTEP(ops[0], ops[1], b, 1, true, false)
        // sub-step 1: multiply (ks,1); read + unpack (ks,2); request ks+2 into the registers just written out
        QR_SP2_SUBSTEP(ops[1], ops[0], b, 2, false, true)
        // sub-step 2: multiply (ks,2); read + unpack (ks,3)
        QR_SP2_SUBSTEP(ops[0], ops[1], b, 3, false, false)
        __syncthreads();                                    // stage ks+1 visible; stage ks fully read
        // sub-step 3: multiply (ks,3); read + unpack (ks+1,0)
        QR_SP2_SUBSTEP(ops[1], ops[0], nb, 0, false, false)
    }
    }
#undef QR_SP2_SUBSTEP
    __syncthreads();                                        // stage buffers free for the output slabs

    // Epilogue: lane l, register v -> n = (v/4)*8 + (l/32)*4 + v%4, m = l%32.
    const bool by_rows = DEQ && n0 + BN <= N && (N & 7) == 0 && (((uintptr_t)Y) & 15) == 0;
    if (DEQ && by_rows) {
#pragma unroll
        for (int jb = 0; jb < JN; jb += 2) {
            f16x4 sbh[2][4], bih[2][4];
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    const int col = n0 + wn * TN + (jb + jj) * 32 + gq * 8 + khalf * 4;
                    sbh[jj][gq] = *(const f16x4*)(sB + col);
                    bih[jj][gq] = bias ? *(const f16x4*)(bias + col) : f16x4{(f16)0, (f16)0, (f16)0, (f16)0};
                }
#pragma unroll
            for (int i = 0; i < IM; ++i) {
                const int row0 = m0 + wm * TM + i * 32;       // (rows past M: computed on a clamped scale, not stored)
                if (row0 >= M) continue;
                const f16 sa = sA[min(row0 + (lane & 31), M - 1)];
                f16x4 o[2][4];
#pragma unroll
                for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                    for (int gq = 0; gq < 4; ++gq)
                        o[jj][gq] = dequant4(acc[i][jb + jj][gq * 4], acc[i][jb + jj][gq * 4 + 1], acc[i][jb + jj][gq * 4 + 2],
                                             acc[i][jb + jj][gq * 4 + 3], sa, sbh[jj][gq], bih[jj][gq], bias != nullptr);
                store_slab_rows<2>((u32x2*)(sp2_lds + wave * 256), o, lane,
                                   Y + (int64_t)row0 * N + n0 + wn * TN + jb * 32, N, M - row0);
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < IM; ++i) {
        const int row = m0 + wm * TM + i * 32 + (lane & 31);
        if (row >= M) continue;
        f16 sa = (f16)0;
        if (DEQ) sa = sA[row];
#pragma unroll
        for (int j = 0; j < JN; ++j) {
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const int col = n0 + wn * TN + j * 32 + gq * 8 + khalf * 4;
                if (col >= N) continue;
                int v4[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v4[e] = acc[i][j][gq * 4 + e] >> 8;
                if (DEQ) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (col + e < N) {
                            f16 yv = (f16)(sa * sB[col + e]) * (f16)(float)v4[e];
                            if (bias) yv = yv + bias[col + e];
                            Y[(int64_t)row * N + col + e] = yv;
                        }
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < N) C[(int64_t)row * N + col + e] = v4[e];
                }
            }
        }
    }
}

template <bool DEQ, bool RAGGED>
__global__ __launch_bounds__(256) void gemm_spk_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, int M, int N, int Kb, int32_t* __restrict__ C,
    f16* __restrict__ Y, const f16* __restrict__ sA, const f16* __restrict__ sB, const f16* __restrict__ bias,
    int tiles_m, int tiles_n, int nxcd) {
    constexpr int BM = 128, BN = 256, NT = 256;
    constexpr int TM = 128, TN = 128, IM = 4, JN = 4;
    constexpr int CH = (BM + BN) * 8;                       // 16-byte chunks per stage
    constexpr int NL = CH / NT;                             // 12 per thread
    constexpr int NF = IM + JN;                             // fragments per sub-step
    constexpr int NMF = 2 * IM * JN;                        // MFMAs (= slots) per sub-step
    constexpr int UNP = NF * 12;                            // unpacking instructions per sub-step
    constexpr int S0 = 4;                                   // first slot that unpacks (LDS reads are issued in slots 0..7, in fragment order)
    // Whole stages (K % 256 == 0) go from global memory straight into LDS (buffer_load ... lds, 16
    // bytes per lane): no staging registers, no LDS write instructions, a third stage buffer instead.
    // Measured 3-5 % faster than the register-staged form (kept for ragged K, where dead pieces must
    // be written as zeros) at M = 2048, N = 4096, K = 11008 and K = 4096.
    constexpr bool DIRECT = !RAGGED;
    extern __shared__ u32x4 spk_lds[];                       // [DIRECT ? 3 : 2][CH]; later the output slabs

    const int per_xcd = gridDim.x / nxcd;
    int tile = (blockIdx.x % nxcd) * per_xcd + blockIdx.x / nxcd;
    if (tile >= tiles_m * tiles_n) return;
    constexpr int GROUP_M = 8;
    const int group_sz = GROUP_M * tiles_n;
    const int g = tile / group_sz;
    const int gm0 = g * GROUP_M;
    const int gh = (tiles_m - gm0) < GROUP_M ? (tiles_m - gm0) : GROUP_M;
    const int tm = gm0 + (tile - g * group_sz) % gh;
    const int tn = (tile - g * group_sz) / gh;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = 0, wn = wave & 1, kg = wave >> 1;        // K-group kg multiplies sub-steps 2 kg and 2 kg + 1 of every stage
    const int khalf = lane >> 5;
    const int stages = (Kb + 127) / 128;
    auto slot8 = [](int row, int chunk) { return row * 8 + (chunk ^ ((row >> 1) & 7)); };

    // staging: chunk id = tid + i * 256: row = tid / 8 + 32 i, piece tid % 8
    const int srow = tid >> 3;
    const int scoff = (tid & 7) * 16;
    const int dst0 = slot8(srow, tid & 7);                  // rows differ by multiples of 32: same swizzle key
    u32 goff[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int row = srow + i * 32;
        int gr = row < BM ? m0 + row : n0 + row - BM;
        const int lim = row < BM ? M - 1 : N - 1;
        gr = gr < lim ? gr : lim;
        // direct form: a lane's data lands at LDS position (row, tid % 8), so the lane fetches the
        // piece that the XOR-keyed layout keeps there (the key is the same for all of a lane's rows)
        goff[i] = (u32)gr * (u32)Kb + (RAGGED ? 0u : DIRECT ? (u32)(((tid & 7) ^ ((srow >> 1) & 7)) * 16) : (u32)scoff);
    }
    u32x4 regs[2][NL];                                      // two sets: loads run two stages ahead of their LDS write
    // One 16-byte chunk of stage st (branch-free: stages past the end repeat the last one), as a raw
    // buffer load: scalar descriptor + scalar stage offset + constant 32-bit per-thread offset, so
    // the address costs no vector instruction and half the address traffic of a 64-bit pointer.
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, (int)((u32)M * (u32)Kb), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void*)B, 0, (int)((u32)N * (u32)Kb), 0x00020000);
    auto fetch1 = [&](int st, int set, int i) {
        const int kb = (st < stages ? st : stages - 1) * 128;
        u32 off = goff[i];
        if (RAGGED) off += (u32)((kb + scoff < Kb) ? scoff : 0);
        regs[set][i] = (i * 32 < BM) ? __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, off, kb, 0)
                                     : __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, off, kb, 0);
    };
    auto deposit1 = [&](int st, int buf, int set, int i) {    // st past the end: a repeat of the last stage, never read
        const bool dead = RAGGED && st >= stages - 1 && (stages - 1) * 128 + scoff >= Kb;
        spk_lds[buf * CH + dst0 + i * 32 * 8] = dead ? u32x4{0, 0, 0, 0} : regs[set][i];
    };

    // direct form: chunk i of stage st into stage buffer buf; a wave's 64 lanes fill 1 KB of consecutive
    // LDS (8 rows of 128 bytes).  Stages past the end repeat the last one into a buffer nobody reads, so
    // that every stage issues the same number of loads (the waits below count them).
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    auto dma1 = [&](int st, int buf, int i) {
        const int kb = (st < stages ? st : stages - 1) * 128;
        __attribute__((address_space(3))) void* dst =
            (__attribute__((address_space(3))) void*)(spk_lds + buf * CH + i * NT + wave_u * 64);
        if (i * 32 < BM) __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, dst, 16, goff[i], kb, 0, 0);
        else __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, dst, 16, goff[i], kb, 0, 0);
    };

    i32x16 acc[IM][JN];
#pragma unroll
    for (int i = 0; i < IM; ++i)
#pragma unroll
        for (int j = 0; j < JN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

    // fragment slots of this wave's two sub-steps u0 = 2 kg, u1 = 2 kg + 1: logical chunk 2 u + khalf
    const int u0 = 2 * kg, u1 = 2 * kg + 1;
    const int aslot0 = slot8(wm * TM + (lane & 31), 2 * u0 + khalf), aslot1 = slot8(wm * TM + (lane & 31), 2 * u1 + khalf);
    const int bslot0 = slot8(BM + wn * TN + (lane & 31), 2 * u0 + khalf), bslot1 = slot8(BM + wn * TN + (lane & 31), 2 * u1 + khalf);
    // fragments: index 0..1 = A (32-row tiles of the wave tile), 2..5 = B
    struct Packed {
        u32x4 f[IM + JN];
    };
    struct Ops {
        i32x4 lo[IM + JN], hi[IM + JN];
    };
    // K-group 1 holds its B fragments (and so its accumulator columns) with the two 64-column halves
    // swapped: either group then KEEPS accumulator tiles j = 0, 1 and SENDS j = 2, 3, with
    // compile-time register indices on both sides
    const int bswap = kg * 64 * 8;                          // LDS offset of 64 rows
    auto read1 = [&](int buf, int second, int r, Packed& p) {  // second: sub-step u1 rather than u0
        const int as = second ? aslot1 : aslot0, bs = second ? bslot1 : bslot0;
        if (r < IM) p.f[r] = spk_lds[buf * CH + as + r * 32 * 8];
        else p.f[r] = spk_lds[buf * CH + bs + ((r - IM) * 32 * 8 ^ bswap)];
    };
    // unpacking as UNP single instructions: dword d = n / 3 of the packed dwords,
    // n % 3 = 0: lo = p << 4;  1: lo &= mask;  2: hi = p & mask
    auto unpack1 = [&](const Packed& p, Ops& o, int n) {
        const int d = n / 3, f = d >> 2, e = d & 3, kind = n % 3;
        if (kind == 0) o.lo[f][e] = (int)(p.f[f][e] << 4);
        else if (kind == 1) o.lo[f][e] = o.lo[f][e] & (int)0xF0F0F0F0u;
        else o.hi[f][e] = (int)(p.f[f][e] & 0xF0F0F0F0u);
    };
    auto mfma1 = [&](const Ops& o, int q) {
        const int t = q % (IM * JN), i = t / JN, j = t % JN;
        if (q < IM * JN) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.lo[IM + j], o.lo[i], acc[i][j], 0, 0, 0);
        else acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.hi[IM + j], o.hi[i], acc[i][j], 0, 0, 0);
    };
    // One 64-k sub-step = NMF = 32 slots.  Slot q: MFMA q of the current operands; slots 0..7 read
    // the packed fragments of this wave's NEXT sub-step (one fragment buffer), slots S0.. unpack
    // them (4 instructions per slot); slots 8.. of a stage's first sub-step also write one chunk
    // of stage ks+1 to LDS each, slots 8.. of its second sub-step request the same chunks of stage
    // ks+3 (one memory instruction per slot at most).  A full scheduling barrier after every slot
    // keeps this order.
#define QR_SPK_SUBSTEP(CUR, NXT, RBUF, RU, DEP, FET, SET)                                        \
    _Pragma("unroll") for (int q_ = 0; q_ < NMF; ++q_) {                                         \
        mfma1(CUR, q_);                                                                          \
        if (q_ < NF) read1(RBUF, RU, q_, pk);                                                    \
        if (q_ >= S0) {                                                                          \
            _Pragma("unroll") for (int n_ = ((q_ - S0) * UNP) / (NMF - S0); n_ < ((q_ - S0 + 1) * UNP) / (NMF - S0); ++n_) \
                unpack1(pk, NXT, n_);                                                            \
        }                                                                                        \
        if ((DEP) && q_ >= 8 && q_ < 8 + NL) deposit1(ks_ + 1, nb_, SET, q_ - 8);                \
        if ((FET) && q_ >= 8 && q_ < 8 + NL) fetch1(ks_ + 3, SET, q_ - 8);                       \
        __builtin_amdgcn_sched_barrier(0);                                                       \
    }
    // one stage: KS = stage index, B = its LDS buffer (compile-time), SET = register set that holds
    // stage KS+1 on entry and receives stage KS+3
#define QR_SPK_STAGE(KS, B, SET)                                                                 \
    {                                                                                            \
        const int ks_ = (KS);                                                                    \
        constexpr int b_ = (B), nb_ = 1 - (B);                                                   \
        /* first sub-step: multiply (ks,u0); read + unpack (ks,u1); stage ks+1 -> LDS */         \
        QR_SPK_SUBSTEP(ops[0], ops[1], b_, 1, true, false, SET)                                  \
        __syncthreads(); /* stage ks+1 visible; stage ks fully read */                           \
        /* second sub-step: multiply (ks,u1); read + unpack (ks+1,u0); request ks+3 */           \
        QR_SPK_SUBSTEP(ops[1], ops[0], nb_, 0, false, true, SET)                                 \
    }

    Packed pk;
    Ops ops[2];
    if constexpr (DIRECT) {
        // Three stage buffers.  Stage s lives in buffer s % 3; its sub-step u0 is read during the second
        // sub-step of stage s - 1, its sub-step u1 during the first sub-step of stage s; the barrier
        // of stage s (between its two sub-steps) is the last point at which anybody reads buffer
        // s % 3, and the loads of stage s + 3 into it are issued right after.  A wave's loads complete
        // in order, so "at most NL outstanding" at the barrier of stage s means its part of stage
        // s + 1 has landed (only stage s + 2 may still be in flight); the barrier then covers the other
        // waves' parts.  The wait is written by hand: the compiler would wait for all loads.
#define QR_SPKD_BARRIER(ALLOWED)                                                                 \
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(ALLOWED) : "memory");
#define QR_SPKD_SUBSTEP(CUR, NXT, RBUF, RU, FET, FBUF)                                           \
    _Pragma("unroll") for (int q_ = 0; q_ < NMF; ++q_) {                                         \
        mfma1(CUR, q_);                                                                          \
        if (q_ < NF) read1(RBUF, RU, q_, pk);                                                    \
        if (q_ >= S0) {                                                                          \
            _Pragma("unroll") for (int n_ = ((q_ - S0) * UNP) / (NMF - S0); n_ < ((q_ - S0 + 1) * UNP) / (NMF - S0); ++n_) \
                unpack1(pk, NXT, n_);                                                            \
        }                                                                                        \
        if ((FET) && q_ >= 8 && q_ < 8 + NL) dma1(ks_ + 3, FBUF, q_ - 8);                        \
        __builtin_amdgcn_sched_barrier(0);                                                       \
    }
#define QR_SPKD_STAGE(KS, B)                                                                     \
    {                                                                                            \
        const int ks_ = (KS);                                                                    \
        constexpr int b_ = (B), nb_ = ((B) + 1) % 3;                                             \
        /* multiply (ks,u0); read + unpack (ks,u1) */                                            \
        QR_SPKD_SUBSTEP(ops[0], ops[1], b_, 1, false, b_)                                        \
        QR_SPKD_BARRIER(NL) /* stage ks+1 landed; buffer b_ fully read */                        \
        /* multiply (ks,u1); read + unpack (ks+1,u0); stage ks+3 -> buffer b_ */                 \
        QR_SPKD_SUBSTEP(ops[1], ops[0], nb_, 0, true, b_)                                        \
    }
#pragma unroll
        for (int i = 0; i < NL; ++i) dma1(0, 0, i);
#pragma unroll
        for (int i = 0; i < NL; ++i) dma1(1, 1, i);
#pragma unroll
        for (int i = 0; i < NL; ++i) dma1(2, 2, i);
        QR_SPKD_BARRIER(2 * NL)
#pragma unroll
        for (int r = 0; r < NF; ++r) read1(0, 0, r, pk);
#pragma unroll
        for (int n = 0; n < UNP; ++n) unpack1(pk, ops[0], n);
        int ks = 0;
        for (; ks + 2 < stages; ks += 3) {
            QR_SPKD_STAGE(ks, 0)
            QR_SPKD_STAGE(ks + 1, 1)
            QR_SPKD_STAGE(ks + 2, 2)
        }
        if (ks < stages) {
            QR_SPKD_STAGE(ks, 0)
            if (ks + 1 < stages) QR_SPKD_STAGE(ks + 1, 1)
        }
#undef QR_SPKD_STAGE
#undef QR_SPKD_SUBSTEP
#undef QR_SPKD_BARRIER
        // the repeats of the last stage are still landing in the stage buffers, which the epilogue reuses
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else {
    // prologue: stage 0 into LDS, stages 1 and 2 requested; this wave's first sub-step unpacked
#pragma unroll
    for (int i = 0; i < NL; ++i) fetch1(0, 0, i);
#pragma unroll
    for (int i = 0; i < NL; ++i) fetch1(2, 1, i);
#pragma unroll
    for (int i = 0; i < NL; ++i) deposit1(0, 0, 0, i);
#pragma unroll
    for (int i = 0; i < NL; ++i) fetch1(1, 0, i);
    __syncthreads();
#pragma unroll
    for (int r = 0; r < NF; ++r) read1(0, 0, r, pk);
#pragma unroll
    for (int n = 0; n < UNP; ++n) unpack1(pk, ops[0], n);
    // (pairs of stages without a branch in between: the wait before an LDS write then counts the
    // other set's loads as still allowed in flight)
    int ks = 0;
    for (; ks + 1 < stages; ks += 2) {
        QR_SPK_STAGE(ks, 0, 0)
        QR_SPK_STAGE(ks + 1, 1, 1)
    }
    if (ks < stages) QR_SPK_STAGE(ks, 0, 0)
    }
#undef QR_SPK_STAGE
#undef QR_SPK_SUBSTEP

    // K-split: the two K-groups hold partial sums of the same 128x128 wave tile.  Each finalises the
    // 64 output columns held in its accumulator tiles j = 0, 1 (group 0: columns 0..63 of the wave
    // tile, group 1: 64..127) and sends tiles j = 2, 3 across through LDS, two 32-row tiles (i) per
    // round, four 16-byte pieces per lane and tile.
    {
        // (all four 32-row tiles in one round: 32 KB per wave, 128 KB of the stage buffers' 144 KB in the direct form;
        // the register-staged form has 96 KB of LDS and takes two rounds)
        u32x4* xbuf = spk_lds;
        constexpr int IR = DIRECT ? IM : 2;                   // 32-row tiles per round
#pragma unroll
        for (int ip = 0; ip < IM; ip += IR) {
            __syncthreads();
#pragma unroll
            for (int ii = 0; ii < IR; ++ii)
#pragma unroll
                for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                    for (int qv = 0; qv < 4; ++qv) {
                        const i32x16& t = acc[ip + ii][2 + jj];
                        xbuf[((((wn * 2 + (1 - kg)) * IR + ii) * 2 + jj) * 4 + qv) * 64 + lane] =
                            u32x4{(u32)t[qv * 4], (u32)t[qv * 4 + 1], (u32)t[qv * 4 + 2], (u32)t[qv * 4 + 3]};
                    }
            __syncthreads();
#pragma unroll
            for (int ii = 0; ii < IR; ++ii)
#pragma unroll
                for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                    for (int qv = 0; qv < 4; ++qv) {
                        const u32x4 piece = xbuf[((((wn * 2 + kg) * IR + ii) * 2 + jj) * 4 + qv) * 64 + lane];
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[ip + ii][jj][qv * 4 + e] += (int)piece[e];
                    }
        }
    }
    __syncthreads();                                        // stage buffers free for the output slabs

    // Epilogue: lane l, register v -> n = (v/4)*8 + (l/32)*4 + v%4, m = l%32.
    const bool by_rows = DEQ && n0 + BN <= N && (N & 7) == 0 && (((uintptr_t)Y) & 15) == 0;
    if (DEQ && by_rows) {
        const int jb = 2 * kg;
        {
            f16x4 sbh[2][4], bih[2][4];
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    const int col = n0 + wn * TN + (jb + jj) * 32 + gq * 8 + khalf * 4;
                    sbh[jj][gq] = *(const f16x4*)(sB + col);
                    bih[jj][gq] = bias ? *(const f16x4*)(bias + col) : f16x4{(f16)0, (f16)0, (f16)0, (f16)0};
                }
#pragma unroll
            for (int i = 0; i < IM; ++i) {
                const int row0 = m0 + wm * TM + i * 32;       // (rows past M: computed on a clamped scale, not stored)
                if (row0 >= M) continue;
                const f16 sa = sA[min(row0 + (lane & 31), M - 1)];
                f16x4 o[2][4];
#pragma unroll
                for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                    for (int gq = 0; gq < 4; ++gq)
                        o[jj][gq] = dequant4(acc[i][jj][gq * 4], acc[i][jj][gq * 4 + 1], acc[i][jj][gq * 4 + 2],
                                             acc[i][jj][gq * 4 + 3], sa, sbh[jj][gq], bih[jj][gq], bias != nullptr);
                store_slab_rows<2>((u32x2*)(spk_lds + wave * 256), o, lane,
                                   Y + (int64_t)row0 * N + n0 + wn * TN + jb * 32, N, M - row0);
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < IM; ++i) {
        const int row = m0 + wm * TM + i * 32 + (lane & 31);
        if (row >= M) continue;
        f16 sa = (f16)0;
        if (DEQ) sa = sA[row];
#pragma unroll
        for (int j = 0; j < 2; ++j) {                       // this K-group's tiles: output column tiles j + 2 kg
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const int col = n0 + wn * TN + (j + 2 * kg) * 32 + gq * 8 + khalf * 4;
                if (col >= N) continue;
                int v4[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v4[e] = acc[i][j][gq * 4 + e] >> 8;
                if (DEQ) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (col + e < N) {
                            f16 yv = (f16)(sa * sB[col + e]) * (f16)(float)v4[e];
                            if (bias) yv = yv + bias[col + e];
                            Y[(int64_t)row * N + col + e] = yv;
                        }
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < N) C[(int64_t)row * N + col + e] = v4[e];
                }
            }
        }
    }
}

int launch_spk(const void* A, const void* B, int M, int N, int Kb, void* C, void* Y, const void* sA, const void* sB,
               const void* bias, hipStream_t st) {
    const int tiles_m = (M + 127) / 128, tiles_n = (N + 255) / 256;
    const int64_t tiles = (int64_t)tiles_m * tiles_n;
    if (tiles > 0x3fffffff) return QR_E_SHAPE;
    const int nxcd = qr_device().xcds;                      // the grid is a whole number of rounds over the XCDs
    const unsigned grid = (unsigned)((tiles + nxcd - 1) / nxcd * nxcd);
    const bool ragged = (Kb & 127) != 0;
    // stage buffers of 48 KB: two behind staging registers, three when loaded straight into LDS
    const size_t LDS = (size_t)(ragged ? 2 : 3) * (128 + 256) * 8 * 16;
    if ((int64_t)M * Kb >= (1LL << 32) || (int64_t)N * Kb >= (1LL << 32)) return QR_E_UNSUPPORTED;   // (the dispatcher routes these away)
    hipError_t e;
    if (Y) {
        auto kern = ragged ? gemm_spk_kernel<true, true> : gemm_spk_kernel<true, false>;
        e = qr_allow_dynamic_lds((const void*)kern, LDS);
        if (e != hipSuccess) return (int)e;
        kern<<<dim3(grid), dim3(256), LDS, st>>>((const uint8_t*)A, (const uint8_t*)B, M, N, Kb, nullptr, (f16*)Y,
                                                 (const f16*)sA, (const f16*)sB, (const f16*)bias, tiles_m, tiles_n, nxcd);
    } else {
        auto kern = ragged ? gemm_spk_kernel<false, true> : gemm_spk_kernel<false, false>;
        e = qr_allow_dynamic_lds((const void*)kern, LDS);
        if (e != hipSuccess) return (int)e;
        kern<<<dim3(grid), dim3(256), LDS, st>>>((const uint8_t*)A, (const uint8_t*)B, M, N, Kb, (int32_t*)C, nullptr,
                                                 nullptr, nullptr, nullptr, tiles_m, tiles_n, nxcd);
    }
    return qr_launch_status();
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
int launch_cfg(const void* A, const void* B, int M, int N, int Kb, void* C, void* Y, const void* sA, const void* sB,
               const void* bias, hipStream_t st);

// bm: rows of a tile, 256 or 192 (192: eleven row tiles instead of eight at 2048 tokens -- shapes whose
// 256-row tiles would occupy a fraction of the CUs and whose 128-row tiles need a second round)
int launch_sp256(const void* A, const void* B, int M, int N, int Kb, void* C, void* Y, const void* sA, const void* sB,
                 const void* bias, hipStream_t st, int bm = 256) {
    const size_t LDS = (size_t)2 * (size_t)(bm + 256) * 8 * 16;
    const int tiles_m = (M + bm - 1) / bm, tiles_n = (N + 255) / 256;
    const int64_t tiles = (int64_t)tiles_m * tiles_n;
    if (tiles > 0x3fffffff) return QR_E_SHAPE;
    const int nxcd = qr_device().xcds;                      // the grid is a whole number of rounds over the XCDs
    const unsigned grid = (unsigned)((tiles + nxcd - 1) / nxcd * nxcd);
    const bool ragged = (Kb & 127) != 0;
    // operands are addressed through 32-bit buffer offsets (the dispatcher routes larger ones away)
    if ((int64_t)M * Kb >= (1LL << 32) || (int64_t)N * Kb >= (1LL << 32)) return QR_E_UNSUPPORTED;
    using Kern = void (*)(const uint8_t*, const uint8_t*, int, int, int, int32_t*, f16*, const f16*, const f16*, const f16*,
                          int, int, int);
    static const Kern table[2][2][2] = {
        {{gemm_sp256_kernel<false, false, 256>, gemm_sp256_kernel<false, true, 256>},
         {gemm_sp256_kernel<true, false, 256>, gemm_sp256_kernel<true, true, 256>}},
        {{gemm_sp256_kernel<false, false, 192>, gemm_sp256_kernel<false, true, 192>},
         {gemm_sp256_kernel<true, false, 192>, gemm_sp256_kernel<true, true, 192>}}};
    const Kern kern = table[bm == 192 ? 1 : 0][Y ? 1 : 0][ragged ? 1 : 0];
    const hipError_t e = qr_allow_dynamic_lds((const void*)kern, LDS);
    if (e != hipSuccess) return (int)e;
    if (Y)
        kern<<<dim3(grid), dim3(256), LDS, st>>>((const uint8_t*)A, (const uint8_t*)B, M, N, Kb, nullptr, (f16*)Y,
                                                 (const f16*)sA, (const f16*)sB, (const f16*)bias, tiles_m, tiles_n, nxcd);
    else
        kern<<<dim3(grid), dim3(256), LDS, st>>>((const uint8_t*)A, (const uint8_t*)B, M, N, Kb, (int32_t*)C, nullptr,
                                                 nullptr, nullptr, nullptr, tiles_m, tiles_n, nxcd);
    return qr_launch_status();
}

// ------------------------------------------------------------------------------------------------
// Decode (M <= 64) with too few column tiles for the tiled kernels, or few tokens.  A workgroup of
// eight waves owns 8 / KW groups of 32 weight rows; the KW waves of a group split K into contiguous
// ranges and their partial 32 x M tiles are summed through LDS and dequantised (KW = 8 when K is
// long and N small, 2 or 4 when a wave would otherwise get only a handful of steps).  Nothing is shared between waves in the main loop, so there
// are no barriers in it: every wave streams its own slices of W and X with coalesced 16-byte loads
// (SB / 16 lanes per row piece of SB bytes, PF steps ahead in a register ring) and turns them into
// MFMA fragments (lane = row) through a wave-private LDS buffer.  Loading fragments straight from
// global memory makes every instruction touch 32 different lines and was measured 1.5-2x slower.
// XL = load instructions per step that carry rows of X (64 / CPR rows each): with few tokens only
// the first ceil(M / (64 / CPR)) of them are issued and staged; the remaining rows of the 32-row
// MFMA operand keep whatever the buffer holds, and the output rows they produce are never stored.
template <int MT, int SB, int XL, int PF, int KW, bool DEQ>
__global__ __launch_bounds__(512) void decode_i4_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                        int M, int N, int Kb, int32_t* __restrict__ C,
                                                        f16* __restrict__ Y, const f16* __restrict__ sA,
                                                        const f16* __restrict__ sB, const f16* __restrict__ bias) {
    constexpr int CPR = SB / 16;                            // 16-byte chunks per row and step (4, 8 or 16)
    constexpr int ROWS = (1 + MT) * 32;                     // staged rows per wave: 32 of W, then 32 MT of X
    constexpr int NLW = 32 * CPR / 64;                      // chunks per lane and step: rows of W ...
    constexpr int NLD = NLW + XL;                           // ... plus the rows of X that exist
    static_assert(XL >= 1 && XL <= MT * 32 * CPR / 64, "X load groups");
    constexpr int STAGE = ROWS * CPR;                       // u32x4 per wave
    constexpr int RED = MT * 4 * 64;                        // i32x4 per wave for the final sum
    extern __shared__ u32x4 dec_smem[];                     // 8 * max(STAGE, RED)
    i32x4* red = (i32x4*)dec_smem;                          // [wave][m tile][4-register group][lane]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    constexpr int RG = 8 / KW;                              // groups of 32 weight rows per workgroup
    const int kw = wave % KW;                               // this wave's share of K within its row group
    const int n0 = (blockIdx.x * RG + wave / KW) * 32;
    const int steps = (Kb + SB - 1) / SB;
    const int s_begin = (int)((int64_t)steps * kw / KW), s_end = (int)((int64_t)steps * (kw + 1) / KW);
    u32x4* stage = dec_smem + wave * STAGE;
    // chunk position XOR-keyed by the row: the 16 rows of a fragment read spread over all bank groups
    auto slot = [](int row, int chunk) {
        return CPR == 4 ? row * 4 + (chunk ^ ((row >> 2) & 3))
               : CPR == 8 ? row * 8 + (chunk ^ ((row >> 1) & 7)) : row * 16 + (chunk ^ (row & 15));
    };

    // chunk i of this lane: row (lane + 64 i) / CPR, 16-byte piece lane % CPR
    const int piece = lane % CPR;
    const uint8_t* src[NLD];
    int dst[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int row = lane / CPR + (64 / CPR) * i;
        if (row < 32) {
            int nr = n0 + row;
            nr = nr < N ? nr : N - 1;
            src[i] = B + (int64_t)nr * Kb;
        } else {
            int mr = row - 32;
            mr = mr < M ? mr : M - 1;
            src[i] = A + (int64_t)mr * Kb;
        }
        dst[i] = slot(row, piece);
    }
    // K % 64 == 0: a row is a whole number of 32-byte pairs of pieces.  Pieces of the last step that
    // lie beyond the row re-read piece 0 or 1 of that step and are deposited as zeros.
    struct Step {
        u32x4 v[NLD];
    };
    auto fetch = [&](int sidx, Step& st) {
        const int sc = sidx < steps ? sidx : steps - 1;
        const bool dead = sc * SB + piece * 16 >= Kb;
        const int off = sc * SB + (dead ? (piece & 1) : piece) * 16;
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            // weights are used once: streaming loads keep the tokens' codes, which every workgroup
            // re-reads, in the caches
            if (i < NLW) st.v[i] = __builtin_nontemporal_load((const u32x4*)(src[i] + off));
            else st.v[i] = *(const u32x4*)(src[i] + off);
        }
    };
    i32x16 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0;
    auto deposit = [&](int sidx, const Step& st) {
        const bool dead = sidx * SB + piece * 16 >= Kb;
        // LDS operations of one wave execute in order: these writes follow the previous step's reads
#pragma unroll
        for (int i = 0; i < NLD; ++i) stage[dst[i]] = dead ? u32x4{0, 0, 0, 0} : st.v[i];
    };
    auto multiply = [&]() {
#pragma unroll
        for (int c = 0; c < CPR / 2; ++c) {                 // lane half h takes pieces 2c + h of both operands
            const u32x4 wq = stage[slot(r, 2 * c + h)];
            const i32x4 wlo = (i32x4)((wq << 4) & 0xF0F0F0F0u), whi = (i32x4)(wq & 0xF0F0F0F0u);
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const u32x4 xq = stage[slot(32 + t * 32 + r, 2 * c + h)];
                const i32x4 xlo = (i32x4)((xq << 4) & 0xF0F0F0F0u), xhi = (i32x4)(xq & 0xF0F0F0F0u);
                acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wlo, xlo, acc[t], 0, 0, 0);
                acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(whi, xhi, acc[t], 0, 0, 0);
            }
        }
    };
    Step ring[PF];
#pragma unroll
    for (int p = 0; p < PF; ++p) fetch(s_begin + p, ring[p]);
    // whole turns of the ring run without a branch, so that every wait inside them counts exactly the
    // loads issued after the step it needs (a branch in the loop body makes the compiler wait for all
    // outstanding loads once per turn)
    // The loads that refill a ring slot are issued as soon as the slot has been written to LDS, before
    // the step's multiplications; the scheduling barriers keep the compiler from moving them later.
    int s = s_begin;
    for (; s + PF <= s_end; s += PF) {
#pragma unroll
        for (int p = 0; p < PF; ++p) {
            deposit(s + p, ring[p]);
            __builtin_amdgcn_sched_barrier(0);
            fetch(s + p + PF, ring[p]);                     // indices past the end re-read the last step (unused)
            __builtin_amdgcn_sched_barrier(0);
            multiply();
        }
    }
#pragma unroll
    for (int p = 0; p < PF - 1; ++p)
        if (s + p < s_end) {
            deposit(s + p, ring[p]);
            multiply();
        }
    __syncthreads();                                        // the staging buffers become the reduction buffer
    // ---- sum the eight partial tiles
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int gq = 0; gq < 4; ++gq)
            red[((wave * MT + t) * 4 + gq) * 64 + lane] = i32x4{acc[t][gq * 4], acc[t][gq * 4 + 1], acc[t][gq * 4 + 2], acc[t][gq * 4 + 3]};
    __syncthreads();
    // unit u = (row group, m tile, register group): the waves take them in turn
    for (int u = wave; u < RG * MT * 4; u += 8) {
        const int g = u / (MT * 4), t = (u >> 2) % MT, gq = u & 3;
        i32x4 sum = {0, 0, 0, 0};
#pragma unroll
        for (int w = 0; w < KW; ++w) sum += red[(((g * KW + w) * MT + t) * 4 + gq) * 64 + lane];
        const int row = t * 32 + r;
        const int col = (blockIdx.x * RG + g) * 32 + gq * 8 + h * 4;
        if (row < M && col < N) {
            const bool whole = (col + 4 <= N) && ((N & 3) == 0);
            if (DEQ) {
                const f16 sa = sA[row];
                f16 o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int cc = col + e < N ? col + e : N - 1;
                    f16 yv = (f16)(sa * sB[cc]) * (f16)(float)(sum[e] >> 8);
                    if (bias) yv = yv + bias[cc];
                    o[e] = yv;
                }
                f16* yp = Y + (int64_t)row * N + col;
                if (whole) {
                    *(f16x4*)yp = f16x4{o[0], o[1], o[2], o[3]};
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < N) yp[e] = o[e];
                }
            } else {
                int32_t* cp = C + (int64_t)row * N + col;
                if (whole) {
                    *(i32x4*)cp = i32x4{sum[0] >> 8, sum[1] >> 8, sum[2] >> 8, sum[3] >> 8};
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < N) cp[e] = sum[e] >> 8;
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Decode (M <= 64) with many weight rows: a workgroup owns R groups of 32 weight rows (R = 4 .. 8,
// chosen by the host so that the workgroups spread evenly over the CUs: 57344 rows are 256 workgroups
// of 7 groups) and walks K in stages of 128 packed bytes per row.
// * Twelve waves in two roles.  Waves 8..11 only FETCH: eight consecutive threads one 128-byte line,
//   MT + R chunks per thread and stage, into RD register sets that rotate RD stages ahead of the LDS
//   fill; three LDS stage buffers rotate; one barrier per stage.  Waves 0..R-1 only MULTIPLY: wave w
//   takes row group w against all tokens.  With every wave doing both, a wave waits for its loads and
//   then multiplies, the whole CU in step: the multiplications were not hidden behind the memory time
//   (64 tokens: 47 us; with the roles split 42 us, the same as 8 tokens).
// * The tokens' codes are fetched ONCE per workgroup and stage and shared through LDS -- with
//   wave-private staging every wave would pull its own copy through the vector cache, twice the weight
//   bytes at 64 tokens -- and the thread that fetched a chunk of them stores it already unpacked into
//   its two int8 planes, so that no multiplying wave unpacks tokens.
// * The multiplications are software-pipelined over the 64-k sub-steps (see `substep`).
// * Workgroup b starts its walk over K at stage b % stages and wraps around (integer sums do not depend
//   on the order): with a row pitch that is a power of two, workgroups marching through K in step
//   would all be reading the same few memory channels at any one time (measured 49 -> 41 us at
//   57344 x 8192).
// * ksplit > 1 (int32 output only; weights with few rows, 32..64 tokens): `ksplit` workgroups share a block of R
//   groups and each walks its own slice of K, writing its partial sums to its own [M, N] slab of C -- a workgroup then
//   pulls 1 / ksplit of the tokens' codes through its CU's vector memory path, which is what bounds this shape (every
//   CU reading ALL the tokens' codes next to its share of the weights: 0.92 MB beside 0.46 MB at 64 tokens).
template <int MT, int R, int RD, bool DEQ>
__global__ __launch_bounds__(768) void decode_xs_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                        int M, int N, int Kb, int32_t* __restrict__ C,
                                                        f16* __restrict__ Y, const f16* __restrict__ sA,
                                                        const f16* __restrict__ sB, const f16* __restrict__ bias,
                                                        int ksplit) {
    constexpr int XR = MT * 32;                             // staged rows of X
    constexpr int NL = MT + R;                              // 16-byte chunks per loader thread and stage: 32 rows each
    constexpr int XPLANES = XR * 16;                        // slots of the tokens' planes (32 bytes per packed chunk)
    constexpr int CH = XPLANES + R * 32 * 8;                // slots per stage buffer
    constexpr int NBUF = 3;
    extern __shared__ u32x4 xs_lds[];                       // [NBUF][CH]; later the output slabs
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    const bool loader = wave >= 8;                          // waves 8..11 fetch, waves 0..R-1 multiply
    const int rblock = blockIdx.x / ksplit, slice = blockIdx.x - rblock * ksplit;
    const int n0 = rblock * (R * 32);
    const int all_stages = (Kb + 127) / 128;
    const int sfirst = (int)((int64_t)all_stages * slice / ksplit);
    const int stages = (int)((int64_t)all_stages * (slice + 1) / ksplit) - sfirst;      // >= 1: ksplit <= all_stages
    if (ksplit > 1) C += (int64_t)slice * M * N;
    const bool ragged = (Kb & 127) != 0;
    auto slot8 = [](int row, int chunk) { return row * 8 + (chunk ^ ((row >> 1) & 7)); };
    auto slot16 = [](int row, int chunk, int plane) {
        return row * 16 + ((chunk ^ (row & 7)) << 1) + (plane ^ ((row >> 3) & 1));
    };

    const int ltid = tid & 255;
    const int srow = ltid >> 3, piece = ltid & 7;           // chunk i of a loader thread: row srow + 32 i, same piece
    const uint8_t* src[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        if (i < MT) {
            const int mr = srow + 32 * i;
            src[i] = A + (int64_t)(mr < M ? mr : M - 1) * Kb;
        } else {
            const int nr = n0 + srow + 32 * (i - MT);
            src[i] = B + (int64_t)(nr < N ? nr : N - 1) * Kb;
        }
    }
    const int wdst0 = XPLANES + slot8(srow, piece);         // rows differ by multiples of 32: same swizzle
    const int xdst0 = slot16(srow, piece, 0);
    const int s0 = rblock % stages;
    auto stage_of = [&](int st) {                           // absolute stage of this workgroup's st-th step
        int a = (st < stages ? st : stages - 1) + s0;
        return sfirst + (a >= stages ? a - stages : a);
    };
    auto fetch = [&](int st, u32x4(&v)[NL]) {
        const int kb = stage_of(st) * 128;
        const int off = (kb + piece * 16 < Kb) ? kb + piece * 16 : kb;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            // weights are used once: streaming loads keep the tokens' codes, which every workgroup
            // re-reads, in the caches
            if (i >= MT) v[i] = __builtin_nontemporal_load((const u32x4*)(src[i] + off));
            else v[i] = *(const u32x4*)(src[i] + off);
        }
    };
    // stages past the end are written too (into a buffer nobody reads again): without a branch every
    // wait counts exactly the loads issued after the ones it needs
    auto deposit = [&](int st, int buf, const u32x4(&v)[NL]) {
        const bool zero = ragged && stage_of(st) * 128 + piece * 16 >= Kb;
        u32x4* base = xs_lds + buf * CH;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const u32x4 q = zero ? u32x4{0, 0, 0, 0} : v[i];
            if (i < MT) {
                base[xdst0 + i * 32 * 16] = (q << 4) & 0xF0F0F0F0u;
                base[(xdst0 ^ 1) + i * 32 * 16] = q & 0xF0F0F0F0u;
            } else {
                base[wdst0 + (i - MT) * 32 * 8] = q;
            }
        }
    };
    i32x16 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0;
    // logical chunk 2u + h of weight row q sits at slot8(q, h) ^ (2u); plane p of a token row's chunk
    // 2u + h at slot16(q, h, 0) ^ (4u + p): the swizzles only touch the low bits
    const bool computes = wave < R;                         // (waves R..7 only keep the barriers' count)
    const int wslot = XPLANES + slot8((computes ? wave : 0) * 32 + r, h), xslot = slot16(r, h, 0);
    // The multiplications are software-pipelined over the 64-k sub-steps: while the 2 MT MFMAs of one
    // sub-step run, the operands of the next one (the first of the next stage after the last: that
    // buffer became visible with the previous barrier) are read from LDS and the weights unpacked.
    // Written as slots of one MFMA plus its share of the reads and unpacking, with a scheduling barrier
    // after every slot: left to itself the compiler reads, unpacks and multiplies in three phases, and
    // with the two waves of a SIMD in step after every barrier the three pipes then take turns
    // (measured: LDS, vector and matrix time added up to the whole launch).
    struct Ops {
        u32x4 w;
        i32x4 wlo, whi, xlo[MT], xhi[MT];
    };
    Ops ops[2];
    auto read_w = [&](const u32x4* base, int uu, Ops& o) { o.w = base[wslot ^ (2 * uu)]; };
    auto read_x = [&](const u32x4* base, int uu, int t, int plane, Ops& o) {
        const i32x4 q = (i32x4)base[(xslot ^ (4 * uu + plane)) + t * 32 * 16];
        if (plane) o.xhi[t] = q;
        else o.xlo[t] = q;
    };
    auto unpack_lo = [&](Ops& o) { o.wlo = (i32x4)((o.w << 4) & 0xF0F0F0F0u); };
    auto unpack_hi = [&](Ops& o) { o.whi = (i32x4)(o.w & 0xF0F0F0F0u); };
    auto substep = [&](const Ops& cur, Ops& nxt, const u32x4* nbase, int nu) {
        // slot 0
        acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(cur.wlo, cur.xlo[0], acc[0], 0, 0, 0);
        read_w(nbase, nu, nxt);
        read_x(nbase, nu, 0, 0, nxt);
        if (MT == 1) read_x(nbase, nu, 0, 1, nxt);
        __builtin_amdgcn_sched_barrier(0);
        if (MT == 2) {
            acc[MT - 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(cur.wlo, cur.xlo[MT - 1], acc[MT - 1], 0, 0, 0);
            read_x(nbase, nu, 0, 1, nxt);
            read_x(nbase, nu, MT - 1, 0, nxt);
            __builtin_amdgcn_sched_barrier(0);
        }
        acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(cur.whi, cur.xhi[0], acc[0], 0, 0, 0);
        if (MT == 2) read_x(nbase, nu, MT - 1, 1, nxt);
        unpack_lo(nxt);
        if (MT == 1) unpack_hi(nxt);
        __builtin_amdgcn_sched_barrier(0);
        if (MT == 2) {
            acc[MT - 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(cur.whi, cur.xhi[MT - 1], acc[MT - 1], 0, 0, 0);
            unpack_hi(nxt);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    if (loader) {
        u32x4 regs[RD][NL];
#pragma unroll
        for (int q = 0; q < RD; ++q) fetch(q, regs[q]);
        deposit(0, 0, regs[0]);
        fetch(RD, regs[0]);
        deposit(1, 1, regs[1 % RD]);
        fetch(RD + 1, regs[1 % RD]);
        __syncthreads();                                    // stages 0 and 1 visible
        int bfill = 2;
        auto iteration = [&](int ks, u32x4(&v)[NL]) {
            deposit(ks + 2, bfill, v);
            __builtin_amdgcn_sched_barrier(0);
            fetch(ks + 2 + RD, v);
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
            bfill = bfill == NBUF - 1 ? 0 : bfill + 1;
        };
        int ks0 = 0;
        for (; ks0 + RD <= stages; ks0 += RD) {
#pragma unroll
            for (int q = 0; q < RD; ++q) iteration(ks0 + q, regs[(q + 2) % RD]);
        }
#pragma unroll
        for (int q = 0; q < RD - 1; ++q)
            if (ks0 + q < stages) iteration(ks0 + q, regs[(q + 2) % RD]);
        return;
    }
    __syncthreads();                                        // stages 0 and 1 visible
    if (computes) {
        read_w(xs_lds, 0, ops[0]);
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            read_x(xs_lds, 0, t, 0, ops[0]);
            read_x(xs_lds, 0, t, 1, ops[0]);
        }
        unpack_lo(ops[0]);
        unpack_hi(ops[0]);
    }
    {
        int bcur = 0;
        for (int ks = 0; ks < stages; ++ks) {
            const int bnext = bcur == NBUF - 1 ? 0 : bcur + 1;
            if (computes) {
                const u32x4* cb = xs_lds + bcur * CH;
                substep(ops[0], ops[1], cb, 1);
                substep(ops[1], ops[0], cb, 2);
                substep(ops[0], ops[1], cb, 3);
                substep(ops[1], ops[0], xs_lds + bnext * CH, 0);   // after the last stage: read, never used
            }
            __syncthreads();
            bcur = bnext;
        }
    }

    // ---- epilogue: lane l, register v -> weight row (v/4)*8 + (l/32)*4 + v%4 of the group, token l%32
    auto finish = [&](const i32x16& a, int g, int t) {
        const int c0 = n0 + g * 32;
        const int row = t * 32 + r;
        const bool by_rows = DEQ && c0 + 32 <= N && (N & 7) == 0 && (((uintptr_t)Y) & 15) == 0 && t * 32 + 32 <= M;
        f16x4 sb4[4], bi4[4];
        if (DEQ) {
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const int col = c0 + gq * 8 + h * 4;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int cc = col + e < N ? col + e : N - 1;
                    sb4[gq][e] = sB[cc];
                    bi4[gq][e] = bias ? bias[cc] : (f16)0;
                }
            }
        }
        if (DEQ && by_rows) {
            const f16 sa = sA[row];
            f16x4 o[1][4];
#pragma unroll
            for (int gq = 0; gq < 4; ++gq)
                o[0][gq] = dequant4(a[gq * 4], a[gq * 4 + 1], a[gq * 4 + 2], a[gq * 4 + 3], sa, sb4[gq], bi4[gq], bias != nullptr);
            store_slab_rows<1>((u32x2*)(xs_lds + wave * 128), o, lane, Y + (int64_t)(t * 32) * N + c0, N);
            return;
        }
        if (row >= M) return;
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
            const int col = c0 + gq * 8 + h * 4;
            if (col >= N) continue;
            const bool whole = (col + 4 <= N) && ((N & 3) == 0);
            if (DEQ) {
                const f16x4 o = dequant4(a[gq * 4], a[gq * 4 + 1], a[gq * 4 + 2], a[gq * 4 + 3], sA[row], sb4[gq], bi4[gq],
                                         bias != nullptr);
                f16* yp = Y + (int64_t)row * N + col;
                if (whole) {
                    *(f16x4*)yp = o;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < N) yp[e] = o[e];
                }
            } else {
                int32_t* cp = C + (int64_t)row * N + col;
                if (whole) {
                    *(i32x4*)cp = i32x4{a[gq * 4] >> 8, a[gq * 4 + 1] >> 8, a[gq * 4 + 2] >> 8, a[gq * 4 + 3] >> 8};
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < N) cp[e] = a[gq * 4 + e] >> 8;
                }
            }
        }
    };
    if (!computes) return;
#pragma unroll
    for (int t = 0; t < MT; ++t) finish(acc[t], wave, t);
}

// ------------------------------------------------------------------------------------------------
// Decode with very few tokens (M <= 8): a matrix-vector style kernel on the native int4 dot product
// (v_dot8_i32_i4: eight signed 4-bit products per lane and instruction, no unpacking).  A wave owns
// groups of four weight rows and walks K in 1 KB segments: lane l loads bytes [l*16, l*16+16) of
// each row's segment -- every load instruction reads 1 KB of contiguous weight bytes -- and the
// matching 16 bytes of each token's codes (shared by the four rows, L1/L2 resident).  A wave takes
// `ng` consecutive row groups as one flattened sequence of segments, so the loads of the next group
// are already in flight while the current one finishes.  The 64 partial sums of each (row, token)
// pair are added across the wave by a halving exchange (each step gives away half of the values a
// lane still holds), which costs one cross-lane move per value instead of six.
template <int MB, bool DEQ>
__global__ __launch_bounds__(256) void gemv_i4_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                      int M, int N, int Kb, int ng, int32_t* __restrict__ C,
                                                      f16* __restrict__ Y, const f16* __restrict__ sA,
                                                      const f16* __restrict__ sB, const f16* __restrict__ bias) {
    constexpr int R = 4;                                    // rows per group
    constexpr int NV = R * MB;                              // sums per group
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g0 = (blockIdx.x * 4 + wave) * ng;            // first row group of this wave
    const int groups = (N + R - 1) / R;
    if (g0 >= groups) return;
    const int gcount = groups - g0 < ng ? groups - g0 : ng;
    const int nseg = (Kb + 1023) / 1024;
    const int total = gcount * nseg;                        // flattened (group, segment) items
    const uint8_t* xp[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        const int mr = m < M ? m : M - 1;
        xp[m] = A + (int64_t)mr * Kb + lane * 16;
    }
    // which of a group's NV sums this lane stores at the end of the exchange below (log2(NV) lane
    // bits from bit 5 downwards), and its token's scale
    constexpr int LV = NV == 4 ? 2 : NV == 8 ? 3 : NV == 16 ? 4 : 5;
    const int vidx = lane >> (6 - LV);
    const int my_m = vidx / R, my_r = vidx % R;
    f16 my_sa = (f16)0;
    if (DEQ) my_sa = sA[my_m < M ? my_m : M - 1];
    struct Seg {
        u32x4 w[R], x[MB];
        f16 sb, bi;                                         // column scale and bias of the lane's output
    };
    // fetch side: position (fg, fs) runs ahead of the consume side
    int fg = 0, fs = 0;
    auto fetch = [&](Seg& g) {
        // a lane whose 16 bytes lie beyond the row end re-reads the row start and contributes nothing;
        // items past the end of the sequence re-read the last one
        const int off = (fs * 1024 + lane * 16 < Kb) ? fs * 1024 + lane * 16 : 0;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int nr = (g0 + fg) * R + r;
            nr = nr < N ? nr : N - 1;
            g.w[r] = __builtin_nontemporal_load((const u32x4*)(B + (int64_t)nr * Kb + off));
        }
#pragma unroll
        for (int m = 0; m < MB; ++m) g.x[m] = *(const u32x4*)(xp[m] - lane * 16 + off);
        // every segment carries its group's scale along: loading it at the group's end would make
        // the wave wait for everything it has in flight
        if (DEQ) {
            int col = (g0 + fg) * R + my_r;
            col = col < N ? col : N - 1;
            g.sb = sB[col];
            g.bi = (bias ? bias : sB)[col];                 // (no bias: a harmless second read of the scale)
        }
        if (fs + 1 < nseg) ++fs;
        else if (fg + 1 < gcount) { ++fg; fs = 0; }
    };
    int acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] = 0;
    int cg = 0, cs = 0;
    auto consume = [&](const Seg& g) {
        // lanes beyond the row end multiply by zero (no branch around the products: a branch here
        // makes the compiler wait for every outstanding load once per turn of the ring)
        const bool live = cs * 1024 + lane * 16 < Kb;
#pragma unroll
        for (int m = 0; m < MB; ++m)
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const int xv = live ? (int)g.x[m][d] : 0;
#pragma unroll
                for (int r = 0; r < R; ++r)
                    acc[m * R + r] = __builtin_amdgcn_sdot8((int)g.w[r][d], xv, acc[m * R + r], false);
            }
        if (++cs < nseg) return;
        // ---- end of a row group: halving exchange.  After the steps with offsets 32, 16, ... a lane
        // holds the sum of value index (bits of its lane id, most significant first) over the lanes
        // that agree with it on those bits; the remaining offsets finish the sum.
        int vals[NV];
#pragma unroll
        for (int v = 0; v < NV; ++v) vals[v] = acc[v];
        int off = 32;
#pragma unroll
        for (int cur = NV; cur > 1; cur >>= 1) {
            const bool upper = (lane & off) != 0;
#pragma unroll
            for (int i = 0; i < cur / 2; ++i) {
                const int give = upper ? vals[i] : vals[i + cur / 2];
                const int keep = upper ? vals[i + cur / 2] : vals[i];
                vals[i] = keep + __shfl_xor(give, off, QR_WAVE);
            }
            off >>= 1;
        }
        int sum = vals[0];
        for (; off > 0; off >>= 1) sum += __shfl_xor(sum, off, QR_WAVE);
        if ((lane & ((1 << (6 - LV)) - 1)) == 0) {
            const int col = (g0 + cg) * R + my_r;
            if (my_m < M && col < N) {
                if (DEQ) {
                    f16 yv = (f16)(my_sa * g.sb) * (f16)(float)sum;
                    if (bias) yv = yv + g.bi;
                    Y[(int64_t)my_m * N + col] = yv;
                } else {
                    C[(int64_t)my_m * N + col] = sum;
                }
            }
        }
#pragma unroll
        for (int v = 0; v < NV; ++v) acc[v] = 0;
        cs = 0;
        ++cg;
    };
    Seg ga, gb, gc;
    fetch(ga);
    fetch(gb);
    fetch(gc);
    int it = 0;
    for (; it + 3 <= total; it += 3) {                      // whole turns of the ring: no branch around the loads
        consume(ga);
        fetch(ga);
        consume(gb);
        fetch(gb);
        consume(gc);
        fetch(gc);
    }
    if (it < total) consume(ga);
    if (it + 1 < total) consume(gb);
}

int launch_gemv(const void* A, const void* B, int M, int N, int Kb, void* C, void* Y, const void* sA, const void* sB,
                const void* bias, hipStream_t st) {
    const int groups = (N + 3) / 4;
    // row groups per wave: about 64 KB of weights per wave, but keep >= 8 waves per CU when N allows ...
    int ng = (65536 + 4 * Kb - 1) / (4 * Kb);
    const int cus = qr_device().cus;
    while (ng > 1 && groups / ng < 8 * cus) --ng;
    // ... and, when all workgroups are resident at once (up to five per CU), a count that spreads
    // evenly over the CUs: 3.5 workgroups per CU run as long as 4.  Among ng / 2 ... 2 ng the
    // value nearest to ng whose last round over the CUs is at least 97 % full, else the fullest.
    {
        auto fill = [&](int g) {
            const int wgs = ((groups + g - 1) / g + 3) / 4;
            if (wgs > 5 * cus) return 1.0;
            return (double)wgs / (double)(((wgs + cus - 1) / cus) * cus);
        };
        int best = ng;
        double best_fill = fill(ng);
        for (int d = 1; d <= ng && best_fill < 0.97; ++d) {
            const int cand[2] = {ng - d, ng + d};
            for (int c = 0; c < 2; ++c) {
                const int g = cand[c];
                if (g < 1 || 2 * g < ng || g > 2 * ng) continue;
                const double f = fill(g);
                if (f >= 0.97 ? best_fill < 0.97 : f > best_fill) {
                    best = g;
                    best_fill = f;
                }
            }
        }
        ng = best;
    }
    const int waves = (groups + ng - 1) / ng;
    const unsigned grid = (unsigned)((waves + 3) / 4);
#define QR_GEMV(MB)                                                                                                   \
    do {                                                                                                              \
        if (Y)                                                                                                        \
            gemv_i4_kernel<MB, true><<<dim3(grid), dim3(256), 0, st>>>((const uint8_t*)A, (const uint8_t*)B, M, N, Kb, \
                                                                       ng, nullptr, (f16*)Y, (const f16*)sA,          \
                                                                       (const f16*)sB, (const f16*)bias);             \
        else                                                                                                          \
            gemv_i4_kernel<MB, false><<<dim3(grid), dim3(256), 0, st>>>((const uint8_t*)A, (const uint8_t*)B, M, N,   \
                                                                        Kb, ng, (int32_t*)C, nullptr, nullptr,        \
                                                                        nullptr, nullptr);                            \
    } while (0)
    if (M <= 1) QR_GEMV(1);
    else if (M <= 2) QR_GEMV(2);
    else if (M <= 4) QR_GEMV(4);
    else QR_GEMV(8);
#undef QR_GEMV
    return qr_launch_status();
}

int launch_decode(const void* A, const void* B, int M, int N, int Kb, void* C, void* Y, const void* sA, const void* sB,
                  const void* bias, hipStream_t st, int kw = 0) {
#define QR_DEC(MT, SB, XL, PF, KW)                                                                                          \
    do {                                                                                                              \
        constexpr int STAGE = (1 + MT) * 32 * (SB / 16), RED = MT * 4 * 64;                                           \
        constexpr size_t LDS = (size_t)8 * (STAGE > RED ? STAGE : RED) * 16;                                          \
        hipError_t e;                                                                                                 \
        if (Y) {                                                                                                      \
            auto kern = decode_i4_kernel<MT, SB, XL, PF, KW, true>;                                                       \
            e = qr_allow_dynamic_lds((const void*)kern, LDS);                                                         \
            if (e != hipSuccess) return (int)e;                                                                       \
            kern<<<dim3((unsigned)((N + 32 * (8 / KW) - 1) / (32 * (8 / KW)))), dim3(512), LDS, st>>>(                \
                (const uint8_t*)A, (const uint8_t*)B, M, N, Kb, nullptr,                                              \
                                                     (f16*)Y, (const f16*)sA, (const f16*)sB, (const f16*)bias);      \
        } else {                                                                                                      \
            auto kern = decode_i4_kernel<MT, SB, XL, PF, KW, false>;                                                      \
            e = qr_allow_dynamic_lds((const void*)kern, LDS);                                                         \
            if (e != hipSuccess) return (int)e;                                                                       \
            kern<<<dim3((unsigned)((N + 32 * (8 / KW) - 1) / (32 * (8 / KW)))), dim3(512), LDS, st>>>(                \
                (const uint8_t*)A, (const uint8_t*)B, M, N, Kb, (int32_t*)C,                                          \
                                                     nullptr, nullptr, nullptr, nullptr);                             \
        }                                                                                                             \
    } while (0)
    // a load instruction carries eight rows of X (128-byte pieces): issue only those that exist
    // K is split KW ways within a row group (8 / KW row groups per workgroup).  One workgroup is
    // resident per CU, so the launch takes rounds(workgroups / 256) times a workgroup's time, which
    // is a fixed part (start, first loads, final sum: about six steps' worth) plus its steps per wave.
    if (kw == 0) {
        kw = 8;
        const int cus = qr_device().cus;
        if (M <= 32) {
            const int steps = (Kb + 127) / 128;
            double best = 0;
            for (int c = 8; c >= 2; c >>= 1) {
                const int wgs = (N + 32 * (8 / c) - 1) / (32 * (8 / c));
                const double cost = (double)((wgs + cus - 1) / cus) * (6.0 + (double)steps / c);
                if (c == 8 || cost < best) {
                    best = cost;
                    kw = c;
                }
            }
        }
    }
    if (M <= 8) {
        if (kw == 2) QR_DEC(1, 128, 1, 3, 2);
        else if (kw == 4) QR_DEC(1, 128, 1, 3, 4);
        else QR_DEC(1, 128, 1, 3, 8);
    } else if (M <= 16) {
        if (kw == 2) QR_DEC(1, 128, 2, 3, 2);
        else if (kw == 4) QR_DEC(1, 128, 2, 3, 4);
        else QR_DEC(1, 128, 2, 3, 8);
    } else if (M <= 32) {
        if (kw == 2) QR_DEC(1, 128, 4, 3, 2);
        else if (kw == 4) QR_DEC(1, 128, 4, 3, 4);
        else QR_DEC(1, 128, 4, 3, 8);
    } else if (M <= 48) QR_DEC(2, 128, 6, 3, 8);
    else QR_DEC(2, 128, 8, 3, 8);
#undef QR_DEC
    return qr_launch_status();
}

// Row groups per workgroup for the shared-token decode kernel: the count among 4 .. 8 with the least
// work on the busiest CU (rounds of workgroups over the CUs times groups per workgroup), larger counts first
// (fewer copies of the tokens' codes).  0: too few row groups to fill the CUs this way.
int decode_xs_groups(int N) {
    const int groups = (N + 31) / 32, cus = qr_device().cus;
    int best = 0, best_cost = 0;
    for (int rg = 8; rg >= 4; --rg) {
        const int wgs = (groups + rg - 1) / rg;
        if (wgs < cus * 3 / 4) continue;
        const int cost = ((wgs + cus - 1) / cus) * rg;
        if (best == 0 || cost < best_cost) {
            best = rg;
            best_cost = cost;
        }
    }
    return best;
}

int launch_decode_xs(const void* A, const void* B, int M, int N, int Kb, void* C, void* Y, const void* sA,
                     const void* sB, const void* bias, hipStream_t st, int rg, int ksplit = 1) {
    if (ksplit > 1 && Y) return QR_E_UNSUPPORTED;           // partial sums exist only as int32
    const unsigned grid = (unsigned)((((N + 31) / 32 + rg - 1) / rg) * ksplit);
#define QR_XS(MT, R)                                                                                                  \
    do {                                                                                                              \
        constexpr int RD = 3;   /* deeper rings were measured slower (4: +3 %, 5: +6 %) */                            \
        constexpr size_t LDS = (size_t)3 * (MT * 32 * 16 + ((MT * 32 + R * 32 + 63) / 64 * 64 - MT * 32) * 8) * 16;       \
        hipError_t e;                                                                                                 \
        if (Y) {                                                                                                      \
            auto kern = decode_xs_kernel<MT, R, RD, true>;                                                            \
            e = qr_allow_dynamic_lds((const void*)kern, LDS);                                                         \
            if (e != hipSuccess) return (int)e;                                                                       \
            kern<<<dim3(grid), dim3(768), LDS, st>>>((const uint8_t*)A, (const uint8_t*)B, M, N, Kb, nullptr, (f16*)Y, \
                                                     (const f16*)sA, (const f16*)sB, (const f16*)bias, 1);            \
        } else {                                                                                                      \
            auto kern = decode_xs_kernel<MT, R, RD, false>;                                                           \
            e = qr_allow_dynamic_lds((const void*)kern, LDS);                                                         \
            if (e != hipSuccess) return (int)e;                                                                       \
            kern<<<dim3(grid), dim3(768), LDS, st>>>((const uint8_t*)A, (const uint8_t*)B, M, N, Kb, (int32_t*)C,     \
                                                     nullptr, nullptr, nullptr, nullptr, ksplit);                     \
        }                                                                                                             \
    } while (0)
#define QR_XS_R(MT)                                                                                                   \
    do {                                                                                                              \
        if (rg == 8) QR_XS(MT, 8);                                                                                    \
        else if (rg == 7) QR_XS(MT, 7);                                                                               \
        else if (rg == 6) QR_XS(MT, 6);                                                                               \
        else if (rg == 5) QR_XS(MT, 5);                                                                               \
        else QR_XS(MT, 4);                                                                                            \
    } while (0)
    if (M <= 32) QR_XS_R(1);
    else QR_XS_R(2);
#undef QR_XS_R
#undef QR_XS
    return qr_launch_status();
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
int launch_cfg(const void* A, const void* B, int M, int N, int Kb, void* C, void* Y, const void* sA, const void* sB,
               const void* bias, hipStream_t st) {
    constexpr int NT = 64 * WAVES_M * WAVES_N;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const int64_t tiles = (int64_t)tiles_m * tiles_n;
    if (tiles > 0x3fffffff) return QR_E_SHAPE;
    const int nxcd = qr_device().xcds;                      // the grid is a whole number of rounds over the XCDs
    const unsigned grid = (unsigned)((tiles + nxcd - 1) / nxcd * nxcd);
    if (Y)
        gemm_i4_kernel<BM, BN, WAVES_M, WAVES_N, true><<<dim3(grid), dim3(NT), 0, st>>>(
            (const uint8_t*)A, (const uint8_t*)B, M, N, Kb, nullptr, (f16*)Y, (const f16*)sA, (const f16*)sB,
            (const f16*)bias, tiles_m, tiles_n, nxcd);
    else
        gemm_i4_kernel<BM, BN, WAVES_M, WAVES_N, false><<<dim3(grid), dim3(NT), 0, st>>>(
            (const uint8_t*)A, (const uint8_t*)B, M, N, Kb, (int32_t*)C, nullptr, nullptr, nullptr, nullptr, tiles_m,
            tiles_n, nxcd);
    return qr_launch_status();
}

// ---- K split across workgroups (shapes with too few tiles to fill the CUs) ------------------------
// y = fp16(fp16(sA[r] * sB[c]) * fp16(acc[r, c])) (+ bias[c] as a fourth rounded operation), acc = the sum
// of `slabs` partial products: the epilogue of the fused kernels, applied to the K slices' results.
// Four columns per thread when rows are whole groups of four.
__global__ __launch_bounds__(256) void dequant_slabs_kernel(const int32_t* __restrict__ part, int slabs,
                                                            const f16* __restrict__ sA, const f16* __restrict__ sB,
                                                            const f16* __restrict__ bias, int64_t M, int64_t N,
                                                            f16* __restrict__ Y) {
    const int64_t cells = M * N;
    const int64_t stride = (int64_t)gridDim.x * 256;
    if ((N & 3) == 0) {
        for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < cells / 4; g += stride) {
            const int64_t i = g * 4, r = i / N, c = i - r * N;
            i32x4 acc = *(const i32x4*)(part + i);
            for (int s = 1; s < slabs; ++s) acc += *(const i32x4*)(part + (int64_t)s * cells + i);
            const f16 sa = sA[r];
            const f16x4 sb = *(const f16x4*)(sB + c);
            f16x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                f16 yv = (f16)(sa * sb[e]) * (f16)(float)acc[e];
                if (bias) yv = yv + bias[c + e];
                o[e] = yv;
            }
            *(f16x4*)(Y + i) = o;
        }
    } else {
        for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < cells; i += stride) {
            const int64_t r = i / N, c = i - r * N;
            int acc = part[i];
            for (int s = 1; s < slabs; ++s) acc += part[(int64_t)s * cells + i];
            f16 yv = (f16)(sA[r] * sB[c]) * (f16)(float)acc;
            if (bias) yv = yv + bias[c];
            Y[i] = yv;
        }
    }
}

// Number of K slices for the 64x256-tile kernel, 1 when the shape has no use for a split.  Only
// prompts of a few hundred tokens qualify (64 < M, fewer than 128 tiles of 128x256): decode batches
// were measured no faster split than with the decode kernel.  A small cost model in microseconds
// (6 for launch + prologue + epilogue, 2 more for the second launch, 1.0 per 256-k stage and round
// of 256 workgroups, slabs written and re-read at 4 TB/s) picks the slice count, and the split is
// used only when it promises a fifth less time.  Against a sweep of forced slice counts on
// M = 96..768, N = 4096..12288, K = 4096..28672 the model is within 10 % and picks the measured
// optimum or its neighbour (e.g. 256 x 4096 x 11008: 48 -> 26 us with four slices, 256 x 8192 x
// 28672: 119 -> 78 us with two; 512 x 4096 x 4096 and 256 x 11008 x 4096 stay unsplit).
// Decode against a weight with too few rows for the shared-token kernel to fill the CUs (70B down_proj: 8192 rows =
// 64 blocks of four groups): at 40 and more tokens each CU's intake of the tokens' codes bounds the barrier-free
// kernel.  With scratch from the caller the shared-token kernel runs with four groups per workgroup and as many K
// slices per block as fill the CUs, and dequant_slabs_kernel adds the slabs.  Measured (8192 x 28672, both launches):
// 64 tokens 35.5 -> 30.6 us, 48 tokens 31.3 -> 29.8; level at 32 and behind below that, and behind at every token count
// when K is 8192 (the slices get too short for their fixed costs): those shapes keep the barrier-free kernel.
int decode_split(int64_t M, int64_t N, int64_t Kb) {
    if (M < 40 || M > 64 || Kb < 8192 || decode_xs_groups((int)N) != 0) return 1;
    const int64_t blocks = ((N + 31) / 32 + 3) / 4, cus = qr_device().cus, all_stages = (Kb + 127) / 128;
    int64_t s = cus / blocks;
    if (s > all_stages / 16) s = all_stages / 16;
    if (s > 8) s = 8;
    return s >= 2 ? (int)s : 1;
}

int ks_split(int64_t M, int64_t N, int64_t Kb) {
    if (M <= 64) return decode_split(M, N, Kb);
    if (N <= 128) return 1;
    const int64_t tn = (N + 255) / 256;
    const int64_t cus = qr_device().cus;
    if (((M + 127) / 128) * tn >= cus / 2) return 1;
    const int64_t tiles = ((M + 63) / 64) * tn;
    const int64_t all_stages = (Kb + 127) / 128;
    const double t_unsplit = 6.0 + 1.0 * (double)all_stages * (double)((tiles + cus - 1) / cus);
    int best = 1;
    double t_best = 0.8 * t_unsplit;
    for (int64_t ks = 2; ks <= 16 && ks <= all_stages / 4; ++ks) {
        const double slabs_us = 2.0 * (double)ks * (double)M * (double)N * 4.0 / 4.0e6;
        const double t = 8.0 + 1.0 * (double)((all_stages + ks - 1) / ks) * (double)((tiles * ks + cus - 1) / cus) + slabs_us;
        if (t < t_best) {
            t_best = t;
            best = (int)ks;
        }
    }
    return best;
}

int gemm_dispatch(const void* A, const void* B, int64_t M, int64_t N, int64_t K, void* C, void* Y, const void* sA,
                  const void* sB, const void* bias, hipStream_t st, void* ws = nullptr, size_t ws_bytes = 0) {
    if (M < 0 || N < 0 || K < 0) return QR_E_SHAPE;
    if (M == 0 || N == 0) return QR_OK;
    if (K == 0 || K % 64 != 0 || K > 131008 || M > 0x7fffffff || N > 0x7fffffff) return QR_E_SHAPE;
    if (!A || !B || (!C && !Y)) return QR_E_NULL;
    if (((uintptr_t)A & 15) || ((uintptr_t)B & 15)) return QR_E_ALIGN;
    if (Y ? ((uintptr_t)Y & 7) : ((uintptr_t)C & 15)) return QR_E_ALIGN;
    const int m = (int)M, n = (int)N, kb = (int)(K / 2);
    // An operand of 4 GiB or more: every specialised kernel below addresses its operands through 32-bit offsets;
    // the plain tiled kernel computes 64-bit row addresses and takes any shape (rows beyond M or N are clamped).
    if (M * (int64_t)kb >= (1LL << 32) || N * (int64_t)kb >= (1LL << 32)) {
        if (M <= 128) return launch_cfg<128, 128, 2, 2>(A, B, m, n, kb, C, Y, sA, sB, bias, st);
        return launch_cfg<256, 256, 4, 2>(A, B, m, n, kb, C, Y, sA, sB, bias, st);
    }
    const int64_t t256 = ((M + 255) / 256) * ((N + 255) / 256);
    // one to four tokens: the dot-product kernel -- except two to four tokens against a weight with enough rows for the
    // shared-token kernel, which is ahead there (57344 x 8192: 40.2 against 42.9 us)
    if (M == 1 || (M <= 4 && decode_xs_groups(n) == 0)) return launch_gemv(A, B, m, n, kb, C, Y, sA, sB, bias, st);
    // too few tiles for the CUs: split K across workgroups when the caller passed scratch for the
    // slices' partial sums
    const int split = ks_split(M, N, kb);
    if (split > 1 && Y && ws && ws_bytes >= (size_t)split * (size_t)M * (size_t)N * 4 && ((uintptr_t)ws & 15) == 0) {
        int rc = M <= 64 ? launch_decode_xs(A, B, m, n, kb, ws, nullptr, nullptr, nullptr, nullptr, st, 4, split)
                         : launch_ks<64, 256, 1, 4>(A, B, m, n, kb, ws, nullptr, nullptr, nullptr, nullptr, st, split);
        if (rc != QR_OK) return rc;
        int64_t db = (M * N / 4 + 255) / 256;
        db = db < 1 ? 1 : (db > 4096 ? 4096 : db);
        dequant_slabs_kernel<<<dim3((unsigned)db), dim3(256), 0, st>>>((const int32_t*)ws, split, (const f16*)sA,
                                                                      (const f16*)sB, (const f16*)bias, M, N, (f16*)Y);
        return qr_launch_status();
    }
    if (M <= 64) {
        // weight streaming: with enough groups of 32 rows to fill the CUs the kernel that shares the
        // tokens' codes through LDS (they are read once per workgroup); otherwise the barrier-free
        // kernel in which the waves of a workgroup split K over groups of 32 rows
        if (const int rg = decode_xs_groups(n)) return launch_decode_xs(A, B, m, n, kb, C, Y, sA, sB, bias, st, rg);
        return launch_decode(A, B, m, n, kb, C, Y, sA, sB, bias, st);
    }
    const int64_t t128x256 = ((M + 127) / 128) * ((N + 255) / 256);
    const int64_t cus = qr_device().cus;
    if (t128x256 >= cus / 2) {
        // Taller tiles run faster per unit of work (3 unpacking instructions per MFMA at 256 rows, 3.5 at 192,
        // 4.5 at 128) but quantise worse over the 256 CUs: compare rounds of tiles, a 128x256 tile costing 0.57
        // and a 192x256 tile 0.80 of a 256x256 one (measured over 300..4096 tokens against 4096..27648 weight
        // rows: rounds of 27-29 / 40-41 / 48-51 us at K = 4096; with these ratios every one of those shapes gets
        // the fastest kernel).  Ties go to the taller tile.
        const int64_t t192 = ((M + 191) / 192) * ((N + 255) / 256);
        const double rounds256 = (double)((t256 + cus - 1) / cus);
        const double rounds192 = (double)((t192 + cus - 1) / cus) * 0.80;
        const double rounds128 = (double)((t128x256 + cus - 1) / cus) * 0.57;
        if (rounds256 <= rounds128 && rounds256 <= rounds192) return launch_sp256(A, B, m, n, kb, C, Y, sA, sB, bias, st);
        if (rounds192 <= rounds128) return launch_sp256(A, B, m, n, kb, C, Y, sA, sB, bias, st, 192);
        return launch_spk(A, B, m, n, kb, C, Y, sA, sB, bias, st);
    }
    if (N > 128) return launch_ks<64, 256, 1, 4>(A, B, m, n, kb, C, Y, sA, sB, bias, st);
    return launch_cfg<128, 128, 2, 2>(A, B, m, n, kb, C, Y, sA, sB, bias, st);
}

}  // namespace

extern "C" int qr_matmul_i4_i32(const void* A, const void* B, int64_t M, int64_t N, int64_t K, void* C, void* stream) {
    if (M > 0 && N > 0 && !C) return QR_E_NULL;
    return gemm_dispatch(A, B, M, N, K, C, nullptr, nullptr, nullptr, nullptr, (hipStream_t)stream);
}

extern "C" int qr_linear_i4_f16(const void* A, const void* sA, const void* W, const void* sW, const void* bias_or_null,
                                int64_t M, int64_t N, int64_t K, void* y, void* stream) {
    if (M > 0 && N > 0 && (!y || !sA || !sW)) return QR_E_NULL;
    return gemm_dispatch(A, W, M, N, K, nullptr, y, sA, sW, bias_or_null, (hipStream_t)stream);
}

extern "C" size_t qr_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0 || K % 64 != 0) return 0;
    const int split = ks_split(M, N, K / 2);
    return split > 1 ? (size_t)split * (size_t)M * (size_t)N * 4 : 0;
}

// ---- the entry point that allocates nothing ---------------------------------------------------------
// Slabs of int32 partial sums for the K split, held by the library itself: one array per GPU, alive
// until the process ends.  Host code must never hand the array's NAME to a kernel (in host code it is a
// stand-in, not a device address): the per-device address comes from hipGetSymbolAddress, once per
// device, and only that pointer is used afterwards.
static __device__ __align__(256) unsigned char scratch[QR_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void* scratch_ptr[kMaxDevices];                 // per device: its own copy of `scratch`, at its own address
std::mutex scratch_guard;

// Address of `scratch` on the current device (looked up on the first call on that device).
int static_scratch(void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return QR_E_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(scratch_guard);
    if (!scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return (int)hipErrorInvalidSymbol;
        scratch_ptr[dev] = p;
    }
    *out = scratch_ptr[dev];
    return QR_OK;
}
}  // namespace

extern "C" int qr_linear_i4_f16_static(const void* A, const void* sA, const void* W, const void* sW,
                                       const void* bias_or_null, int64_t M, int64_t N, int64_t K, void* y, void* stream) {
    if (M > 0 && N > 0 && (!y || !sA || !sW)) return QR_E_NULL;
    const size_t need = qr_workspace_bytes(M, N, K);
    if (need > (size_t)QR_STATIC_SCRATCH_BYTES) return QR_E_SCRATCH_LIMIT;
    void* ws = nullptr;
    if (need) {                                  // every slab cell is written before it is read: nothing to clear
        const int rc = static_scratch(&ws);
        if (rc != QR_OK) return rc;
    }
    return gemm_dispatch(A, W, M, N, K, nullptr, y, sA, sW, bias_or_null, (hipStream_t)stream, ws, need);
}

extern "C" int qr_linear_i4_f16_ws(const void* A, const void* sA, const void* W, const void* sW,
                                   const void* bias_or_null, int64_t M, int64_t N, int64_t K, void* y, void* workspace,
                                   size_t workspace_bytes, void* stream) {
    if (M > 0 && N > 0 && (!y || !sA || !sW)) return QR_E_NULL;
    return gemm_dispatch(A, W, M, N, K, nullptr, y, sA, sW, bias_or_null, (hipStream_t)stream, workspace, workspace_bytes);
}
