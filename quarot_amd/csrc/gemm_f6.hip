// int4 x int4 GEMM on the FP6 matrix path of gfx950, exact, for prefill shapes.
//
// Every int4 code -8 .. 7 is a value of FP6 E3M2 ("bf6": 1, 2, 3 = 1.5 * 2, 4 .. 7 = 1.00 .. 1.75 * 4,
// 8 = 1.0 * 8), every product is an integer of at most 64 and every partial sum an integer below 2^24
// (K < 131072), so v_mfma_scale_f32_32x32x64_f8f6f4 with both operands as bf6 and unit scales returns
// the int4 dot product exactly in fp32 -- at about 1.8 times the issue rate of the int8 instruction.
//
// The price is the operand format: 6 bits per value, and no cheap way from packed nibbles to packed
// 6-bit codes inside a GEMM loop.  Operands are therefore converted once (weights when they are
// loaded, activations by a pass behind the quantiser) into a layout made for this kernel:
//   X6 / W6: [K / 64 stages][rows][48 bytes]   -- stage-major: the 64 values of a row and stage are 48
//   contiguous bytes (two MFMA operands of 24 bytes: k 0..31 for lanes 0..31, k 32..63 for lanes 32..63),
//   and the rows of a stage are contiguous, so the 256 rows of a tile and stage are ONE 12 KB run.
// The order of the 32 values inside an operand is the converter's own (both operands use it, so every
// product pairs the same k); see f6_pack8.
#include "qr_common.h"
#include "qr_epilogue.h"

namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef unsigned long long u64;

// 6-bit E3M2 codes of the sixteen nibble values (two's complement), one byte each, as two 8-byte tables
// for v_perm_b32: nibble n < 8 -> kPos byte n, n >= 8 (value n - 16) -> kNeg byte n - 8.
//   value:  0     1     2     3     4     5     6     7        -8    -7    -6    -5    -4    -3    -2    -1
//   code :  0x00  0x0C  0x10  0x12  0x14  0x15  0x16  0x17     0x38  0x37  0x36  0x35  0x34  0x32  0x30  0x2C
constexpr u32 kPosLo = 0x12100C00u, kPosHi = 0x17161514u, kNegLo = 0x35363738u, kNegHi = 0x2C303234u;

// codes of the four nibbles held one per byte in `nib` (values 0 .. 15)
__device__ __forceinline__ u32 f6_codes4(u32 nib) {
    const u32 sel = nib & 0x07070707u;
    const u32 pos = __builtin_amdgcn_perm(kPosHi, kPosLo, sel);
    const u32 neg = __builtin_amdgcn_perm(kNegHi, kNegLo, sel);
    const u32 m = ((nib >> 3) & 0x01010101u) * 0xFFu;       // 0xFF in the bytes whose nibble is >= 8
    return (neg & m) | (pos & ~m);
}
// four code bytes -> 24 bits
__device__ __forceinline__ u32 f6_squeeze(u32 c) {
    return (c & 0x3Fu) | ((c >> 2) & 0xFC0u) | ((c >> 4) & 0x3F000u) | ((c >> 6) & 0xFC0000u);
}
// one packed word (8 nibbles) -> 48 bits: its even nibbles (k = 0, 2, 4, 6 of the word), then its odd ones
__device__ __forceinline__ u64 f6_pack8(u32 p) {
    const u32 even = f6_squeeze(f6_codes4(p & 0x0F0F0F0Fu)), odd = f6_squeeze(f6_codes4((p >> 4) & 0x0F0F0F0Fu));
    return (u64)even | ((u64)odd << 24);
}

// codes uint8 [rows, K / 2] (two nibbles per byte, even k low) -> stage-major 6-bit operands.  One thread per
// (row, 32 values): 16 bytes in, 24 bytes out.  A workgroup takes 32 rows x 8 groups: eight lanes read one
// 128-byte line of a row, and the wave's writes to one stage are 8 rows x 48 bytes in a row.
__global__ __launch_bounds__(256) void convert_i4_f6_kernel(const u32x4* __restrict__ src, int64_t rows, int groups,
                                                            u32x2* __restrict__ dst) {
    const int64_t row = (int64_t)blockIdx.y * 32 + (threadIdx.x >> 3);
    const int gr = blockIdx.x * 8 + (threadIdx.x & 7);      // 32-value group of the row: stage gr / 2, half gr % 2
    if (row >= rows || gr >= groups) return;
    const int64_t idx = row * groups + gr;
    const u32x4 p = src[idx];
    const u64 a = f6_pack8(p[0]), b = f6_pack8(p[1]), c = f6_pack8(p[2]), d = f6_pack8(p[3]);
    const u64 w0 = a | (b << 48), w1 = (b >> 16) | (c << 32), w2 = (c >> 32) | (d << 16);
    // The kernel reads an operand as 16 bytes + 8 bytes; for the second half of a row the 16-byte piece has
    // to be the aligned one (bytes 32..47), so that half is stored as [w2][w0][w1] and comes back in order.
    u32x2* out = dst + (((int64_t)(gr >> 1) * rows + row) * 6 + (gr & 1) * 3);
    const u32x2 v0 = {(u32)w0, (u32)(w0 >> 32)}, v1 = {(u32)w1, (u32)(w1 >> 32)}, v2 = {(u32)w2, (u32)(w2 >> 32)};
    if (gr & 1) {
        out[0] = v2;
        out[1] = v0;
        out[2] = v1;
    } else {
        out[0] = v0;
        out[1] = v1;
        out[2] = v2;
    }
}

// ------------------------------------------------------------------------------------------------
// TM x 256 tile (TM = 256, or 192 / 128 when taller tiles would leave compute units idle), four waves (one per
// SIMD) as 2 (M) x 2 (N), each a TM/2 x 128 wave tile = TM/64 x 4 accumulator tiles of 32 x 32.  A stage
// is 64 k: TM * 48 bytes of X6 and 12 KB of W6, each one contiguous run, loaded straight into LDS
// (buffer_load ... lds: a wave's 64 lanes fill 1 KB of consecutive LDS); six stage buffers, loads five
// stages ahead.  (At TM = 128 the X6 run is 1.5 rounds of the workgroup's 4 KB, at TM = 192 2.25: the waves
// without a share of the last round aim it past the end of the operand, which fetches nothing, and at a spare
// 2 KB of LDS, so that every wave has the same number of loads in flight and one wait count serves all.)  Rows are 48 bytes apart in LDS: the 16 rows that a quarter-wave
// reads at one offset start in 16 different groups of four banks (12 r mod 64), so the 16-byte and 8-byte
// reads that assemble an operand (24 bytes: halves of the row at byte 0 / 16 and 32 / 24) have no bank
// conflicts and nothing is padded or swizzled.  Nothing is unpacked: fragments go from LDS to the
// matrix instruction; the fragments of the next stage are read while the 16 MFMAs of the current one run.
template <int TM, bool DEQ_BIAS>
__global__ __launch_bounds__(256) void gemm_f6_kernel(const uint8_t* __restrict__ A6, const uint8_t* __restrict__ B6, int M,
                                                      int N, int stages, f16* __restrict__ Y, const f16* __restrict__ sA,
                                                      const f16* __restrict__ sB, const f16* __restrict__ bias, int tiles_m,
                                                      int tiles_n, int nxcd) {
    constexpr int NBUF = 6, AHEAD = 5;
    constexpr int IM = TM / 64;                             // accumulator tiles of a wave along M
    constexpr int ASLOTS = TM * 3, AROUNDS = (ASLOTS + 255) / 256;
    constexpr int BUF = ASLOTS + 768;                       // 16-byte slots per stage buffer: X6, then 768 of W6
    constexpr int LOADS = AROUNDS + 3;                      // loads per wave and stage
    extern __shared__ u32x4 f6_lds[];
    const int per_xcd = gridDim.x / nxcd;
    const int tile = (blockIdx.x % nxcd) * per_xcd + blockIdx.x / nxcd;
    if (tile >= tiles_m * tiles_n) return;
    constexpr int GROUP_M = 8;
    const int group_sz = GROUP_M * tiles_n;
    const int g = tile / group_sz;
    const int gm0 = g * GROUP_M;
    const int gh = (tiles_m - gm0) < GROUP_M ? (tiles_m - gm0) : GROUP_M;
    const int tm = gm0 + (tile - g * group_sz) % gh;
    const int tn = (tile - g * group_sz) / gh;
    const int m0 = tm * TM, n0 = tn * 256;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int r = lane & 31, kh = lane >> 5;

    // loads beyond the operand (rows past M or N in the last stage) return zero
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void*)A6, 0, (int)((u32)stages * (u32)M * 48u), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void*)B6, 0, (int)((u32)stages * (u32)N * 48u), 0x00020000);
    auto dma = [&](int st, int buf) {
        const int sc = st < stages ? st : stages - 1;       // past the end: repeat the last stage into a buffer nobody reads
        const u32 sa = ((u32)sc * (u32)M + (u32)m0) * 48u, sb = ((u32)sc * (u32)N + (u32)n0) * 48u;
#pragma unroll
        for (int i = 0; i < AROUNDS; ++i) {
            const bool spare = (i * 256 + 256 > ASLOTS) && wave >= (ASLOTS - i * 256) / 64;    // wave-uniform
            __attribute__((address_space(3))) void* da = (__attribute__((address_space(3))) void*)(
                spare ? f6_lds + NBUF * BUF + (wave & 1) * 64 : f6_lds + buf * BUF + i * 256 + wave * 64);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, da, 16, spare ? 0xFFFFFF00u : (u32)(tid * 16 + i * 4096),
                                                     spare ? 0u : sa, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            __attribute__((address_space(3))) void* db =
                (__attribute__((address_space(3))) void*)(f6_lds + buf * BUF + ASLOTS + i * 256 + wave * 64);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, db, 16, (u32)(tid * 16 + i * 4096), sb, 0, 0);
        }
    };
    // fragment (row, kh): 16 bytes at row * 48 + (kh ? 32 : 0) and 8 bytes at row * 48 + (kh ? 24 : 16)
    struct Frags {
        i32x8 a[IM], b[4];
    };
    const int a16 = (wm * (TM / 2) + r) * 3 + (kh ? 2 : 0), a8 = (wm * (TM / 2) + r) * 6 + (kh ? 3 : 2);
    const int b16 = ASLOTS + (wn * 128 + r) * 3 + (kh ? 2 : 0), b8 = ASLOTS * 2 + (wn * 128 + r) * 6 + (kh ? 3 : 2);
    auto read_a = [&](int buf, int t, Frags& f) {
        const u32x4 q = f6_lds[buf * BUF + a16 + t * 96];
        const u32x2 e = ((const u32x2*)f6_lds)[buf * BUF * 2 + a8 + t * 192];
        f.a[t] = i32x8{(int)q[0], (int)q[1], (int)q[2], (int)q[3], (int)e[0], (int)e[1], 0, 0};
    };
    auto read_b = [&](int buf, int t, Frags& f) {
        const u32x4 q = f6_lds[buf * BUF + b16 + t * 96];
        const u32x2 e = ((const u32x2*)f6_lds)[buf * BUF * 2 + b8 + t * 192];
        f.b[t] = i32x8{(int)q[0], (int)q[1], (int)q[2], (int)q[3], (int)e[0], (int)e[1], 0, 0};
    };
    f32x16 acc[IM][4];
#pragma unroll
    for (int i = 0; i < IM; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

#define QR_F6_BARRIER(ALLOWED) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(ALLOWED) : "memory")
    // The epilogue's scales (and bias) of this tile's columns and rows are fetched first and parked in LDS
    // behind the stage buffers, so that the epilogue finds them without waiting for memory (indices clamped
    // to the matrix: values of rows and columns beyond it are never stored).
    f16* const scale_lds = (f16*)(f6_lds + NBUF * BUF + (TM == 256 ? 0 : 128));     // [256] sB, [256] bias, [TM] sA
    const int ccol = n0 + tid < N ? n0 + tid : N - 1, crow = m0 + tid < M ? m0 + tid : M - 1;
    const f16 pre_sb = sB[ccol], pre_bi = DEQ_BIAS ? bias[ccol] : (f16)0, pre_sa = sA[crow];
#pragma unroll
    for (int s = 0; s < AHEAD; ++s) dma(s, s);
    QR_F6_BARRIER(3 * LOADS);                               // stages 0 and 1 have landed (three stages of loads may be out)
    scale_lds[tid] = pre_sb;                                // (published by the barriers of the K loop)
    scale_lds[256 + tid] = pre_bi;
    if (tid < TM) scale_lds[512 + tid] = pre_sa;
    Frags fr[2];
#pragma unroll
    for (int t = 0; t < IM; ++t) read_a(0, t, fr[0]);
#pragma unroll
    for (int t = 0; t < 4; ++t) read_b(0, t, fr[0]);
    // One stage: the IM * 4 MFMAs of `cur`, one fragment read of the next stage (already landed: the barrier
    // before this stage waited for it) behind each of the first IM + 4, the loads of stage s + 5 into the
    // buffer of stage s - 1 (last read during stage s - 2) behind the next ones.
    auto stage = [&](int s, int bnext, int bfill, const Frags& cur, Frags& nxt) {
#pragma unroll
        for (int q = 0; q < IM * 4; ++q) {
            const int i = q >> 2, j = q & 3;
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(cur.b[j], cur.a[i], acc[i][j], 3, 3, 0, 0, 0, 0);
            if (q < IM) read_a(bnext, q, nxt);
            else if (q < IM + 4) read_b(bnext, q - IM, nxt);
            if (q == (IM == 4 ? 8 : 6)) dma(s + AHEAD, bfill);
            __builtin_amdgcn_sched_barrier(0);
        }
        QR_F6_BARRIER(3 * LOADS);                                 // stage s + 2 has landed; every wave is done reading stage s
    };
    int b = 0;                                              // buffer of the current stage
    auto next = [](int v) { return v == NBUF - 1 ? 0 : v + 1; };
    auto prev = [](int v) { return v == 0 ? NBUF - 1 : v - 1; };
    int s = 0;
    for (; s + 2 <= stages; s += 2) {
        stage(s, next(b), prev(b), fr[0], fr[1]);
        b = next(b);
        stage(s + 1, next(b), prev(b), fr[1], fr[0]);
        b = next(b);
    }
    if (s < stages) {
        stage(s, next(b), prev(b), fr[0], fr[1]);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");        // the trailing repeats of the last stage
    __syncthreads();                                        // ... before the stage buffers become output slabs

    // ---- epilogue: lane l, register v -> column (v/4)*8 + (l/32)*4 + v%4 of the W tile, token l%32
    f16x4 sbh[4][4], bih[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
            const int c = wn * 128 + j * 32 + gq * 8 + kh * 4;
            sbh[j][gq] = *(const f16x4*)(scale_lds + c);
            bih[j][gq] = *(const f16x4*)(scale_lds + 256 + c);
        }
    const bool lines = (N & 7) == 0 && (((uintptr_t)Y) & 15) == 0;
#pragma unroll
    for (int i = 0; i < IM; ++i) {
        const int row0 = m0 + wm * (TM / 2) + i * 32;
        const int row = row0 + r;
        const f16 sa = scale_lds[512 + wm * (TM / 2) + i * 32 + r];
#pragma unroll
        for (int jb = 0; jb < 4; jb += 2) {
            const int col0 = n0 + wn * 128 + jb * 32;
            f16x4 o[2][4];
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                for (int gq = 0; gq < 4; ++gq)
                    o[jj][gq] = dequant4_f32(acc[i][jb + jj][gq * 4], acc[i][jb + jj][gq * 4 + 1], acc[i][jb + jj][gq * 4 + 2],
                                             acc[i][jb + jj][gq * 4 + 3], sa, sbh[jb + jj][gq], bih[jb + jj][gq], DEQ_BIAS);
            if (lines && col0 + 64 <= N) {                  // (a last row tile stores the rows that exist)
                store_slab_rows<2>((u32x2*)(f6_lds + wave * 256), o, lane, Y + (int64_t)row0 * N + col0, N, M - row0);
            } else if (row < M) {
#pragma unroll
                for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                    for (int gq = 0; gq < 4; ++gq) {
                        const int col = col0 + jj * 32 + gq * 8 + kh * 4;
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (col + e < N) Y[(int64_t)row * N + col + e] = o[jj][gq][e];
                    }
            }
        }
    }
#undef QR_F6_BARRIER
}

}  // namespace

extern "C" size_t qr_f6_bytes(int64_t rows, int64_t K) {
    if (rows <= 0 || K <= 0 || K % 64 != 0) return 0;
    return (size_t)rows * (size_t)K / 4 * 3;
}

extern "C" int qr_convert_i4_f6(const void* codes, int64_t rows, int64_t K, void* out, void* stream) {
    if (rows < 0 || K < 0) return QR_E_SHAPE;
    if (rows == 0 || K == 0) return QR_OK;
    if (K % 64 != 0 || K > 131008 || rows > 0x7fffffff) return QR_E_SHAPE;
    if (!codes || !out) return QR_E_NULL;
    if (((uintptr_t)codes & 15) || ((uintptr_t)out & 7)) return QR_E_ALIGN;
    const int groups = (int)(K / 32);
    const int64_t row_blocks = (rows + 31) / 32;
    if (row_blocks > 65535) return QR_E_UNSUPPORTED;        // more than 2 097 120 rows (grid.y)
    convert_i4_f6_kernel<<<dim3((unsigned)((groups + 7) / 8), (unsigned)row_blocks), dim3(256), 0, (hipStream_t)stream>>>(
        (const u32x4*)codes, rows, groups, (u32x2*)out);
    return qr_launch_status();
}

extern "C" int qr_linear_f6_f16(const void* A6, const void* sA, const void* W6, const void* sW, const void* bias_or_null,
                                int64_t M, int64_t N, int64_t K, void* y, void* stream) {
    if (M < 0 || N < 0 || K < 0) return QR_E_SHAPE;
    if (M == 0 || N == 0) return QR_OK;
    if (K == 0 || K % 64 != 0 || K > 131008 || M > 0x7fffffff || N > 0x7fffffff) return QR_E_SHAPE;
    if (!A6 || !W6 || !sA || !sW || !y) return QR_E_NULL;
    if (((uintptr_t)A6 & 15) || ((uintptr_t)W6 & 15) || ((uintptr_t)y & 7)) return QR_E_ALIGN;
    // operands are addressed through 32-bit buffer offsets
    if ((double)M * (double)K * 0.75 >= 4294901760.0 || (double)N * (double)K * 0.75 >= 4294901760.0) return QR_E_UNSUPPORTED;
    const int nxcd = qr_device().xcds, cus = qr_device().cus;
    const int tiles_n = (int)((N + 255) / 256);
    // 256-row tiles unless 192- or 128-row ones fill the device in fewer rounds (measured on single rounds at
    // K = 4096 .. 13824: a 128-row tile costs 0.73 and a 192-row tile 0.87 of a 256-row one); ties go to the
    // taller tile
    const int64_t t256 = (M + 255) / 256 * tiles_n, t192 = (M + 191) / 192 * tiles_n, t128 = (M + 127) / 128 * tiles_n;
    const double r256 = (double)((t256 + cus - 1) / cus), r192 = (double)((t192 + cus - 1) / cus) * 0.87,
                 r128 = (double)((t128 + cus - 1) / cus) * 0.73;
    int tm_rows = (r256 <= r192 && r256 <= r128) ? 256 : (r192 <= r128 ? 192 : 128);
    const int tiles_m = (int)((M + tm_rows - 1) / tm_rows);
    const int64_t tiles = (int64_t)tiles_m * tiles_n;
    if (tiles > 0x3fffffff) return QR_E_SHAPE;
    const unsigned grid = (unsigned)((tiles + nxcd - 1) / nxcd * nxcd);
    hipStream_t st = (hipStream_t)stream;
    auto launch = [&](auto kernel, size_t lds) -> int {
        hipError_t e = qr_allow_dynamic_lds((const void*)kernel, lds);
        if (e != hipSuccess) return (int)e;
        kernel<<<dim3(grid), dim3(256), lds, st>>>((const uint8_t*)A6, (const uint8_t*)W6, (int)M, (int)N, (int)(K / 64), (f16*)y,
                                                   (const f16*)sA, (const f16*)sW, (const f16*)bias_or_null, tiles_m, tiles_n, nxcd);
        return qr_launch_status();
    };
    // six stage buffers (+ the spare 2 KB that idle loads of 128- and 192-row tiles aim at) + 1.5 KB of scales for the epilogue
    constexpr size_t LDS256 = (size_t)(6 * (768 + 768) + 96) * 16, LDS192 = (size_t)(6 * (576 + 768) + 128 + 96) * 16,
                     LDS128 = (size_t)(6 * (384 + 768) + 128 + 96) * 16;
    if (tm_rows == 128) return bias_or_null ? launch(gemm_f6_kernel<128, true>, LDS128) : launch(gemm_f6_kernel<128, false>, LDS128);
    if (tm_rows == 192) return bias_or_null ? launch(gemm_f6_kernel<192, true>, LDS192) : launch(gemm_f6_kernel<192, false>, LDS192);
    return bias_or_null ? launch(gemm_f6_kernel<256, true>, LDS256) : launch(gemm_f6_kernel<256, false>, LDS256);
}
