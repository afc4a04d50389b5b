// Online Hadamard transform  y = x . (hadK (x) H_m)^T * scale  along rows of length n = K * m,
// optionally fused with the per-token int4 quantiser.
//
// One workgroup (256 threads) owns one row at a time; the row lives in LDS as fp32.
//   phase 1  global -> registers: each thread takes 16-byte chunks of 8 elements; butterflies on
//            index bits 0..2 in registers, on bits 3..8 across lanes (DPP / swizzle / permute);
//            result written to LDS.
//   phase 2  remaining power-of-two bits (m > 512) by in-LDS radix-8/16 passes on float4 vectors.
//   phase 3  (K > 1) the K x K factor on the matrix cores: Y[K, m] = hadK[K, K] . T[K, m] with T
//            rounded to fp16 (fp16 staging) or split into fp16 hi + lo (fp32 mode), fp32 accumulate,
//            written back in place.
//   phase 4  LDS -> global: round to the I/O type; when fused, row abs-max -> scale -> int4 codes.
#include "qr_common.h"

namespace {

constexpr int HT = 256;
constexpr int KS_MAX = 6;        // contraction steps of 32: hadK order <= 192

// ---- cross-lane exchange: value held by lane (id ^ MASK) ---------------------------------------
template <int MASK>
__device__ __forceinline__ float lane_xor(float v) {
    int i = __builtin_bit_cast(int, v);
    int r;
    if constexpr (MASK == 1) r = __builtin_amdgcn_mov_dpp(i, 0xB1, 0xF, 0xF, true);         // quad_perm [1,0,3,2]
    else if constexpr (MASK == 2) r = __builtin_amdgcn_mov_dpp(i, 0x4E, 0xF, 0xF, true);    // quad_perm [2,3,0,1]
    else if constexpr (MASK == 4) r = __builtin_amdgcn_ds_swizzle(i, 0x101F);               // xor 4 within 32 lanes
    else if constexpr (MASK == 8) r = __builtin_amdgcn_mov_dpp(i, 0x128, 0xF, 0xF, true);   // row_ror:8 == xor 8
    else if constexpr (MASK == 16) r = __builtin_amdgcn_ds_swizzle(i, 0x401F);              // xor 16 within 32 lanes
    else r = __shfl_xor(i, MASK, QR_WAVE);
    return __builtin_bit_cast(float, r);
}

template <int MASK>
__device__ __forceinline__ void lane_stage(float (&v)[8], int lane) {
    const float sgn = (lane & MASK) != 0 ? -1.0f : 1.0f;     // upper lane of a pair: partner - own
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float p = lane_xor<MASK>(v[e]);
        v[e] = __builtin_fmaf(v[e], sgn, p);
    }
}

__device__ __forceinline__ void reg_fwht8(float (&v)[8]) {
#pragma unroll
    for (int h = 1; h < 8; h <<= 1)
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if ((i & h) == 0) {
                float a = v[i], b = v[i | h];
                v[i] = a + b;
                v[i | h] = a - b;
            }
}

__device__ __forceinline__ void load8(const f16* p, float (&v)[8]) {
    u32x4 raw = *((const u32x4*)p);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = (float)f16_from_bits((unsigned short)(raw[i] & 0xffffu));
        v[2 * i + 1] = (float)f16_from_bits((unsigned short)(raw[i] >> 16));
    }
}
__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
    f32x4 a = *((const f32x4*)p);
    f32x4 b = *((const f32x4*)p + 1);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[i] = a[i];
        v[i + 4] = b[i];
    }
}

// fp16 rounding of 8 floats, packed two per word (element 0 in the low half)
__device__ __forceinline__ u32x4 to_f16x8(const float (&v)[8]) {
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        o[i] = narrow_f16x2(v[2 * i], v[2 * i + 1]);
    return o;
}

// In-LDS butterflies on index bits [b, b + R_LOG2) for every float4 vector of the row.
template <int R_LOG2>
__device__ __forceinline__ void lds_pass(float* buf, int n, int b) {
    constexpr int R = 1 << R_LOG2;
    const int stride = 1 << b;              // floats
    const int vecs_low = stride >> 2;       // float4 vectors below bit b
    const int items = n >> (2 + R_LOG2);
    for (int g = threadIdx.x; g < items; g += HT) {
        const int lowv = g & (vecs_low - 1);
        const int high = g / vecs_low;
        float* base = buf + ((int64_t)high << (b + R_LOG2)) + lowv * 4;
        f32x4 v[R];
#pragma unroll
        for (int j = 0; j < R; ++j) v[j] = *(const f32x4*)(base + j * stride);
#pragma unroll
        for (int h = 1; h < R; h <<= 1)
#pragma unroll
            for (int j = 0; j < R; ++j)
                if ((j & h) == 0) {
                    f32x4 a = v[j], c = v[j | h];
                    v[j] = a + c;
                    v[j | h] = a - c;
                }
#pragma unroll
        for (int j = 0; j < R; ++j) *(f32x4*)(base + j * stride) = v[j];
    }
}

// IO: element type of x and y.  MODE32: keep fp32 precision through the hadK stage (hadK is fp32);
// otherwise round the power-of-two stage to fp16 first (hadK is fp16).  QUANT: quantise the fp16
// rounding of the result (q, scales), y optional.
template <typename IO, bool MODE32, bool QUANT>
__global__ __launch_bounds__(HT) void hadamard_kernel(const IO* __restrict__ x, IO* __restrict__ y, int64_t rows, int n,
                                                      int K, int log2m, const void* __restrict__ hadK, float scale,
                                                      float clip, u32* __restrict__ q, f16* __restrict__ scales,
                                                      int hs_stride) {
    extern __shared__ f32x4 smem_raw[];
    float* buf = (float*)smem_raw;                      // [n] fp32 working row
    f16* Hs = (f16*)(buf + n);                          // [Kr][hs_stride] zero-padded hadK, fp16
    __shared__ u32 red[HT / QR_WAVE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m = 1 << log2m;
    const int nchunks = n >> 3;
    const int Kr = (K + 15) & ~15;
    const int ksteps = (K + 31) >> 5;

    if (K > 1) {
        // stage hadK once per workgroup, padded with zeros to [Kr][hs_stride]
        for (int idx = tid; idx < Kr * hs_stride; idx += HT) {
            const int r = idx / hs_stride, c = idx - r * hs_stride;
            f16 h = (f16)0;
            if (r < K && c < K) h = MODE32 ? (f16)((const float*)hadK)[r * K + c] : ((const f16*)hadK)[r * K + c];
            Hs[idx] = h;
        }
    }
    const int lane_stages = log2m - 3 < 6 ? log2m - 3 : 6;

    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const IO* xr = x + row * (int64_t)n;
        __syncthreads();        // previous row's phase 4 (and the hadK staging) done before buf is overwritten
        // ---- phase 1 (loads issued four chunks ahead of their use)
        for (int c0 = 0; c0 < nchunks; c0 += 4 * HT) {
            float v[4][8];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int c = c0 + u * HT + tid;
                if (c < nchunks) load8(xr + (int64_t)c * 8, v[u]);
                else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[u][e] = 0.f;
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                // whole waves share `live`: nchunks % 64 != 0 only when m < 512, and then the
                // exchanges stay inside a segment's lanes, which are all live or all dead
                const int c = c0 + u * HT + tid;
                if (c0 + u * HT >= nchunks) break;
                reg_fwht8(v[u]);
                if (lane_stages > 0) lane_stage<1>(v[u], lane);
                if (lane_stages > 1) lane_stage<2>(v[u], lane);
                if (lane_stages > 2) lane_stage<4>(v[u], lane);
                if (lane_stages > 3) lane_stage<8>(v[u], lane);
                if (lane_stages > 4) lane_stage<16>(v[u], lane);
                if (lane_stages > 5) lane_stage<32>(v[u], lane);
                if (c < nchunks) {
                    *(f32x4*)(buf + c * 8) = f32x4{v[u][0], v[u][1], v[u][2], v[u][3]};
                    *(f32x4*)(buf + c * 8 + 4) = f32x4{v[u][4], v[u][5], v[u][6], v[u][7]};
                }
            }
        }
        __syncthreads();
        // ---- phase 2: bits 9 .. log2m-1
        for (int b = 9; b < log2m;) {
            const int left = log2m - b;
            if (left >= 4 && left != 6 && left != 5) { lds_pass<4>(buf, n, b); b += 4; }
            else if (left >= 3) { lds_pass<3>(buf, n, b); b += 3; }
            else if (left == 2) { lds_pass<2>(buf, n, b); b += 2; }
            else { lds_pass<1>(buf, n, b); b += 1; }
            __syncthreads();
        }
        // ---- phase 3: hadK factor on the matrix cores, in place
        if (K > 1) {
            const int col_tiles = (m + 15) >> 4;
            const int row_tiles = Kr >> 4;
            const int kq = lane >> 4;
            for (int ct = wave; ct < col_tiles; ct += HT / QR_WAVE) {
                const int r = ct * 16 + (lane & 15);
                const bool rin = r < m;
                f16x8 bh[KS_MAX], bl[KS_MAX];
#pragma unroll
                for (int ks = 0; ks < KS_MAX; ++ks) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const int k = ks * 32 + kq * 8 + j;
                        float t = 0.f;
                        if (ks < ksteps && k < K && rin) t = buf[k * m + r] * scale;
                        f16 hi = narrow_f16(t);
                        bh[ks][j] = hi;
                        if (MODE32) bl[ks][j] = (f16)(t - (float)hi);
                    }
                }
                for (int rt = 0; rt < row_tiles; ++rt) {
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
                    const f16* hrow = Hs + (rt * 16 + (lane & 15)) * hs_stride + kq * 8;
#pragma unroll
                    for (int ks = 0; ks < KS_MAX; ++ks) {
                        if (ks < ksteps) {
                            f16x8 a = *(const f16x8*)(hrow + ks * 32);
                            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bh[ks], acc, 0, 0, 0);
                            if (MODE32) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bl[ks], acc, 0, 0, 0);
                        }
                    }
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int kp = rt * 16 + kq * 4 + v;
                        if (kp < K && rin) buf[kp * m + r] = acc[v];
                    }
                }
            }
            __syncthreads();
        }
        // ---- phase 4
        const float osc = K > 1 ? 1.0f : scale;
        if (QUANT) {
            u32 mx = 0;
            for (int c = tid; c < nchunks; c += HT) {
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = buf[c * 8 + e] * osc;
                u32x4 h = to_f16x8(v);
                u32 mc = absmax_bits8(h);
                mx = mx > mc ? mx : mc;
            }
            mx = wave_max_u32(mx);
            if (lane == 0) red[wave] = mx;
            __syncthreads();
#pragma unroll
            for (int w = 0; w < HT / QR_WAVE; ++w) mx = mx > red[w] ? mx : red[w];
            const f16 sh = quantizer_scale(f16_from_bits((unsigned short)mx), clip);
            if (tid == 0) scales[row] = sh;
            const float s = (float)sh;
            const bool lean = fast_quant_ok(mx, s);
            const FastRecip fr = make_fast_recip(lean ? s : 1.0f);
            const bool fast = scale_fast_ok(s);
            const float rs = fast ? 1.0f / s : 0.0f;
            for (int c = tid; c < nchunks; c += HT) {
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = buf[c * 8 + e] * osc;
                u32x4 h = to_f16x8(v);
                q[row * (int64_t)nchunks + c] = lean ? sym_codes8_fast(h, fr) : sym_codes8(h, s, rs, fast);
                if (y) __builtin_nontemporal_store(h, (u32x4*)((f16*)y + row * (int64_t)n) + c);
            }
        } else {
            IO* yr = y + row * (int64_t)n;
            for (int c = tid; c < nchunks; c += HT) {
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = buf[c * 8 + e] * osc;
                if constexpr (sizeof(IO) == 2) {
                    __builtin_nontemporal_store(to_f16x8(v), (u32x4*)yr + c);
                } else {
                    __builtin_nontemporal_store(f32x4{v[0], v[1], v[2], v[3]}, (f32x4*)yr + 2 * c);
                    __builtin_nontemporal_store(f32x4{v[4], v[5], v[6], v[7]}, (f32x4*)yr + 2 * c + 1);
                }
            }
        }
    }
}

// ---- K > 1 with a short power-of-two factor (16 <= m <= 256), fp16 I/O -------------------------
// The butterflies need no LDS (a segment spans at most 32 lanes); hadK lives in REGISTERS as MFMA
// A-fragments (each wave owns every fourth 16-row tile), which leaves LDS for two small fp16
// arrays -- the transposed, scaled, fp16-rounded T (so a B-fragment is one 16-byte read) and the
// result -- and lets several workgroups share a CU.  The next row's global loads are issued before
// the matrix stage of the current one.
constexpr int RT_W = 3;          // 16-row tiles per wave: hadK order <= 192

template <bool MODE32, bool QUANT, int NCH>
__global__ __launch_bounds__(HT) void hadamard_km_kernel(const f16* __restrict__ x, f16* __restrict__ y, int64_t rows,
                                                         int n, int K, int log2m, const void* __restrict__ hadK,
                                                         float scale, float clip, u32* __restrict__ q,
                                                         f16* __restrict__ scales) {
    extern __shared__ f32x4 smem_raw[];
    __shared__ u32 red[HT / QR_WAVE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m = 1 << log2m;
    const int nchunks = n >> 3;
    const int Kc = (K + 31) & ~31;
    const int TS = Kc + 8;                       // halves per row of Tt (row = one column r of T)
    const int YS = m + 8;                        // halves per row of Yl (row = one output k')
    const int ksteps = Kc >> 5;
    const int row_tiles = (K + 15) >> 4;
    f16* Tt = (f16*)smem_raw;                    // [m][TS]; 8-half blocks XOR-swizzled by (r >> 3) & 3
    f16* Tlo = Tt + m * TS;                      // second plane, fp32 mode only
    f16* Yl = Tt + (MODE32 ? 2 : 1) * m * TS;    // [K][YS]
    const int kq = lane >> 4;

    // hadK -> A-fragments in registers (zero padded)
    f16x8 hf[RT_W][KS_MAX];
#pragma unroll
    for (int t = 0; t < RT_W; ++t) {
        const int hr = (wave + 4 * t) * 16 + (lane & 15);
#pragma unroll
        for (int ks = 0; ks < KS_MAX; ++ks)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int hc = ks * 32 + kq * 8 + j;
                f16 h = (f16)0;
                if (hr < K && hc < K)
                    h = MODE32 ? (f16)((const float*)hadK)[hr * K + hc] : ((const f16*)hadK)[hr * K + hc];
                hf[t][ks][j] = h;
            }
    }
    // the padding of Tt (k >= K) is never written afterwards: clear everything once
    for (int i = tid; i < ((MODE32 ? 2 : 1) * m * TS) / 8; i += HT) ((u32x4*)Tt)[i] = u32x4{0, 0, 0, 0};

    const int lane_stages = log2m - 3;
    u32x4 raw[NCH];
    int64_t row = blockIdx.x;
    if (row < rows) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + i * HT;
            raw[i] = c < nchunks ? *((const u32x4*)(x + row * (int64_t)n) + c) : u32x4{0, 0, 0, 0};
        }
    }
    __syncthreads();
    for (; row < rows; row += gridDim.x) {
        // ---- phase 1: butterflies in registers and across lanes, scatter to Tt
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + i * HT;
            if (i * HT >= nchunks) break;
            float v[8];
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                v[2 * w] = (float)f16_from_bits((unsigned short)(raw[i][w] & 0xffffu));
                v[2 * w + 1] = (float)f16_from_bits((unsigned short)(raw[i][w] >> 16));
            }
            reg_fwht8(v);
            if (lane_stages > 0) lane_stage<1>(v, lane);
            if (lane_stages > 1) lane_stage<2>(v, lane);
            if (lane_stages > 2) lane_stage<4>(v, lane);
            if (lane_stages > 3) lane_stage<8>(v, lane);
            if (lane_stages > 4) lane_stage<16>(v, lane);
            if (c < nchunks) {
                const int k = (c * 8) >> log2m;
                const int r0 = (c * 8) & (m - 1);
                const int pb = (k >> 3) ^ ((r0 >> 3) & 3);
                f16* dst = Tt + r0 * TS + pb * 8 + (k & 7);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float t = v[e] * scale;
                    const f16 hi = narrow_f16(t);
                    dst[e * TS] = hi;
                    if (MODE32) dst[e * TS + m * TS] = (f16)(t - (float)hi);
                }
            }
        }
        // next row's loads fly during the matrix stage
        const int64_t nrow = row + gridDim.x;
        if (nrow < rows) {
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int c = tid + i * HT;
                raw[i] = c < nchunks ? *((const u32x4*)(x + nrow * (int64_t)n) + c) : u32x4{0, 0, 0, 0};
            }
        }
        __syncthreads();
        // ---- phase 3: Y[K, m] = hadK . T on the matrix cores
        for (int ct = 0; ct < (m >> 4); ++ct) {
            const int r = ct * 16 + (lane & 15);
            const int sw = (r >> 3) & 3;
            f16x8 bh[KS_MAX], bl[KS_MAX];
#pragma unroll
            for (int ks = 0; ks < KS_MAX; ++ks)
                if (ks < ksteps) {
                    const int off = r * TS + (((ks << 2) + kq) ^ sw) * 8;
                    bh[ks] = *(const f16x8*)(Tt + off);
                    if (MODE32) bl[ks] = *(const f16x8*)(Tlo + off);
                }
#pragma unroll
            for (int t = 0; t < RT_W; ++t) {
                const int rt = wave + 4 * t;
                if (rt < row_tiles) {
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < KS_MAX; ++ks)
                        if (ks < ksteps) {
                            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(hf[t][ks], bh[ks], acc, 0, 0, 0);
                            if (MODE32) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(hf[t][ks], bl[ks], acc, 0, 0, 0);
                        }
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int kp = rt * 16 + kq * 4 + v;
                        if (kp < K) Yl[kp * YS + r] = (f16)acc[v];
                    }
                }
            }
        }
        __syncthreads();
        // ---- phase 4: Yl -> global (and the quantiser)
        if (QUANT) {
            u32 mx = 0;
            for (int c = tid; c < nchunks; c += HT) {
                const u32x4 h = *(const u32x4*)(Yl + ((c * 8) >> log2m) * YS + ((c * 8) & (m - 1)));
                const u32 mc = absmax_bits8(h);
                mx = mx > mc ? mx : mc;
            }
            mx = wave_max_u32(mx);
            if (lane == 0) red[wave] = mx;
            __syncthreads();
#pragma unroll
            for (int w = 0; w < HT / QR_WAVE; ++w) mx = mx > red[w] ? mx : red[w];
            const f16 sh = quantizer_scale(f16_from_bits((unsigned short)mx), clip);
            if (tid == 0) scales[row] = sh;
            const float s = (float)sh;
            const bool lean = fast_quant_ok(mx, s);
            const FastRecip fr = make_fast_recip(lean ? s : 1.0f);
            const bool fast = scale_fast_ok(s);
            const float rs = fast ? 1.0f / s : 0.0f;
            for (int c = tid; c < nchunks; c += HT) {
                const u32x4 h = *(const u32x4*)(Yl + ((c * 8) >> log2m) * YS + ((c * 8) & (m - 1)));
                q[row * (int64_t)nchunks + c] = lean ? sym_codes8_fast(h, fr) : sym_codes8(h, s, rs, fast);
                if (y) __builtin_nontemporal_store(h, (u32x4*)(y + row * (int64_t)n) + c);
            }
        } else {
            for (int c = tid; c < nchunks; c += HT) {
                const u32x4 h = *(const u32x4*)(Yl + ((c * 8) >> log2m) * YS + ((c * 8) & (m - 1)));
                __builtin_nontemporal_store(h, (u32x4*)(y + row * (int64_t)n) + c);
            }
        }
        // red[] and Yl are next written after the barrier that follows the next phase 1
    }
}

template <bool MODE32, bool QUANT>
int launch_hadamard_km(const void* x, void* y, int64_t rows, int n, int K, int log2m, const void* hadK, float scale,
                       float clip, void* q, void* scales, hipStream_t st) {
    const int m = 1 << log2m;
    const int Kc = (K + 31) & ~31;
    const size_t lds = (size_t)(MODE32 ? 2 : 1) * m * (Kc + 8) * 2 + (size_t)K * (m + 8) * 2;
    const int nch = ((n >> 3) + HT - 1) / HT;
#define QR_KM(NCH)                                                                                                    \
    do {                                                                                                              \
        auto kern = hadamard_km_kernel<MODE32, QUANT, NCH>;                                                           \
        if (lds > 48 * 1024) {                                                                                        \
            hipError_t e = qr_allow_dynamic_lds((const void*)kern, lds); \
            if (e != hipSuccess) return (int)e;                                                                       \
        }                                                                                                             \
        const int64_t cap = (int64_t)qr_device().cus * qr_blocks_per_cu((const void*)kern, HT, lds);                                     \
        const unsigned grid = (unsigned)(rows < cap ? rows : cap);                                                    \
        kern<<<dim3(grid), dim3(HT), lds, st>>>((const f16*)x, (f16*)y, rows, n, K, log2m, hadK, scale, clip, (u32*)q, \
                                                (f16*)scales);                                                        \
    } while (0)
    if (nch <= 2) QR_KM(2);
    else if (nch <= 4) QR_KM(4);
    else if (nch <= 6) QR_KM(6);
    else if (nch <= 8) QR_KM(8);
    else QR_KM(16);
#undef QR_KM
    return qr_launch_status();
}

// true when the register-resident-hadK kernel applies
bool km_applies(int n, int K, bool mode32) {
    if (K <= 1) return false;
    const int m = n / K;
    if (m < 16 || m > 256) return false;
    const int Kc = (K + 31) & ~31;
    const size_t lds = (size_t)(mode32 ? 2 : 1) * m * (Kc + 8) * 2 + (size_t)K * (m + 8) * 2;
    return lds <= 150 * 1024 && (n >> 3) <= 16 * HT;
}

// ---- K > 1, m = 64 or 128, fp16 I/O: both factors on the matrix cores ---------------------------
// Per row (token), with X viewed as [K, m]:
//   stage 1   T = X . H_m            A-fragments straight from global memory (a lane's 8 consecutive
//                                    r of one k are 16 contiguous bytes), H_m fragments generated in
//                                    registers from popcount parity.  The accumulator of two 16-row
//                                    tiles, scaled and rounded to fp16, IS one 32-deep fragment of T
//                                    for stage 2 when the contraction index is taken in the order
//                                    k = 32 s + 16 (j / 4) + 4 (lane / 16) + j % 4 -- no transposition;
//                                    it goes to LDS as one 16-byte write per lane.
//   stage 2   Y^T = T^T . hadK^T     hadK fragments (same k order) live in registers, each wave owns
//                                    every fourth 16-row tile of hadK and reads all of T from LDS;
//                                    a lane ends with 4 consecutive r of one output k: 8-byte writes
//                                    into the fp16 result row in LDS.
//   stage 3   result row -> global, with the quantiser when fused.
template <bool MODE32, bool QUANT, int LOG2M, int KS2, bool XLDS>
__global__ __launch_bounds__(HT) void hadamard_mm_kernel(const f16* __restrict__ x, f16* __restrict__ y, int64_t rows,
                                                         int n, int K, const void* __restrict__ hadK, float scale,
                                                         float clip, u32* __restrict__ q, f16* __restrict__ scales,
                                                         int ident) {
    constexpr int M_ = 1 << LOG2M;
    constexpr int KS1 = M_ / 32;                 // contraction steps of stage 1
    constexpr int CT = M_ / 16;                  // 16-column tiles of T / Y
    constexpr int NCT = CT / 4;                  // column tiles per wave in stage 1
    constexpr int YS = M_ + 8;                   // halves per row of Yl
    // Rows of m = 64: a whole row of stage-1 fragments (KS2 tile pairs) is kept in registers and
    // each pair is re-requested for the NEXT row as soon as it has been consumed, so global loads
    // run one full row ahead.  m = 128 would need twice the registers: one pair ahead only.
    constexpr bool FULL_ROW = (M_ == 64);
    constexpr int SLOTS = FULL_ROW ? KS2 : 2;
    extern __shared__ f32x4 smem_raw[];
    __shared__ u32 red[2 * (HT / QR_WAVE)];       // per-wave row maxima, double-buffered by row parity
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int nchunks = n >> 3;
    const int row_tiles = (K + 15) >> 4;
    u32x4* Tl = (u32x4*)smem_raw;                              // [CT][KS2][64 lanes] fragments of T (hi plane)
    u32x4* Tlo = Tl + CT * KS2 * 64;                           // lo plane (fp32 mode)
    f16* Yl = (f16*)(Tl + (MODE32 ? 2 : 1) * CT * KS2 * 64);   // [K][YS]
    // XLDS: the input row is fetched with fully coalesced 16-byte loads (consecutive lanes,
    // consecutive addresses), one row ahead in registers, and staged in LDS, from where the stage-1
    // fragments are read; fragment loads straight from global memory touch sixteen different lines
    // per instruction and were measured to bound the kernel.  Xl: [32 KS2 rows][PPR 16-byte pieces],
    // piece index XOR-keyed by the row so that the sixteen rows of a fragment read spread over all
    // bank groups; rows K.. are zero.
    constexpr int PPR = M_ / 8;
    constexpr int NCH = KS2 * M_ / 64;          // 16-byte chunks per thread: n / 8 <= 32 KS2 M_ / 8
    u32x4* Xl = (u32x4*)(Yl + ((K * YS + 7) & ~7));
    auto xslot = [](int row, int piece) { return row * PPR + (piece ^ ((PPR == 8 ? row >> 1 : row) & (PPR - 1))); };
    u32x4 xr[XLDS ? NCH : 1];
    auto load_row = [&](const f16* src) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            int c = tid + i * HT;
            c = c < nchunks ? c : nchunks - 1;
            xr[i] = *((const u32x4*)src + c);
        }
    };
    auto deposit_row = [&]() {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + i * HT;
            if (c < nchunks) Xl[xslot(c / PPR, c % PPR)] = xr[i];
        }
    };
    if (XLDS) {
        for (int i = K * PPR + tid; i < KS2 * 32 * PPR; i += HT) Xl[i] = u32x4{0, 0, 0, 0};
    }

    // hadK fragments, contraction index in the stage-1 accumulator order: for each (step, half) a
    // lane needs 4 consecutive k -- one 8-byte (fp16) or 16-byte (fp32) load (every order is a
    // multiple of 4, so a group of 4 is inside or outside the matrix as a whole)
    f16x8 hf[RT_W][KS2];
#pragma unroll
    for (int t = 0; t < RT_W; ++t) {
        const int hr = (wave + 4 * t) * 16 + l16;
#pragma unroll
        for (int ks = 0; ks < KS2; ++ks)
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                const int hc = ks * 32 + hh * 16 + g * 4;
                f16x4 v = {(f16)0, (f16)0, (f16)0, (f16)0};
                if (hr < K && hc < K) {
                    if (hadK == nullptr) {
                        // power-of-two row: the outer factor is the Sylvester matrix of order K itself
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = (__builtin_popcount(hr & (hc + e)) & 1) ? (f16)-1.0f : (f16)1.0f;
                    } else if (MODE32) {
                        const f32x4 w = *(const f32x4*)((const float*)hadK + hr * K + hc);
                        v = f16x4{(f16)w[0], (f16)w[1], (f16)w[2], (f16)w[3]};
                    } else {
                        v = *(const f16x4*)((const f16*)hadK + hr * K + hc);
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) hf[t][ks][hh * 4 + e] = v[e];
            }
    }
    // Sylvester fragments: H_m[r][r'] = (-1)^popcount(r & r').  With `ident` the inner factor is the
    // identity instead, y = x . (hadK (x) I_m)^T * scale: the transform ACROSS m-wide groups, which is what
    // OnlineHadamard(num_heads) on the transposed attention output computes (e2e/quantized_llama/
    // modeling_llama.py:108-110), with the same staging as the reference (x * scale rounded to fp16, then
    // hadK @ .: quarot/functional/hadamard.py:94-101 with n / K = 1).
    f16x8 b1[NCT][KS1];
#pragma unroll
    for (int c = 0; c < NCT; ++c)
#pragma unroll
        for (int ks = 0; ks < KS1; ++ks)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int rp = (wave + 4 * c) * 16 + l16;
                const int r = ks * 32 + g * 8 + j;
                const f16 sylv = (__builtin_popcount(r & rp) & 1) ? (f16)-1.0f : (f16)1.0f;
                b1[c][ks][j] = ident ? (r == rp ? (f16)1.0f : (f16)0.0f) : sylv;
            }

    // stage-1 A-fragments for the tile pair s2 of a row: [2 tiles][KS1] 16-byte loads
    auto load_pair = [&](const f16* xr, int s2, u32x4(&dst)[2][KS1]) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k = (2 * s2 + h) * 16 + l16;
#pragma unroll
            for (int ks = 0; ks < KS1; ++ks)
                dst[h][ks] = k < K ? *((const u32x4*)(xr + k * M_ + ks * 32 + g * 8)) : u32x4{0, 0, 0, 0};
        }
    };
    // one tile pair through stage 1: T fragments for this wave's column tile(s) -> LDS
    auto stage1 = [&](int s2, const u32x4(&cur)[2][KS1]) {
#pragma unroll
        for (int c = 0; c < NCT; ++c) {
            f32x4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS1; ++ks) {
                a0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, cur[0][ks]), b1[c][ks], a0, 0, 0, 0);
                a1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, cur[1][ks]), b1[c][ks], a1, 0, 0, 0);
            }
            float t[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                t[e] = a0[e] * scale;
                t[e + 4] = a1[e] * scale;
            }
            u32x4 hi, lo;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const u32 hw = narrow_f16x2(t[2 * e], t[2 * e + 1]);
                hi[e] = hw;
                if (MODE32) {
                    const f16x2 h = as_f16x2(hw);
                    lo[e] = narrow_f16x2(t[2 * e] - (float)h[0], t[2 * e + 1] - (float)h[1]);
                }
            }
            const int slot = ((wave + 4 * c) * KS2 + s2) * 64 + lane;
            Tl[slot] = hi;
            if (MODE32) Tlo[slot] = lo;
        }
    };

    auto lds_pair = [&](int s2, u32x4(&dst)[2][KS1]) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int ks = 0; ks < KS1; ++ks) dst[h][ks] = Xl[xslot((2 * s2 + h) * 16 + l16, ks * 4 + g)];
    };

    u32x4 fr[XLDS ? 1 : SLOTS][2][KS1];
    int row_parity = 0;
    int64_t row = blockIdx.x;
    if (row < rows) {
        if (XLDS) {
            load_row(x + row * (int64_t)n);
        } else if (FULL_ROW) {
#pragma unroll
            for (int s2 = 0; s2 < KS2; ++s2) load_pair(x + row * (int64_t)n, s2, fr[s2 % SLOTS]);
        } else {
            load_pair(x + row * (int64_t)n, 0, fr[0]);
        }
    }
    for (; row < rows; row += gridDim.x) {
        const f16* xr = x + row * (int64_t)n;
        const int64_t nrow = row + gridDim.x;
        // ---- stage 1
        if (XLDS) {
            deposit_row();
            if (nrow < rows) load_row(x + nrow * (int64_t)n);
            __syncthreads();
        }
#pragma unroll
        for (int s2 = 0; s2 < KS2; ++s2) {
            if (XLDS) {
                lds_pair(s2, fr[0]);
                stage1(s2, fr[0]);
            } else if (FULL_ROW) {
                stage1(s2, fr[s2 % SLOTS]);
                if (nrow < rows) load_pair(x + nrow * (int64_t)n, s2, fr[s2 % SLOTS]);
            } else {
                // slot parity alternates per pair; with an odd KS2 the next row starts on the other slot,
                // so the last pair's successor (next row, pair 0) is copied into slot 0 below
                if (s2 + 1 < KS2) load_pair(xr, s2 + 1, fr[(s2 + 1) % SLOTS]);
                else if (nrow < rows) load_pair(x + nrow * (int64_t)n, 0, fr[(s2 + 1) % SLOTS]);
                stage1(s2, fr[s2 % SLOTS]);
            }
        }
        if (!XLDS && !FULL_ROW && (KS2 % 2) == 1) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int ks = 0; ks < KS1; ++ks) fr[0][h][ks] = fr[1][h][ks];
        }
        __syncthreads();
        // ---- stage 2 (when fused, the row's abs-max is taken from the rounded results on the way)
        u16x2 mx2 = {0, 0};
        for (int ct = 0; ct < CT; ++ct) {
            f16x8 th[KS2], tl[KS2];
#pragma unroll
            for (int ks = 0; ks < KS2; ++ks) {
                th[ks] = __builtin_bit_cast(f16x8, Tl[(ct * KS2 + ks) * 64 + lane]);
                if (MODE32) tl[ks] = __builtin_bit_cast(f16x8, Tlo[(ct * KS2 + ks) * 64 + lane]);
            }
#pragma unroll
            for (int t = 0; t < RT_W; ++t) {
                const int rt = wave + 4 * t;
                if (rt < row_tiles) {
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < KS2; ++ks) {
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(th[ks], hf[t][ks], acc, 0, 0, 0);
                        if (MODE32) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(tl[ks], hf[t][ks], acc, 0, 0, 0);
                    }
                    const int kp = rt * 16 + l16;
                    if (kp < K) {
                        u32x2 o;
                        o[0] = narrow_f16x2(acc[0], acc[1]);
                        o[1] = narrow_f16x2(acc[2], acc[3]);
                        *(u32x2*)(Yl + kp * YS + ct * 16 + g * 4) = o;
                        if (QUANT) {
                            mx2 = __builtin_elementwise_max(mx2, __builtin_bit_cast(u16x2, o[0] & 0x7fff7fffu));
                            mx2 = __builtin_elementwise_max(mx2, __builtin_bit_cast(u16x2, o[1] & 0x7fff7fffu));
                        }
                    }
                }
            }
        }
        u32 mx = 0;
        if (QUANT) {
            mx = mx2[0] > mx2[1] ? mx2[0] : mx2[1];
            mx = wave_max_u32(mx);
            if (lane == 0) red[(row_parity << 2) + wave] = mx;
        }
        __syncthreads();
        // ---- stage 3
        if (QUANT) {
#pragma unroll
            for (int w = 0; w < HT / QR_WAVE; ++w) mx = mx > red[(row_parity << 2) + w] ? mx : red[(row_parity << 2) + w];
            row_parity ^= 1;
            const f16 sh = quantizer_scale(f16_from_bits((unsigned short)mx), clip);
            if (tid == 0) scales[row] = sh;
            const float s = (float)sh;
            // two chunks (16 elements) per thread and step: 8-byte stores of codes
            const int nunits = nchunks >> 1;
            u32x2* qrow = (u32x2*)(q + row * (int64_t)nchunks);
            if (fast_quant_ok(mx, s)) {
                const FastRecip fq = make_fast_recip(s);
                for (int u = tid; u < nunits; u += HT) {
                    const f16* src = Yl + ((u * 16) >> LOG2M) * YS + ((u * 16) & (M_ - 1));
                    const u32x4 h0 = *(const u32x4*)src, h1 = *(const u32x4*)(src + 8);
                    qrow[u] = u32x2{sym_codes8_fast(h0, fq), sym_codes8_fast(h1, fq)};
                    if (y) {
                        __builtin_nontemporal_store(h0, (u32x4*)(y + row * (int64_t)n) + 2 * u);
                        __builtin_nontemporal_store(h1, (u32x4*)(y + row * (int64_t)n) + 2 * u + 1);
                    }
                }
            } else {
                const bool fast = scale_fast_ok(s);
                const float rs = fast ? 1.0f / s : 0.0f;
                for (int u = tid; u < nunits; u += HT) {
                    const f16* src = Yl + ((u * 16) >> LOG2M) * YS + ((u * 16) & (M_ - 1));
                    const u32x4 h0 = *(const u32x4*)src, h1 = *(const u32x4*)(src + 8);
                    qrow[u] = u32x2{sym_codes8(h0, s, rs, fast), sym_codes8(h1, s, rs, fast)};
                    if (y) {
                        __builtin_nontemporal_store(h0, (u32x4*)(y + row * (int64_t)n) + 2 * u);
                        __builtin_nontemporal_store(h1, (u32x4*)(y + row * (int64_t)n) + 2 * u + 1);
                    }
                }
            }
        } else {
            for (int c = tid; c < nchunks; c += HT) {
                const u32x4 h = *(const u32x4*)(Yl + ((c * 8) >> LOG2M) * YS + ((c * 8) & (M_ - 1)));
                __builtin_nontemporal_store(h, (u32x4*)(y + row * (int64_t)n) + c);
            }
        }
    }
}

// ---- K > 1, m = 64, fp16 I/O: the same two matrix-core stages, organised for latency ------------
// hadamard_mm_kernel above is bound by exposed latencies (every LDS read, dependent MFMA chain and
// conversion waits for the one before it) and reads the staged input four times.  Here
//   * a wave owns whole 16-row tiles of X (tile t = wave + 4 i): it fetches them with coalesced
//     16-byte loads one row ahead, stages them in a wave-private LDS region (no workgroup barrier:
//     LDS operations of one wave execute in order) and reads its stage-1 fragments from there, so X
//     is read from LDS once; all column tiles of T for these rows come from eight Sylvester
//     fragments held in registers;
//   * T is kept as [column tile][16-row tile][lane] 8-byte halves: stage 1 writes 8 contiguous bytes
//     per lane, stage 2 assembles a 32-deep fragment from two of them;
//   * stage 2 fetches the fragments of the next column tile while the MFMAs of the current one run,
//     all hadK tiles of a wave are independent accumulator chains in one basic block (rows of hadK
//     beyond K are zero fragments and produce zero rows of Y: no branches), stage 3 issues all its
//     LDS reads before the first conversion.
// Two workgroup barriers per row.
template <bool MODE32, bool QUANT, int KS2>
__global__ __launch_bounds__(HT, (KS2 <= 2 ? 4 : 2)) void hadamard_m64_kernel(
    const f16* __restrict__ x, f16* __restrict__ y, int64_t rows, int n, int K, const void* __restrict__ hadK,
    float scale, float clip, u32* __restrict__ q, f16* __restrict__ scales) {
    constexpr int CT = 4;                        // 16-column tiles of T / Y
    constexpr int YS = 64 + 8;                   // halves per row of Yl
    constexpr int NT = 2 * KS2;                  // 16-row tiles of X / T / hadK (order padded to 32 KS2)
    constexpr int TPW = (NT + 3) / 4;            // tiles per wave
    constexpr int YROWS = TPW * 64;              // every wave writes TPW full tiles of Y
    extern __shared__ f32x4 smem_raw[];
    __shared__ u32 red[HT / QR_WAVE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int nchunks = n >> 3;
    u32x2* Tl = (u32x2*)smem_raw;                                      // [CT][NT][64 lanes], hi plane
    u32x2* Tlo = Tl + CT * NT * 64;                                    // lo plane (fp32 mode)
    f16* Yl = (f16*)(Tl + (MODE32 ? 2 : 1) * CT * NT * 64);            // [YROWS][YS]
    u32x4* Xs = (u32x4*)(Yl + YROWS * YS) + wave * (TPW * 128);        // wave-private [TPW][16 rows][8 pieces]

    // T slots of tiles beyond K and staged rows beyond K are never written afterwards: clear once
    for (int i = tid; i < (MODE32 ? 2 : 1) * CT * NT * 32; i += HT) ((u32x4*)Tl)[i] = u32x4{0, 0, 0, 0};
    for (int i = lane; i < TPW * 128; i += QR_WAVE) Xs[i] = u32x4{0, 0, 0, 0};

    // hadK fragments of this wave's tiles (second MFMA operand of stage 2), contraction index in
    // the order k = 32 s + 16 (j / 4) + 4 (lane / 16) + j % 4
    f16x8 hf[TPW][KS2];
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
        const int hr = (wave + 4 * t) * 16 + l16;
#pragma unroll
        for (int ks = 0; ks < KS2; ++ks)
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                const int hc = ks * 32 + hh * 16 + g * 4;
                f16x4 v = {(f16)0, (f16)0, (f16)0, (f16)0};
                if (hr < K && hc < K) {
                    if (hadK == nullptr) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = (__builtin_popcount(hr & (hc + e)) & 1) ? (f16)-1.0f : (f16)1.0f;
                    } else if (MODE32) {
                        const f32x4 w = *(const f32x4*)((const float*)hadK + hr * K + hc);
                        v = f16x4{(f16)w[0], (f16)w[1], (f16)w[2], (f16)w[3]};
                    } else {
                        v = *(const f16x4*)((const f16*)hadK + hr * K + hc);
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) hf[t][ks][hh * 4 + e] = v[e];
            }
    }
    // Sylvester fragments of all four column tiles: H_64[r][r'] = (-1)^popcount(r & r') with
    // r = 32 ks + 8 g + j, r' = 16 ct + l16.  The sign factors by index bits: bits 0..3 give a base
    // fragment, bit 4 contributes (g >> 1) & (ct & 1) (lane-dependent: a second base for odd ct) and
    // bit 5 contributes ks & (ct >> 1), the same for every lane.  Two bases and their negations
    // (16 registers) stand for all eight fragments; which one an MFMA takes is known at compile time.
    f16x8 sb[2][2];                                          // [ct & 1][negated]
#pragma unroll
    for (int o = 0; o < 2; ++o)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const bool neg = ((__builtin_popcount(((g & 1) * 8 + j) & l16) + ((g >> 1) & o)) & 1) != 0;
            sb[o][0][j] = neg ? (f16)-1.0f : (f16)1.0f;
            sb[o][1][j] = neg ? (f16)1.0f : (f16)-1.0f;
        }

    // staging: load c of a tile covers its rows 8 c .. 8 c + 7, lane -> (row 8 c + lane / 8, piece
    // lane % 8): 1 KB of consecutive addresses per instruction.  Pieces are XOR-keyed by the row so
    // that the sixteen rows of a fragment read fall into sixteen different bank groups.
    int dslot[2], rslot[2], goff[TPW][2];
    bool dval[TPW][2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const int rc = c * 8 + (lane >> 3);
        dslot[c] = rc * 8 + ((lane & 7) ^ ((rc >> 1) & 7));
        rslot[c] = l16 * 8 + ((c * 4 + g) ^ ((l16 >> 1) & 7));
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            dval[i][c] = (wave + 4 * i) * 16 + rc < K;
            goff[i][c] = dval[i][c] ? (wave + 4 * i) * 128 + c * 64 + lane : 0;
        }
    }
    u32x4 xr[TPW][2];
    auto load_row = [&](const f16* src) {
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int c = 0; c < 2; ++c) xr[i][c] = *((const u32x4*)src + goff[i][c]);
    };
    u32 amask[TPW];                                          // magnitude bits of this lane's output row in tile i, 0 beyond K
#pragma unroll
    for (int i = 0; i < TPW; ++i) amask[i] = (wave + 4 * i) * 16 + l16 < K ? 0x7fff7fffu : 0u;

    int64_t row = blockIdx.x;
    if (row < rows) load_row(x + row * (int64_t)n);
    // the hadK fragments must have arrived before the loop: otherwise their first use in every
    // iteration would also wait for the row just requested
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int ks = 0; ks < KS2; ++ks) asm volatile("" : "+v"(hf[t][ks]));
    __syncthreads();
    for (; row < rows; row += gridDim.x) {
        const int64_t nrow = row + gridDim.x;
        // ---- stage 1: T = X . H_64 for this wave's tiles
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int c = 0; c < 2; ++c)
                if (dval[i][c]) Xs[i * 128 + dslot[c]] = xr[i][c];
        if (nrow < rows) load_row(x + nrow * (int64_t)n);
        u32x4 af[TPW][2];
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) af[i][ks] = Xs[i * 128 + rslot[ks]];
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            const int t = wave + 4 * i;
            if (4 * i + 3 < NT || t < NT) {
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, af[i][0]), sb[ct & 1][0], acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, af[i][1]), sb[ct & 1][ct >> 1], acc, 0, 0, 0);
                    float tv[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) tv[e] = acc[e] * scale;
                    u32x2 hi, lo;
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        const u32 hw = narrow_f16x2(tv[2 * e], tv[2 * e + 1]);
                        hi[e] = hw;
                        if (MODE32) {
                            const f16x2 h = as_f16x2(hw);
                            lo[e] = narrow_f16x2(tv[2 * e] - (float)h[0], tv[2 * e + 1] - (float)h[1]);
                        }
                    }
                    Tl[(ct * NT + t) * 64 + lane] = hi;
                    if (MODE32) Tlo[(ct * NT + t) * 64 + lane] = lo;
                }
            }
        }
        __syncthreads();
        // ---- stage 2: Y^T = T^T . hadK^T (the row's abs-max is taken from the rounded results)
        u16x2 mx2 = {0, 0};
        u32x4 th[2][KS2], tlo[2][KS2];
        auto fetch = [&](int ct, int b) {
#pragma unroll
            for (int ks = 0; ks < KS2; ++ks) {
                const u32x2 p0 = Tl[(ct * NT + 2 * ks) * 64 + lane], p1 = Tl[(ct * NT + 2 * ks + 1) * 64 + lane];
                th[b][ks] = u32x4{p0[0], p0[1], p1[0], p1[1]};
                if (MODE32) {
                    const u32x2 r0 = Tlo[(ct * NT + 2 * ks) * 64 + lane], r1 = Tlo[(ct * NT + 2 * ks + 1) * 64 + lane];
                    tlo[b][ks] = u32x4{r0[0], r0[1], r1[0], r1[1]};
                }
            }
        };
        fetch(0, 0);
        f16* ybase = Yl + (wave * 16 + l16) * YS + g * 4;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            if (ct + 1 < CT) fetch(ct + 1, (ct + 1) & 1);
            __builtin_amdgcn_sched_barrier(0);               // the next tile's reads are issued before this tile's MFMAs
            f32x4 acc[TPW];
#pragma unroll
            for (int i = 0; i < TPW; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS2; ++ks)
#pragma unroll
                for (int i = 0; i < TPW; ++i) {
                    acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, th[ct & 1][ks]), hf[i][ks], acc[i], 0, 0, 0);
                    if (MODE32)
                        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, tlo[ct & 1][ks]), hf[i][ks], acc[i], 0, 0, 0);
                }
#pragma unroll
            for (int i = 0; i < TPW; ++i) {
                u32x2 o;
                o[0] = narrow_f16x2(acc[i][0], acc[i][1]);
                o[1] = narrow_f16x2(acc[i][2], acc[i][3]);
                *(u32x2*)(ybase + i * 64 * YS + ct * 16) = o;
                if (QUANT) {
                    // rows beyond K do not exist: they are zero except when the row holds an infinity (0 . inf)
                    mx2 = __builtin_elementwise_max(mx2, __builtin_bit_cast(u16x2, o[0] & amask[i]));
                    mx2 = __builtin_elementwise_max(mx2, __builtin_bit_cast(u16x2, o[1] & amask[i]));
                }
            }
        }
        // ---- stage 3
        if (QUANT) {
            u32 mx = mx2[0] > mx2[1] ? mx2[0] : mx2[1];
            mx = wave_max_u32_dpp(mx);
            if (lane == 0) red[wave] = mx;
            // Units of 16 elements (two chunks, 8-byte stores of codes).  Unit (i, lane) is row
            // kp = 16 (wave + 4 i) + lane / 4, columns 16 (lane % 4)..: rows of this wave's own tiles,
            // which it wrote itself, so the reads are issued before the barrier that publishes the row
            // maximum.  Lanes on rows beyond K repeat the unit of their first tile (K >= 64: always
            // inside) and store it again, the same value from the same lane: all stores are
            // unconditional, so their number is known when the next row's loads are awaited and that
            // wait need not include them.
            int un[TPW];
            u32x4 h[TPW][2];
#pragma unroll
            for (int i = 0; i < TPW; ++i) {
                int kp = (wave + 4 * i) * 16 + (lane >> 2);
                kp = kp < K ? kp : wave * 16 + (lane >> 2);
                const f16* src = Yl + kp * YS + (lane & 3) * 16;
                h[i][0] = *(const u32x4*)src;
                h[i][1] = *(const u32x4*)(src + 8);
                un[i] = kp * 4 + (lane & 3);
            }
            __syncthreads();
#pragma unroll
            for (int w = 0; w < HT / QR_WAVE; ++w) mx = mx > red[w] ? mx : red[w];
            const f16 sh = quantizer_scale(f16_from_bits((unsigned short)mx), clip);
            const float s = (float)sh;
            u32x2* qrow = (u32x2*)(q + row * (int64_t)nchunks);
            u32x2 codes[TPW];
            if (fast_quant_ok(mx, s)) {
                const FastRecip fq = make_fast_recip(s);
#pragma unroll
                for (int i = 0; i < TPW; ++i) codes[i] = u32x2{sym_codes8_fast(h[i][0], fq), sym_codes8_fast(h[i][1], fq)};
            } else {
                const bool fast = scale_fast_ok(s);
                const float rs = fast ? 1.0f / s : 0.0f;
#pragma unroll
                for (int i = 0; i < TPW; ++i) codes[i] = u32x2{sym_codes8(h[i][0], s, rs, fast), sym_codes8(h[i][1], s, rs, fast)};
            }
#pragma unroll
            for (int i = 0; i < TPW; ++i) qrow[un[i]] = codes[i];
            scales[row] = sh;
            if (y) {
#pragma unroll
                for (int i = 0; i < TPW; ++i) {
                    __builtin_nontemporal_store(h[i][0], (u32x4*)(y + row * (int64_t)n) + 2 * un[i]);
                    __builtin_nontemporal_store(h[i][1], (u32x4*)(y + row * (int64_t)n) + 2 * un[i] + 1);
                }
            }
        } else {
            __syncthreads();
            u32x4 h[KS2];
            int cn[KS2];
#pragma unroll
            for (int j = 0; j < KS2; ++j) {
                const int c = tid + j * HT;
                cn[j] = c < nchunks ? c : nchunks - 1;
                h[j] = *(const u32x4*)(Yl + (cn[j] >> 3) * YS + (cn[j] & 7) * 8);
            }
#pragma unroll
            for (int j = 0; j < KS2; ++j) __builtin_nontemporal_store(h[j], (u32x4*)(y + row * (int64_t)n) + cn[j]);
        }
        // Tl is next written after the barrier above (all of this row's stage-2 reads precede it);
        // red[] is next written after the next row's first barrier; Yl rows and the staging region
        // are private to a wave
    }
}

// ---- K > 1, m = 64, fp16 staging, quantiser fused, no copy of the transformed row: the lean form ---
// The same two matrix-core stages and the same arithmetic as hadamard_m64_kernel (identical fragments
// and accumulation order, so codes and scales are identical bit for bit), with two of its three trips
// through LDS removed:
//   * stage 1 takes its A fragments straight from global memory: lane (row l16 of a 16-row tile, g) loads
//     the 16 bytes k = 8 g .. 8 g + 7 of its row for each of the two k steps: 64 consecutive bytes per
//     row and instruction, both halves of every 128-byte row within one pair of loads;
//   * the fp16 results of stage 2 stay in registers (a lane holds, for ONE output row k', the four
//     columns 16 ct + 4 g .. + 3 of every column tile ct) until the row maximum is known; the codes are
//     then formed in registers and four-lane groups exchange their 16-bit pieces (v_permlane32_swap,
//     v_permlane16_swap, byte permutes: a 4 x 4 transpose of pieces across the lanes l16 + 16 g) so
//     that every lane stores 8 contiguous bytes and a wave 32 contiguous bytes per output row.
// Only T (stage 1's output, read by every wave in stage 2) lives in LDS: 4 KB per 32 hadK columns.
template <int KS2, int LOG2M = 6, bool SMALLK = false>
__global__ __launch_bounds__(HT, (LOG2M == 7 && KS2 >= 5 ? 1 : 2)) void hadamard_m64q_kernel(const f16* __restrict__ x, int64_t rows, int n, int K,
                                                             const f16* __restrict__ hadK, float scale, float clip,
                                                             u32* __restrict__ q, f16* __restrict__ scales) {
    constexpr int M_ = 1 << LOG2M;                           // the power-of-two factor: 64, or 128 (hadK of 64 .. 128)
    constexpr int CT = M_ / 16;                              // column tiles
    constexpr int S1K = M_ / 32;                             // k steps of stage 1
    constexpr int NT = 2 * KS2;
    constexpr int TPW = (NT + 3) / 4;
    extern __shared__ f32x4 smem_raw[];
    __shared__ u32 red[HT / QR_WAVE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int nchunks = n >> 3;
    u32x2* Tl = (u32x2*)smem_raw;                                      // [CT][NT][64 lanes]
    for (int i = tid; i < CT * NT * 32; i += HT) ((u32x4*)Tl)[i] = u32x4{0, 0, 0, 0};

    f16x8 hf[TPW][KS2];
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
        const int hr = (wave + 4 * t) * 16 + l16;
#pragma unroll
        for (int ks = 0; ks < KS2; ++ks)
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                const int hc = ks * 32 + hh * 16 + g * 4;
                // unconditional loads (a clamped address, then a select): all of them are in flight
                // together; a branch around each would serialise 12 KS2 round trips through the cache
                const bool ok = hr < K && hc < K;
                f16x4 v = *(const f16x4*)(hadK + (ok ? hr * K + hc : 0));
                if (!ok) v = f16x4{(f16)0, (f16)0, (f16)0, (f16)0};
#pragma unroll
                for (int e = 0; e < 4; ++e) hf[t][ks][hh * 4 + e] = v[e];
            }
    }
    f16x8 sb[2][2];                                          // Sylvester fragments, as in hadamard_m64_kernel
#pragma unroll
    for (int o = 0; o < 2; ++o)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const bool neg = ((__builtin_popcount(((g & 1) * 8 + j) & l16) + ((g >> 1) & o)) & 1) != 0;
            sb[o][0][j] = neg ? (f16)-1.0f : (f16)1.0f;
            sb[o][1][j] = neg ? (f16)1.0f : (f16)-1.0f;
        }
    // fragment (tile i, k step c) of a row: 16-byte piece 4 c + g of row (wave + 4 i) 16 + l16 of X[K][M_]
    int goff[TPW][S1K];
    bool dval[TPW];
#pragma unroll
    for (int i = 0; i < TPW; ++i) {
        const int r = (wave + 4 * i) * 16 + l16;
        dval[i] = r < K;
#pragma unroll
        for (int c = 0; c < S1K; ++c) goff[i][c] = dval[i] ? r * (M_ / 8) + 4 * c + g : 0;
    }
    u32x4 xr[TPW][S1K];
    auto load_row = [&](const f16* src) {
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int c = 0; c < S1K; ++c) xr[i][c] = *((const u32x4*)src + goff[i][c]);
    };
    u32 amask[TPW];                                          // magnitude bits of this lane's output row in tile i, 0 beyond K:
#pragma unroll                                               // those rows are zero except when the row holds an infinity (0 . inf)
    for (int i = 0; i < TPW; ++i) amask[i] = dval[i] ? 0x7fff7fffu : 0u;
    int64_t row = blockIdx.x;
    if (row < rows) load_row(x + row * (int64_t)n);
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int ks = 0; ks < KS2; ++ks) asm volatile("" : "+v"(hf[t][ks]));
    __syncthreads();
    // The quantiser of row r (~350 vector instructions per lane) is written between the matrix
    // instructions of row r + 1's hadK stage.  What the compiler makes of it: the codes are only used on the
    // lean path of finish_prev, so the optimiser sinks the arithmetic into that branch, behind the stage,
    // and schedules it there as one block.  That is the fastest of the three forms measured at 11008
    // columns (32768 rows): this one 270-283 us; the same arithmetic written after the stage 305-310 us;
    // the interleaving forced (each part pinned with an empty asm statement, 2-5 vector instructions
    // after every matrix instruction in the generated code) 340-350 us -- two workgroups share a SIMD, and
    // a pure matrix phase of one overlaps a pure vector phase of the other better than two mixed streams.
    u32x2 yp[TPW][CT];                                       // previous row's fp16 results (the same lane layout)
    u32 pb[TPW][CT][2];                                      // ... its codes as fp16 1536 + code pairs
    // Before the first row there is no previous one: the turn then "finishes" zeros with scale 1 into the
    // first row's own place, which the real codes overwrite a turn later (same lanes, same addresses, in
    // order).  Every turn thus issues the same memory operations, branch-free.
    FastRecip fqp = make_fast_recip(1.0f);
    float sp = 1.0f;
    u32 mxp = 0x3c00u;
    int64_t prow = blockIdx.x;
#pragma unroll
    for (int i = 0; i < TPW; ++i)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) yp[i][ct] = u32x2{0, 0};
    // One register pair of the previous row in three parts of two vector instructions (the arithmetic
    // of sym_codes8_fast): each part goes behind one matrix instruction, whose 16 cycles leave room for
    // about three vector instructions of the same wave.
    float qa0 = 0.f, qa1 = 0.f;
    auto quant_part = [&](int p, int part) {
        const int i = p / (2 * CT), ct = (p / 2) % CT, w = p & 1;
        if (part == 0) {
            const f16x2 h2 = as_f16x2(yp[i][ct][w]);
            qa0 = __builtin_fmaf((float)h2[0], fqp.r, 0.0f);
            qa1 = __builtin_fmaf((float)h2[1], fqp.r, 0.0f);
        } else if (part == 1) {
            qa0 = __builtin_amdgcn_fmed3f(qa0, -8.0f, 7.0f);
            qa1 = __builtin_amdgcn_fmed3f(qa1, -8.0f, 7.0f);
        } else {
            f16x2 h = {(f16)qa0, (f16)qa1};
            h = h + f16x2{(f16)1536.0f, (f16)1536.0f};
            pb[i][ct][w] = __builtin_bit_cast(u32, h);
        }
    };
    auto quant_pair = [&](int p) {
        quant_part(p, 0);
        quant_part(p, 1);
        quant_part(p, 2);
    };
    auto finish_prev = [&](bool fast) {                      // pack, exchange pieces between lanes, store
        constexpr int HV = CT / 4;                           // groups of four column tiles (64 columns) per row
        u32 c01[TPW][HV], c23[TPW][HV];
        if (fast) {
#pragma unroll
            for (int i = 0; i < TPW; ++i)
#pragma unroll
                for (int hv = 0; hv < HV; ++hv) {
                    const u32 b0[4] = {pb[i][4 * hv][0], pb[i][4 * hv][1], pb[i][4 * hv + 1][0], pb[i][4 * hv + 1][1]};
                    const u32 b1[4] = {pb[i][4 * hv + 2][0], pb[i][4 * hv + 2][1], pb[i][4 * hv + 3][0], pb[i][4 * hv + 3][1]};
                    c01[i][hv] = pack_nibbles8(b0);
                    c23[i][hv] = pack_nibbles8(b1);
                }
        } else {
            const bool fs = scale_fast_ok(sp);
            const float rs = fs ? 1.0f / sp : 0.0f;
#pragma unroll
            for (int i = 0; i < TPW; ++i)
#pragma unroll
                for (int hv = 0; hv < HV; ++hv) {
                    c01[i][hv] = sym_codes8(u32x4{yp[i][4 * hv][0], yp[i][4 * hv][1], yp[i][4 * hv + 1][0], yp[i][4 * hv + 1][1]}, sp, rs, fs);
                    c23[i][hv] = sym_codes8(u32x4{yp[i][4 * hv + 2][0], yp[i][4 * hv + 2][1], yp[i][4 * hv + 3][0], yp[i][4 * hv + 3][1]}, sp, rs, fs);
                }
        }
        u32x2* qrow = (u32x2*)(q + prow * (int64_t)nchunks);
        u32x2 outv[TPW][HV];
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int hv = 0; hv < HV; ++hv) {
                // lanes l16 + 16 g: piece (g, ct) -> lane ct % 4.  First the halves of the wave (g and g ^ 2) ...
                const auto s1 = __builtin_amdgcn_permlane32_swap(c01[i][hv], c23[i][hv], false, false);
                const u32 ev = __builtin_amdgcn_perm(s1[1], s1[0], 0x05040100u);     // the even column tile of this lane's pair
                const u32 od = __builtin_amdgcn_perm(s1[1], s1[0], 0x07060302u);     // the odd one
                // ... then neighbouring rows of 16 lanes (g and g ^ 1)
                const auto s2 = __builtin_amdgcn_permlane16_swap(ev, od, false, false);
                const u32 lo = __builtin_amdgcn_perm(s2[1], s2[0], 0x05040100u);     // pieces of g = 0, 1
                const u32 hi = __builtin_amdgcn_perm(s2[1], s2[0], 0x07060302u);     // pieces of g = 2, 3
                outv[i][hv] = u32x2{lo, hi};
            }
        // lanes on rows beyond K store their first tile's piece once more (K >= 64: that row exists; SMALLK: hadK
        // is smaller than that, a wave's first tile may lie outside it, and the stores are conditional)
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            const int kp = (wave + 4 * i) * 16 + l16;
            const bool ok = kp < K;
#pragma unroll
            for (int hv = 0; hv < HV; ++hv) {
                if (SMALLK) {
                    if (ok) qrow[kp * CT + hv * 4 + g] = outv[i][hv];
                } else {
                    qrow[(ok ? kp : wave * 16 + l16) * CT + hv * 4 + g] = ok ? outv[i][hv] : outv[0][hv];
                }
            }
        }
    };
    for (; row < rows; row += gridDim.x) {
        const int64_t nrow = row + gridDim.x;
        // ---- stage 1: T = X . H_64 for this wave's tiles (rows beyond K are zero fragments)
        u32x4 af[TPW][S1K];
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int c = 0; c < S1K; ++c) af[i][c] = dval[i] ? xr[i][c] : u32x4{0, 0, 0, 0};
        // (unconditional, like every store below: with a fixed number of memory operations per turn the wait
        // for these loads, a turn later, need not include the stores issued after them; the last turn re-reads
        // its own row)
        load_row(x + (nrow < rows ? nrow : row) * (int64_t)n);
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            const int t = wave + 4 * i;
            if (4 * i + 3 < NT || t < NT) {
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
                    // H[k][col] = (-1)^popcount(k & col): the fragment of (k step c, column tile ct) is the base tile of
                    // ct & 1, negated when c and ct / 2 share an odd number of bits
#pragma unroll
                    for (int c = 0; c < S1K; ++c)
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, af[i][c]),
                                                                   sb[ct & 1][__builtin_popcount(c & (ct >> 1)) & 1], acc, 0, 0, 0);
                    u32x2 hi;
                    hi[0] = narrow_f16x2(acc[0] * scale, acc[1] * scale);
                    hi[1] = narrow_f16x2(acc[2] * scale, acc[3] * scale);
                    Tl[(ct * NT + t) * 64 + lane] = hi;
                }
            }
        }
        __syncthreads();
        // ---- stage 2: Y^T = T^T . hadK^T; results stay in registers.  Between the matrix instructions: the
        // previous row's quantiser (when that row takes the lean path; else it is finished afterwards)
        const bool pfast = fast_quant_ok(mxp, sp);
        u16x2 mx2 = {0, 0};
        u32x2 yv[TPW][CT];
        u32x4 th[2][KS2];
        auto fetch = [&](int ct, int b) {
#pragma unroll
            for (int ks = 0; ks < KS2; ++ks) {
                const u32x2 p0 = Tl[(ct * NT + 2 * ks) * 64 + lane], p1 = Tl[(ct * NT + 2 * ks + 1) * 64 + lane];
                th[b][ks] = u32x4{p0[0], p0[1], p1[0], p1[1]};
            }
        };
        fetch(0, 0);
        constexpr int PAIRS = TPW * CT * 2, GROUPS = CT * KS2;      // 24 pairs over 24 groups when KS2 = 6
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            if (ct + 1 < CT) fetch(ct + 1, (ct + 1) & 1);
            __builtin_amdgcn_sched_barrier(0);
            f32x4 acc[TPW];
#pragma unroll
            for (int i = 0; i < TPW; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS2; ++ks) {
                const int grp = ct * KS2 + ks;
                // pairs grp * PAIRS / GROUPS .. (grp + 1) * PAIRS / GROUPS - 1 of the previous row, their parts
                // spread over the group's matrix instructions
                const int p0 = grp * PAIRS / GROUPS, p1 = (grp + 1) * PAIRS / GROUPS, parts = (p1 - p0) * 3;
#pragma unroll
                for (int i = 0; i < TPW; ++i) {
                    acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, th[ct & 1][ks]), hf[i][ks], acc[i], 0, 0, 0);
#pragma unroll
                    for (int e = i * parts / TPW; e < (i + 1) * parts / TPW; ++e) quant_part(p0 + e / 3, e % 3);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int i = 0; i < TPW; ++i) {
                yv[i][ct][0] = narrow_f16x2(acc[i][0], acc[i][1]);
                yv[i][ct][1] = narrow_f16x2(acc[i][2], acc[i][3]);
                mx2 = __builtin_elementwise_max(mx2, __builtin_bit_cast(u16x2, yv[i][ct][0] & amask[i]));
                mx2 = __builtin_elementwise_max(mx2, __builtin_bit_cast(u16x2, yv[i][ct][1] & amask[i]));
            }
        }
        finish_prev(pfast);
        // ---- this row's maximum and scale; its codes are formed during the next row's stage 2
        u32 mx = mx2[0] > mx2[1] ? mx2[0] : mx2[1];
        mx = wave_max_u32_dpp(mx);
        if (lane == 0) red[wave] = mx;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < HT / QR_WAVE; ++w) mx = mx > red[w] ? mx : red[w];
        const f16 sh = quantizer_scale(f16_from_bits((unsigned short)mx), clip);
        scales[row] = sh;                                     // every lane, the same value: no branch around the store
        sp = (float)sh;
        mxp = mx;
        prow = row;
        fqp = fast_quant_ok(mx, sp) ? make_fast_recip(sp) : FastRecip{0.f};
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) yp[i][ct] = yv[i][ct];
        // Tl is next written after this row's second barrier, which every wave reaches only after its
        // stage-2 reads; red[] is next written after the next row's first barrier
    }
    if ((int64_t)blockIdx.x < rows) {                        // the last row's codes
        const bool pfast = fast_quant_ok(mxp, sp);
        if (pfast) {
#pragma unroll
            for (int pq = 0; pq < TPW * CT * 2; ++pq) quant_pair(pq);
        }
        finish_prev(pfast);
    }
}

// ---- K >= 64, m = 64, fp16 staging, quantiser fused: the lean form with the fewest vector instructions ----
// Same decomposition and the same arithmetic as hadamard_m64q_kernel (four waves per row, hadK fragments in
// registers, only T through LDS; identical fragments and accumulation order, so codes and scales are those of
// hadamard_m64_kernel followed by the quantiser, bit for bit).  What the counters and a set of timing-only
// ablations showed about that kernel: its time is the SUM of its vector and matrix instructions' issue cycles on a
// SIMD -- removing the loads, the LDS reads or doubling the waves per SIMD changed little or nothing, removing
// instructions did.  So this form issues fewer of them per row:
//   * the row maximum is taken on the fp32 accumulators (v_max3_f32 with |.| modifiers: one instruction per two
//     values, where the packed 16-bit form took an AND and a maximum per two) and rounded to fp16 once -- rounding is
//     monotone, so that is the maximum of the rounded values.  v_max3 drops NaNs; a NaN or infinity anywhere in a
//     row reaches every output, so one output per lane is tested, and a wave that sees anything non-finite takes
//     the exact bit-pattern maximum of the lean kernel above instead (NaN wins, as in torch.max);
//   * the codes are formed right after the row maximum is known, from the registers the matrix stage left them
//     in: no copies to a "previous row" set, no second set of code registers;
//   * the quotient goes from the packed fp16 pair to the packed fp16 quotient in one mixed-precision instruction
//     per value (sym_pair_fast) and, where the clamp cannot act (clip >= 1, normal scale), without a clamp: three
//     instructions per pair of values where there were six;
//   * zero fragments for rows beyond hadK's order are formed only in the one tile that is partial, and a tile that
//     lies entirely beyond it is skipped.
// TPW: how many of this wave's tiles (rows (wave + 4 i) 16 .. + 15 of hadK) lie inside hadK, at least in part;
// only the last of them can be partial.  (A function of the wave so that every loop below is free of branches.)
// MODE32: the fp32-precision staging of hadamard_m64_kernel<true, ..> -- T = X . H_64 * scale is kept as an fp16 hi and an
// fp16 lo plane (hi = fp16(T), lo = fp16(T - hi)), every product of the hadK stage is a hi and a lo matrix instruction
// in that order, and the result is rounded to fp16 once; hadK is then an fp32 table, or null for a power-of-two row,
// whose outer factor is the Sylvester matrix of order K (generated).
template <bool MODE32, int KS2, int TPW, int CHUNKS>
__device__ __forceinline__ void hadamard_m64r_rows(const f16* __restrict__ x, int64_t rows, int n, int K,
                                                   const void* __restrict__ hadK, float scale, float clip,
                                                   u32* __restrict__ q, f16* __restrict__ scales, f32x4* smem_raw, u32* red,
                                                   int signs) {
    constexpr int CT = 4, NT = 2 * KS2;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, g = lane >> 4;
    const int nchunks = n >> 3;
    u32x2* Tl = (u32x2*)smem_raw;                                      // [CT][NT][64 lanes]
    u32x2* Tlo = Tl + CT * NT * 64;                                    // lo plane (fp32-precision mode)

    // Sylvester fragments of hadamard_m64_kernel: one base per parity of the column tile; where that kernel takes a
    // negated fragment (second contraction step, column tiles 2 and 3) the OTHER operand is negated here instead
    // (sign bits of its fp16 pairs flipped: the products are the same numbers), which saves eight registers
    f16x8 sb[2];
#pragma unroll
    for (int o = 0; o < 2; ++o)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const bool neg = ((__builtin_popcount(((g & 1) * 8 + j) & l16) + ((g >> 1) & o)) & 1) != 0;
            sb[o][j] = neg ? (f16)-1.0f : (f16)1.0f;
        }
    // dval: this lane's row of tile i exists
    bool dval[TPW];
    int goff[TPW];
#pragma unroll
    for (int i = 0; i < TPW; ++i) {
        const int t16 = (wave + 4 * i) * 16;
        dval[i] = t16 + l16 < K;
        goff[i] = (dval[i] ? t16 + l16 : 0) * 8 + g;         // 16-byte pieces g and 4 + g of that row of X[K][64]
    }
    u32x4 xr[TPW][2];
    auto load_row = [&](const f16* src) {
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int c = 0; c < 2; ++c) xr[i][c] = *((const u32x4*)src + goff[i] + 4 * c);
    };
    int64_t row = blockIdx.x;
    if (row < rows) load_row(x + row * (int64_t)n);
    // hadK's fragments (contraction index in the order k = 32 ks + 16 hh + 4 g + e, as in the kernels above), fetched
    // through LDS: the tiles with the same i of the four waves are 64 consecutive rows of hadK, which the workgroup
    // copies as one run of 16-byte pieces (coalesced, every line requested once) into the region that will hold T;
    // each lane then picks its 8-byte pieces from there.  Loading them straight from memory -- a lane's pieces lie 32
    // bytes apart, every workgroup of the grid asks at the same moment -- cost 3 of the 23 us of a 2048-row launch.
    f16x8 hf[TPW][KS2];
    if (signs) {
        // hadK as sign words (uint32 [K][ceil(K / 32)], bit j of word w of row r set where hadK[r][32 w + j] = -1; the
        // table is +-1 by construction): a lane reads the KS2 words of each of its rows -- 4 KB in all where the fp16
        // table is 59 KB per workgroup, two workgroups per CU, through a memory path of 35-60 GB/s per CU: 3 us of a
        // 2048-row launch -- and expands the four bits of every fragment half into four halves of +-1
        const u32* sw = (const u32*)hadK;
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            const int hr = (wave + 4 * i) * 16 + l16;
            const bool rok = hr < K;
#pragma unroll
            for (int ks = 0; ks < KS2; ++ks) {
                const u32 w = sw[rok ? hr * KS2 + ks : 0];
                u32x4 fr;
#pragma unroll
                for (int hh = 0; hh < 2; ++hh) {
                    const u32 nib = (w >> (hh * 16 + g * 4)) & 15u;
                    const bool ok = rok && ks * 32 + hh * 16 + g * 4 < K;
                    const u32 p0 = 0x3C003C00u | ((nib & 1u) << 15) | ((nib & 2u) << 30);
                    const u32 p1 = 0x3C003C00u | ((nib & 4u) << 13) | ((nib & 8u) << 28);
                    fr[hh * 2] = ok ? p0 : 0u;
                    fr[hh * 2 + 1] = ok ? p1 : 0u;
                }
                hf[i][ks] = __builtin_bit_cast(f16x8, fr);
            }
        }
        u32x4* stage = (u32x4*)smem_raw;
        for (int i = tid; i < (MODE32 ? 2 : 1) * CT * NT * 32; i += HT) stage[i] = u32x4{0, 0, 0, 0};
    } else if (MODE32 && hadK == nullptr) {
        // power-of-two row: the outer factor is the Sylvester matrix of order K, generated in place
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            const int hr = (wave + 4 * i) * 16 + l16;
#pragma unroll
            for (int ks = 0; ks < KS2; ++ks)
#pragma unroll
                for (int hh = 0; hh < 2; ++hh) {
                    const int hc = ks * 32 + hh * 16 + g * 4;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        hf[i][ks][hh * 4 + e] = (hr < K && hc < K) ? ((__builtin_popcount(hr & (hc + e)) & 1) ? (f16)-1.0f : (f16)1.0f) : (f16)0.0f;
                }
        }
        u32x4* stage = (u32x4*)smem_raw;
        for (int i = tid; i < 2 * CT * NT * 32; i += HT) stage[i] = u32x4{0, 0, 0, 0};
    } else if constexpr (MODE32) {
        // fp32 table: the same staging as below with the pieces converted on their way into LDS (+-1: exact), 64 rows
        // of the table at a time, the next run's loads in flight while the current one is converted and picked up
        u32x2* stage = (u32x2*)smem_raw;                               // fp16 [64][K] as 8-byte pieces
        const f32x4* src = (const f32x4*)hadK;
        const int total = (K * K) >> 2;                                // 16-byte pieces (four coefficients) of hadK
        const int count = (64 * K) >> 2;                               // ... of 64 rows: at most 2 KS2 per thread
        constexpr int P = 2 * KS2;
        f32x4 hk[2][P];
        auto fetch = [&](int i, int b) {
#pragma unroll
            for (int j = 0; j < P; ++j) {
                const int pc = tid + j * HT, at = i * count + pc;
                hk[b][j] = src[pc < count && at < total ? at : 0];
            }
        };
        fetch(0, 0);
#pragma unroll
        for (int i = 0; i < CHUNKS; ++i) {
            if (i + 1 < CHUNKS) fetch(i + 1, (i + 1) & 1);
#pragma unroll
            for (int j = 0; j < P; ++j) {
                const int pc = tid + j * HT;
                const f32x4 w = hk[i & 1][j];
                if (pc < count) stage[pc] = u32x2{cvt_f16x2(w[0], w[1]), cvt_f16x2(w[2], w[3])};
            }
            __syncthreads();
            if (i < TPW) {
                const int hr = (wave + 4 * i) * 16 + l16;
#pragma unroll
                for (int ks = 0; ks < KS2; ++ks)
#pragma unroll
                    for (int hh = 0; hh < 2; ++hh) {
                        const int hc = ks * 32 + hh * 16 + g * 4;
                        const bool ok = hr < K && hc < K;
                        f16x4 v = *(const f16x4*)((const f16*)stage + (ok ? (wave * 16 + l16) * K + hc : 0));
                        if (!ok) v = f16x4{(f16)0, (f16)0, (f16)0, (f16)0};
#pragma unroll
                        for (int e = 0; e < 4; ++e) hf[i][ks][hh * 4 + e] = v[e];
                    }
            }
            __syncthreads();
        }
        u32x4* clr = (u32x4*)smem_raw;
        for (int i = tid; i < 2 * CT * NT * 32; i += HT) clr[i] = u32x4{0, 0, 0, 0};
    } else {
        u32x4* stage = (u32x4*)smem_raw;
        const u32x4* src = (const u32x4*)hadK;
        const int total = (K * K) >> 3;                                // 16-byte pieces of hadK (orders are multiples of 4)
        const int count = (64 * K) >> 3;                               // ... of 64 rows: at most KS2 per thread
        // every load of every run is issued before the first is used (one memory latency in all)
        u32x4 hk[CHUNKS][KS2];
#pragma unroll
        for (int i = 0; i < CHUNKS; ++i)
#pragma unroll
            for (int j = 0; j < KS2; ++j) {
                const int pc = tid + j * HT, at = i * count + pc;
                hk[i][j] = src[pc < count && at < total ? at : 0];
            }
#pragma unroll
        for (int i = 0; i < CHUNKS; ++i) {
#pragma unroll
            for (int j = 0; j < KS2; ++j) {
                const int pc = tid + j * HT;
                if (pc < count) stage[pc] = hk[i][j];
            }
            __syncthreads();
            if (i < TPW) {
                const int hr = (wave + 4 * i) * 16 + l16;
#pragma unroll
                for (int ks = 0; ks < KS2; ++ks)
#pragma unroll
                    for (int hh = 0; hh < 2; ++hh) {
                        const int hc = ks * 32 + hh * 16 + g * 4;
                        const bool ok = hr < K && hc < K;
                        f16x4 v = *(const f16x4*)((const f16*)stage + (ok ? (wave * 16 + l16) * K + hc : 0));
                        if (!ok) v = f16x4{(f16)0, (f16)0, (f16)0, (f16)0};
#pragma unroll
                        for (int e = 0; e < 4; ++e) hf[i][ks][hh * 4 + e] = v[e];
                    }
            }
            __syncthreads();
        }
        // T slots of tiles beyond K are never written afterwards: clear once
        for (int i = tid; i < CT * NT * 32; i += HT) stage[i] = u32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int ks = 0; ks < KS2; ++ks) asm volatile("" : "+v"(hf[t][ks]));
    __syncthreads();

    for (; row < rows; row += gridDim.x) {
        const int64_t nrow = row + gridDim.x;
        // ---- stage 1: T = X . H_64 for this wave's tiles
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            {
                const int t = wave + 4 * i;
                u32x4 a0 = xr[i][0], a1 = xr[i][1];
                if (i == TPW - 1) {                          // the tile that may be partial: rows beyond K are zero fragments
                    a0 = dval[i] ? a0 : u32x4{0, 0, 0, 0};
                    a1 = dval[i] ? a1 : u32x4{0, 0, 0, 0};
                }
                const u32x4 a1n = a1 ^ 0x80008000u;
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a0), sb[ct & 1], acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, (ct >> 1) ? a1n : a1), sb[ct & 1], acc, 0, 0, 0);
                    u32x2 hi;
                    if constexpr (MODE32) {
                        float tv[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) tv[e] = acc[e] * scale;
                        u32x2 lo;
#pragma unroll
                        for (int e = 0; e < 2; ++e) {
                            hi[e] = narrow_f16x2(tv[2 * e], tv[2 * e + 1]);
                            const f16x2 h = as_f16x2(hi[e]);
                            lo[e] = narrow_f16x2(tv[2 * e] - (float)h[0], tv[2 * e + 1] - (float)h[1]);
                        }
                        Tlo[(ct * NT + t) * 64 + lane] = lo;
                    } else {
                        hi[0] = narrow_f16x2(acc[0] * scale, acc[1] * scale);
                        hi[1] = narrow_f16x2(acc[2] * scale, acc[3] * scale);
                    }
                    Tl[(ct * NT + t) * 64 + lane] = hi;
                }
            }
        }
        // the next row's loads, a whole turn ahead (unconditional, like every store below: with a fixed number of
        // memory operations per turn the wait for these loads, a turn later, need not include the stores issued
        // after them; the last turn re-reads its own row)
        load_row(x + (nrow < rows ? nrow : row) * (int64_t)n);
        __syncthreads();
        // ---- stage 2: Y^T = T^T . hadK^T; results stay in registers
        float mxf = 0.f;
        u32x2 yv[TPW][CT];
        float probe = 0.f;                                   // one output of a row that always exists (K >= 64)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            // fragments of T one contraction step ahead of their use (8 registers; a whole column tile's set ahead
            // was no faster, and three workgroups per CU, which these registers would allow, spilled and lost 15 %)
            auto frag = [&](const u32x2* plane, int ks) {
                const u32x2 p0 = plane[(ct * NT + 2 * ks) * 64 + lane], p1 = plane[(ct * NT + 2 * ks + 1) * 64 + lane];
                return u32x4{p0[0], p0[1], p1[0], p1[1]};
            };
            f32x4 acc[TPW];
#pragma unroll
            for (int i = 0; i < TPW; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
            u32x4 th = frag(Tl, 0), tl = MODE32 ? frag(Tlo, 0) : u32x4{0, 0, 0, 0};
#pragma unroll
            for (int ks = 0; ks < KS2; ++ks) {
                __builtin_amdgcn_sched_barrier(0);           // (keeps the scheduler from hoisting every read to the top)
                const u32x4 cur = th, curl = tl;
                if (ks + 1 < KS2) {
                    th = frag(Tl, ks + 1);
                    if constexpr (MODE32) tl = frag(Tlo, ks + 1);
                }
#pragma unroll
                for (int i = 0; i < TPW; ++i) {
                    acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, cur), hf[i][ks], acc[i], 0, 0, 0);
                    if constexpr (MODE32)
                        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, curl), hf[i][ks], acc[i], 0, 0, 0);
                }
            }
            if (ct == 0) probe = acc[0][0];
#pragma unroll
            for (int i = 0; i < TPW; ++i) {
                yv[i][ct][0] = cvt_f16x2(acc[i][0], acc[i][1]);
                yv[i][ct][1] = cvt_f16x2(acc[i][2], acc[i][3]);
                // (rows of hadK beyond its order are zero fragments: their outputs are 0, or NaN from 0 . inf, which
                // the maximum instruction drops)
                mxf = __builtin_fmaxf(__builtin_fmaxf(mxf, __builtin_fabsf(acc[i][0])), __builtin_fabsf(acc[i][1]));
                mxf = __builtin_fmaxf(__builtin_fmaxf(mxf, __builtin_fabsf(acc[i][2])), __builtin_fabsf(acc[i][3]));
            }
        }
        // ---- this row's maximum: rounded once; a wave that sees anything non-finite takes the exact form
        u32 mx = f16_bits((f16)mxf);
        if (__builtin_amdgcn_ballot_w64(mx >= 0x7c00u || probe != probe) != 0) {
            u16x2 mx2 = {0, 0};
#pragma unroll
            for (int i = 0; i < TPW; ++i)
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    // (magnitude bits; rows beyond hadK's order do not count: 0 . inf leaves NaNs there)
                    mx2 = __builtin_elementwise_max(mx2, __builtin_bit_cast(u16x2, dval[i] ? yv[i][ct][0] & 0x7fff7fffu : 0u));
                    mx2 = __builtin_elementwise_max(mx2, __builtin_bit_cast(u16x2, dval[i] ? yv[i][ct][1] & 0x7fff7fffu : 0u));
                }
            mx = mx2[0] > mx2[1] ? mx2[0] : mx2[1];
        }
        mx = wave_max_u32_dpp(mx);
        if (lane == 0) red[wave] = mx;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < HT / QR_WAVE; ++w) mx = mx > red[w] ? mx : red[w];
        const f16 sh = quantizer_scale(f16_from_bits((unsigned short)mx), clip);
        scales[row] = sh;                                     // every lane, the same value: no branch around the store
        const float sp = (float)sh;
        // ---- codes: lanes l16 + 16 g hold, for output row k' = 16 t + l16, the columns 16 ct + 4 g .. + 3
        u32 c01[TPW], c23[TPW];
        if (fast_quant_ok(mx, sp)) {
            const FastRecip fq = make_fast_recip(sp);
            // no clamp where it cannot act: |x| <= amax and a normal scale >= (amax / 7) (1 - 2^-11)^2 keep |x / s| below 7.5
            if (clip >= 1.0f && sp >= 6.103515625e-05f) {
#pragma unroll
                for (int i = 0; i < TPW; ++i) {
                    u32 b0[4], b1[4];
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        b0[w] = sym_pair_fast<false>(yv[i][w >> 1][w & 1], fq);
                        b1[w] = sym_pair_fast<false>(yv[i][2 + (w >> 1)][w & 1], fq);
                    }
                    c01[i] = pack_nibbles8(b0);
                    c23[i] = pack_nibbles8(b1);
                }
            } else {
#pragma unroll
                for (int i = 0; i < TPW; ++i) {
                    u32 b0[4], b1[4];
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        b0[w] = sym_pair_fast<true>(yv[i][w >> 1][w & 1], fq);
                        b1[w] = sym_pair_fast<true>(yv[i][2 + (w >> 1)][w & 1], fq);
                    }
                    c01[i] = pack_nibbles8(b0);
                    c23[i] = pack_nibbles8(b1);
                }
            }
        } else {
            const bool fs = scale_fast_ok(sp);
            const float rs = fs ? 1.0f / sp : 0.0f;
#pragma unroll
            for (int i = 0; i < TPW; ++i) {
                c01[i] = sym_codes8(u32x4{yv[i][0][0], yv[i][0][1], yv[i][1][0], yv[i][1][1]}, sp, rs, fs);
                c23[i] = sym_codes8(u32x4{yv[i][2][0], yv[i][2][1], yv[i][3][0], yv[i][3][1]}, sp, rs, fs);
            }
        }
        // piece (g, ct) -> lane ct: first the halves of the wave (g and g ^ 2), then neighbouring rows of 16 lanes
        u32x2* qrow = (u32x2*)(q + row * (int64_t)nchunks);
        u32x2 outv[TPW];
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            const auto s1 = __builtin_amdgcn_permlane32_swap(c01[i], c23[i], false, false);
            const u32 ev = __builtin_amdgcn_perm(s1[1], s1[0], 0x05040100u);
            const u32 od = __builtin_amdgcn_perm(s1[1], s1[0], 0x07060302u);
            const auto s2 = __builtin_amdgcn_permlane16_swap(ev, od, false, false);
            outv[i] = u32x2{__builtin_amdgcn_perm(s2[1], s2[0], 0x05040100u), __builtin_amdgcn_perm(s2[1], s2[0], 0x07060302u)};
        }
        // lanes on rows beyond K store their first tile's piece once more (K >= 64: that row exists).  The codes are
        // written THROUGH the L2 (device-scope stores): they stay there for the GEMM that follows, and the 11 MB of a
        // 2048-row launch are not left to be written back in one burst when the kernel ends (2048 x 11008: 20.0 -> 18.9 us)
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            const int kp = (wave + 4 * i) * 16 + l16;
            store_through(&qrow[(dval[i] ? kp : wave * 16 + l16) * CT + g], dval[i] ? outv[i] : outv[0]);
        }
        // Tl is next written after the second barrier of this turn, which every wave reaches only after its stage-2
        // reads; red[] is next written after the next row's first barrier.  (A form with T double-buffered and ONE
        // barrier per row -- the next row's stage 1 ahead of it -- was measured no faster.)
    }
}

template <bool MODE32, int KS2>
__global__ __launch_bounds__(HT, 2) void hadamard_m64r_kernel(const f16* __restrict__ x, int64_t rows, int n, int K,
                                                            const void* __restrict__ hadK, float scale, float clip,
                                                            u32* __restrict__ q, f16* __restrict__ scales, int signs) {
    constexpr int NT = 2 * KS2, TPW = (NT + 3) / 4;
    extern __shared__ f32x4 smem_raw[];
    __shared__ u32 red[HT / QR_WAVE];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // (both forms pass the same barriers: two per 64 rows of hadK and one more before the loop, two per row)
    if ((wave + 4 * (TPW - 1)) * 16 < K) hadamard_m64r_rows<MODE32, KS2, TPW, TPW>(x, rows, n, K, hadK, scale, clip, q, scales, smem_raw, red, signs);
    else hadamard_m64r_rows<MODE32, KS2, TPW - 1, TPW>(x, rows, n, K, hadK, scale, clip, q, scales, smem_raw, red, signs);
}

// A power-of-two row of 1024..16384 elements is H_K (x) H_m with both factors Sylvester: the same
// kernel applies with a generated outer factor, in its fp32-precision mode so that the result is
// rounded to fp16 once, like a plain fp32 transform.  Returns the outer order (0: not applicable).
int pow2_split(int n) {
    if (n < 1024 || n > 16384 || (n & (n - 1)) != 0) return 0;
    return n <= 8192 ? n / 64 : n / 128;
}

bool mm_applies(int n, int K) {
    if (K <= 1 || K > 32 * KS_MAX || (K & 3) != 0) return false;     // hadK is fetched four columns at a time
    const int m = n / K;
    return m == 64 || m == 128;
}

template <bool MODE32, bool QUANT>
int launch_hadamard_mm(const void* x, void* y, int64_t rows, int n, int K, const void* hadK, float scale, float clip,
                       void* q, void* scales, hipStream_t st, int ident = 0, int signs = 0) {
    const int m = n / K;
    const int KS2 = ((K + 31) & ~31) >> 5;
    if (m == 128 && KS2 >= 2 && KS2 != 3 && !ident && !MODE32 && QUANT && y == nullptr && hadK != nullptr && ((uintptr_t)x & 15) == 0) {
        // m = 128 behind one of the reference's tables of order 36 and more (Llama-2-13B: 5120 = 40 x 128, 13824 =
        // 108 x 128): the lean fused kernel with eight column tiles.  Orders 140 .. 172 need more registers than two
        // workgroups per CU leave a wave (231 .. 260 spilled) and run one workgroup per CU.
        const size_t ldsq = (size_t)8192 * KS2;
#define QR_M128Q(KS, SMALL)                                                                                            \
    do {                                                                                                               \
        auto kern = hadamard_m64q_kernel<KS, 7, SMALL>;                                                                \
        const int64_t cap = (int64_t)qr_device().cus * qr_blocks_per_cu((const void*)kern, HT, ldsq);                  \
        const unsigned grid = (unsigned)(rows < cap ? rows : cap);                                                     \
        kern<<<dim3(grid), dim3(HT), ldsq, st>>>((const f16*)x, rows, n, K, (const f16*)hadK, scale, clip, (u32*)q,    \
                                                 (f16*)scales);                                                        \
    } while (0)
        switch (KS2) {
            case 2: QR_M128Q(2, true); break;
            case 4: QR_M128Q(4, false); break;
            case 5: QR_M128Q(5, false); break;
            default: QR_M128Q(6, false); break;
        }
#undef QR_M128Q
        return qr_launch_status();
    }
    if (m == 64 && K >= 64 && !ident) {
        // the latency-organised kernel (it relies on every wave's first tile lying inside hadK), while
        // two workgroups still fit on a CU
        const int tpw = (2 * KS2 + 3) / 4;
        const size_t lds64 = (size_t)(MODE32 ? 2 : 1) * 4096 * KS2 + (size_t)tpw * (64 * 72 * 2 + 4 * 2048);
        if (QUANT && y == nullptr && (MODE32 || hadK != nullptr) && ((uintptr_t)x & 15) == 0 &&
            ((uintptr_t)hadK & (signs ? 3 : 15)) == 0) {
            // fused, no copy of the transformed rows wanted: the lean kernel (T alone in LDS; two planes of it in the
            // fp32-precision mode)
            const size_t ldsq = (size_t)(MODE32 ? 2 : 1) * 4096 * KS2;
#define QR_M64Q(KS)                                                                                                    \
    do {                                                                                                               \
        auto kern = hadamard_m64r_kernel<MODE32, KS>;                                                                  \
        if (ldsq > 48 * 1024) {                                                                                        \
            hipError_t e = qr_allow_dynamic_lds((const void*)kern, ldsq);                                              \
            if (e != hipSuccess) return (int)e;                                                                        \
        }                                                                                                              \
        const int64_t cap = (int64_t)qr_device().cus * qr_blocks_per_cu((const void*)kern, HT, ldsq);                  \
        const unsigned grid = (unsigned)(rows < cap ? rows : cap);                                                     \
        kern<<<dim3(grid), dim3(HT), ldsq, st>>>((const f16*)x, rows, n, K, hadK, scale, clip, (u32*)q, (f16*)scales,  \
                                                 signs);                                                               \
    } while (0)
            // (orders of 64 and more among the reference's tables: 108, 140, 156, 172)
            if (KS2 >= 4) {
                switch (KS2) {
                    case 4: QR_M64Q(4); break;
                    case 5: QR_M64Q(5); break;
                    default: QR_M64Q(6); break;
                }
                return qr_launch_status();
            }
#undef QR_M64Q
        }
        if (signs) return QR_E_UNSUPPORTED;
        if (lds64 <= 80 * 1024) {
#define QR_M64(KS)                                                                                                     \
    do {                                                                                                               \
        auto kern = hadamard_m64_kernel<MODE32, QUANT, KS>;                                                            \
        if (lds64 > 48 * 1024) {                                                                                       \
            hipError_t e = qr_allow_dynamic_lds((const void*)kern, lds64);                                             \
            if (e != hipSuccess) return (int)e;                                                                        \
        }                                                                                                              \
        const int64_t cap = (int64_t)qr_device().cus * qr_blocks_per_cu((const void*)kern, HT, lds64);                                    \
        const unsigned grid = (unsigned)(rows < cap ? rows : cap);                                                     \
        kern<<<dim3(grid), dim3(HT), lds64, st>>>((const f16*)x, (f16*)y, rows, n, K, hadK, scale, clip, (u32*)q,      \
                                                  (f16*)scales);                                                       \
    } while (0)
            switch (KS2) {
                case 1: QR_M64(1); break;
                case 2: QR_M64(2); break;
                case 3: QR_M64(3); break;
                case 4: QR_M64(4); break;
                case 5: QR_M64(5); break;
                default: QR_M64(6); break;
            }
#undef QR_M64
            return qr_launch_status();
        }
    }
    const size_t lds0 = (size_t)(MODE32 ? 2 : 1) * (m / 16) * KS2 * 64 * 16 + (((size_t)K * (m + 8) + 7) & ~(size_t)7) * 2;
    const size_t lds_x = lds0 + (size_t)KS2 * 32 * m * 2;
    // the staged-input form when at least two workgroups still fit on a CU
    const bool xlds = lds_x <= 78 * 1024;
    const size_t lds = xlds ? lds_x : lds0;
#define QR_MM(L2M, KS, XL)                                                                                             \
    do {                                                                                                               \
        auto kern = hadamard_mm_kernel<MODE32, QUANT, L2M, KS, XL>;                                                    \
        if (lds > 48 * 1024) {                                                                                         \
            hipError_t e = qr_allow_dynamic_lds((const void*)kern, lds);                                               \
            if (e != hipSuccess) return (int)e;                                                                        \
        }                                                                                                              \
        const int64_t cap = (int64_t)qr_device().cus * qr_blocks_per_cu((const void*)kern, HT, lds);                                      \
        const unsigned grid = (unsigned)(rows < cap ? rows : cap);                                                     \
        kern<<<dim3(grid), dim3(HT), lds, st>>>((const f16*)x, (f16*)y, rows, n, K, hadK, scale, clip, (u32*)q,        \
                                                (f16*)scales, ident);                                                  \
    } while (0)
#define QR_MM_X(L2M, KS)                 \
    if (xlds) QR_MM(L2M, KS, true);      \
    else QR_MM(L2M, KS, false)
#define QR_MM_K(L2M)                       \
    switch (KS2) {                         \
        case 1: QR_MM_X(L2M, 1); break;    \
        case 2: QR_MM_X(L2M, 2); break;    \
        case 3: QR_MM_X(L2M, 3); break;    \
        case 4: QR_MM_X(L2M, 4); break;    \
        case 5: QR_MM_X(L2M, 5); break;    \
        default: QR_MM_X(L2M, 6); break;   \
    }
    if (m == 64) { QR_MM_K(6) }
    else { QR_MM_K(7) }
#undef QR_MM_K
#undef QR_MM_X
#undef QR_MM
    return qr_launch_status();
}

// ---- K > 1 with a long power-of-two factor (m = 512 or 1024), fp16 I/O ---------------------------
// Decode-sized inputs have few rows, so the row itself must supply the parallelism: 1024 threads per
// row.  The power-of-two factor comes first, segment by segment (a segment = the m values of one k):
//   m = 1024 on the matrix cores, as H_32 (x) H_32 over the segment viewed as [b][c] = [32][32]:
//     stage A  T[b][c'] = sum_c X[b][c] H_32[c][c']: the first operand is a 16 x 32 tile of X exactly as
//              it lies in memory (16 bytes per lane, 1 KB per wave and load), fp32 accumulation;
//     stage B  U[b'][c'] = sum_b H_32[b'][b] T[b][c']: with the contraction index taken in the order
//              b = 16 (t / 4) + 4 (lane / 16) + t % 4, the accumulators of stage A's two row tiles ARE the
//              second operand (no exchange between lanes); T is split into fp16 hi + lo (two MFMAs), so
//              the result has fp32 accuracy and is rounded to fp16 once, after the scale, as in the
//              butterfly form;
//     a wave takes two k and both halves of c' (every byte of the row is loaded once), and packs its two results
//     per position into one 4-byte LDS write in the fragment order of the hadK stage;
//   m = 512 with butterflies in registers (8 values per chunk, 64 lanes: 3 + 6 levels, no LDS), scattered
//     into the same order as 2-byte writes.
// The hadK factor then runs on the matrix cores as in hadamard_mm_kernel (T^T as first operand, hadK
// fragments in registers, 8-byte result writes).  All of a row's loads are issued at once and the next
// row's are requested before the matrix stage.
template <bool QUANT, int CPL>
__global__ __launch_bounds__(1024) void hadamard_bm_kernel(const f16* __restrict__ x, f16* __restrict__ y, int64_t rows,
                                                           int n, int K, const f16* __restrict__ hadK, float scale,
                                                           float clip, u32* __restrict__ q, f16* __restrict__ scales) {
    constexpr int BT = 1024, NW = 16;
    constexpr int M_ = 512 * CPL, LOG2M = CPL == 1 ? 9 : 10;
    constexpr int CT = M_ / 16;                  // 16-column tiles
    constexpr int SPW = 4 / CPL;                 // segments per wave (K <= 16 * SPW)
    constexpr int KS2 = CPL == 1 ? 2 : 1;        // contraction steps of 32
    constexpr int RT = SPW;                      // 16-row tiles of hadK
    constexpr int TS = 17;                       // u32x4 units per (step, k-group, column tile): 16 + 1 pad
    constexpr int YS = M_ + 8;
    extern __shared__ f32x4 smem_raw[];
    __shared__ u32 red[NW];
    u32x4* Tl = (u32x4*)smem_raw;                // [KS2][4][CT][TS]
    f16* Yl = (f16*)(Tl + KS2 * 4 * CT * TS);    // [K][YS]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int nchunks = n >> 3;

    // m = 1024: a wave takes the two segments k = 2 wave, 2 wave + 1 and both halves of c', so that every byte of the
    // row is requested once (a CU's vector memory path takes a row in at ~60 GB/s: with the halves of c' on different
    // waves, each loading the unit's segments, a one-row launch waited 4.3 us for 130 KB); Sylvester fragments of
    // both stages
    constexpr int XL = CPL == 2 ? 4 : SPW * CPL;
    const bool works = CPL == 2 && wave * 2 < K;
    u32x4 raw[XL];
    auto request = [&](int64_t row) {
        if (CPL == 2) {
#pragma unroll
            for (int sg = 0; sg < 2; ++sg)          // (waves beyond the last pair repeat wave 0's loads and drop them: no branch)
#pragma unroll
                for (int bt = 0; bt < 2; ++bt)
                    raw[sg * 2 + bt] = *((const u32x4*)(x + row * (int64_t)n) + ((works ? wave : 0) * 2 + sg) * 128 + bt * 64 + l16 * 4 + g);
            return;
        }
#pragma unroll
        for (int sg = 0; sg < SPW; ++sg) {
            const int k = wave + NW * sg;
#pragma unroll
            for (int i = 0; i < CPL; ++i)
                raw[sg * CPL + i] = k < K ? *((const u32x4*)(x + row * (int64_t)n) + k * (M_ / 8) + i * 64 + lane)
                                          : u32x4{0, 0, 0, 0};
        }
    };
    int64_t row = blockIdx.x;
    if (row < rows) request(row);           // in flight while the fragments are made and T is cleared
    f16x8 ha[2], hb[2];
    if (CPL == 2) {
#pragma unroll
        for (int t = 0; t < 8; ++t) {
#pragma unroll
            for (int cth = 0; cth < 2; ++cth) ha[cth][t] = (__builtin_popcount((g * 8 + t) & (cth * 16 + l16)) & 1) ? (f16)-1.0f : (f16)1.0f;
            const int b = 16 * (t >> 2) + 4 * g + (t & 3);
#pragma unroll
            for (int bt = 0; bt < 2; ++bt) hb[bt][t] = (__builtin_popcount(b & (bt * 16 + l16)) & 1) ? (f16)-1.0f : (f16)1.0f;
        }
    }
    // hadK fragments (second MFMA operand): column k' = rt*16 + l16, contraction k = ks*32 + g*8 + j
    f16x8 hf[RT][KS2];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int ks = 0; ks < KS2; ++ks)
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                const int hr = rt * 16 + l16, hc = ks * 32 + g * 8 + hh * 4;
                f16x4 v = {(f16)0, (f16)0, (f16)0, (f16)0};
                if (hr < K && hc < K) v = *(const f16x4*)(hadK + hr * K + hc);
#pragma unroll
                for (int e = 0; e < 4; ++e) hf[rt][ks][hh * 4 + e] = v[e];
            }
    // slots of T for k >= K are never written afterwards: clear once
    for (int i = tid; i < KS2 * 4 * CT * TS; i += BT) Tl[i] = u32x4{0, 0, 0, 0};

    __syncthreads();
    for (; row < rows; row += gridDim.x) {
        // ---- phase 1: the power-of-two factor of every segment, results in fragment order in LDS
        if (CPL == 2) {
            if (works) {
#pragma unroll
                for (int cth = 0; cth < 2; ++cth) {
                    u32 o[2][2][2];                      // [segment of the pair][b' tile][pair of e]: fp16 pairs
#pragma unroll
                    for (int sg = 0; sg < 2; ++sg) {
                        // T = hi + lo, both fp16, as packed pairs (the difference is exact in fp32, so one rounding each)
                        typedef float f32x2_t __attribute__((ext_vector_type(2)));
                        u32x4 whi, wlo;
#pragma unroll
                        for (int bt = 0; bt < 2; ++bt) {
                            const f32x4 da = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, raw[sg * 2 + bt]), ha[cth],
                                                                                  f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
                            for (int pr = 0; pr < 2; ++pr) {
                                const f16x2 hi = __builtin_convertvector(f32x2_t{da[2 * pr], da[2 * pr + 1]}, f16x2);
                                const f16x2 lo = __builtin_convertvector(f32x2_t{da[2 * pr] - (float)hi[0], da[2 * pr + 1] - (float)hi[1]}, f16x2);
                                whi[bt * 2 + pr] = __builtin_bit_cast(u32, hi);
                                wlo[bt * 2 + pr] = __builtin_bit_cast(u32, lo);
                            }
                        }
                        const f16x8 thi = __builtin_bit_cast(f16x8, whi), tlo = __builtin_bit_cast(f16x8, wlo);
#pragma unroll
                        for (int bt = 0; bt < 2; ++bt) {
                            f32x4 db = __builtin_amdgcn_mfma_f32_16x16x32_f16(hb[bt], thi, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                            db = __builtin_amdgcn_mfma_f32_16x16x32_f16(hb[bt], tlo, db, 0, 0, 0);
                            o[sg][bt][0] = narrow_f16x2(db[0] * scale, db[1] * scale);
                            o[sg][bt][1] = narrow_f16x2(db[2] * scale, db[3] * scale);
                        }
                    }
                    // position (b' = 16 bt + 4 g + e, c' = 16 cth + l16) = column tile 2 b' + cth, column l16; the pair's
                    // two k are one 32-bit word of that position's fragment (k = 2 wave, 2 wave + 1: k-group wave / 4)
                    u32* const dst = (u32*)(Tl + ((wave >> 2) * CT + cth) * TS + l16) + (wave & 3);
#pragma unroll
                    for (int bt = 0; bt < 2; ++bt)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const u32 sel = (e & 1) ? 0x07060302u : 0x05040100u;      // high or low halves of two dwords
                            dst[(2 * (16 * bt + 4 * g + e)) * TS * 4] = __builtin_amdgcn_perm(o[1][bt][e >> 1], o[0][bt][e >> 1], sel);
                        }
                }
            }
        } else {
#pragma unroll
        for (int sg = 0; sg < SPW; ++sg) {
            const int k = wave + NW * sg;
            if (k < K) {
                float v[CPL][8];
#pragma unroll
                for (int i = 0; i < CPL; ++i) {
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        v[i][2 * w] = (float)f16_from_bits((unsigned short)(raw[sg * CPL + i][w] & 0xffffu));
                        v[i][2 * w + 1] = (float)f16_from_bits((unsigned short)(raw[sg * CPL + i][w] >> 16));
                    }
                    reg_fwht8(v[i]);
                    lane_stage<1>(v[i], lane);
                    lane_stage<2>(v[i], lane);
                    lane_stage<4>(v[i], lane);
                    lane_stage<8>(v[i], lane);
                    lane_stage<16>(v[i], lane);
                    lane_stage<32>(v[i], lane);
                }
                const int ks = k >> 5, kgp = (k & 31) >> 3, kj = k & 7;
#pragma unroll
                for (int i = 0; i < CPL; ++i) {
                    const int r0 = (i * 64 + lane) * 8;
                    f16* dst = (f16*)(Tl + ((ks * 4 + kgp) * CT + (r0 >> 4)) * TS + (r0 & 8)) + kj;
#pragma unroll
                    for (int e = 0; e < 8; ++e) dst[e * 8] = narrow_f16(v[i][e] * scale);
                }
            }
        }
        }
        const int64_t nrow = row + gridDim.x;
        if (nrow < rows) request(nrow);
        __syncthreads();
        if constexpr (QUANT && CPL == 2) {
            if (y == nullptr) {
                // ---- no copy of the transformed row wanted (the decode step, prefill): the results of the hadK stage
                // stay in registers and become codes there, as in hadamard_m64r_kernel -- same layout: lanes l16 + 16 g
                // hold, for output row k' = 16 rt + l16, the columns 16 c + 4 g .. + 3 of this wave's four column tiles
                // (64 consecutive columns of the segment) -- so the row's trip through LDS and the second pass over it
                // are gone: one barrier (for the row maximum) instead of a barrier, 16-byte reads and a 120-instruction loop
                bool dval[RT];
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) dval[rt] = rt * 16 + l16 < K;
                f16x8 th4[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) th4[c] = __builtin_bit_cast(f16x8, Tl[(g * CT + wave * 4 + c) * TS + l16]);
                u32x2 yv[RT][4];
                float mxf = 0.f, probe = 0.f;
#pragma unroll
                for (int c = 0; c < 4; ++c)
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) {
                        const f32x4 acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(th4[c], hf[rt][0], f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                        if (c == 0 && rt == 0) probe = acc[0];
                        yv[rt][c][0] = cvt_f16x2(acc[0], acc[1]);
                        yv[rt][c][1] = cvt_f16x2(acc[2], acc[3]);
                        // (rows of hadK beyond its order are zero fragments: their outputs are 0, or NaN from 0 . inf,
                        // which the maximum instruction drops)
                        mxf = __builtin_fmaxf(__builtin_fmaxf(mxf, __builtin_fabsf(acc[0])), __builtin_fabsf(acc[1]));
                        mxf = __builtin_fmaxf(__builtin_fmaxf(mxf, __builtin_fabsf(acc[2])), __builtin_fabsf(acc[3]));
                    }
                // the row's maximum: rounded once (rounding is monotone); an infinity or NaN anywhere in the row reaches
                // every output, so one output per lane tells, and a wave that sees one takes the exact form (NaN wins)
                u32 mx = f16_bits((f16)mxf);
                if (__builtin_amdgcn_ballot_w64(mx >= 0x7c00u || probe != probe) != 0) {
                    u16x2 m2 = {0, 0};
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            m2 = __builtin_elementwise_max(m2, __builtin_bit_cast(u16x2, dval[rt] ? yv[rt][c][0] & 0x7fff7fffu : 0u));
                            m2 = __builtin_elementwise_max(m2, __builtin_bit_cast(u16x2, dval[rt] ? yv[rt][c][1] & 0x7fff7fffu : 0u));
                        }
                    mx = m2[0] > m2[1] ? m2[0] : m2[1];
                }
                mx = wave_max_u32_dpp(mx);
                if (lane == 0) red[wave] = mx;          // (last read before the barrier that follows the previous row's phase 1)
                __syncthreads();
#pragma unroll
                for (int w = 0; w < NW; ++w) mx = mx > red[w] ? mx : red[w];
                const f16 sh = quantizer_scale(f16_from_bits((unsigned short)mx), clip);
                if (tid == 0) scales[row] = sh;
                const float sp = (float)sh;
                u32 c01[RT], c23[RT];
                auto codes_from = [&](auto pair) {
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) {
                        u32 b0[4], b1[4];
#pragma unroll
                        for (int w = 0; w < 4; ++w) {
                            b0[w] = pair(yv[rt][w >> 1][w & 1]);
                            b1[w] = pair(yv[rt][2 + (w >> 1)][w & 1]);
                        }
                        c01[rt] = pack_nibbles8(b0);
                        c23[rt] = pack_nibbles8(b1);
                    }
                };
                if (fast_quant_ok(mx, sp)) {
                    const FastRecip fq = make_fast_recip(sp);
                    if (clamp_cannot_act(clip, sp)) codes_from([&](u32 w) { return sym_pair_fast<false>(w, fq); });
                    else codes_from([&](u32 w) { return sym_pair_fast<true>(w, fq); });
                } else {
                    const bool fs = scale_fast_ok(sp);
                    const float rs = fs ? 1.0f / sp : 0.0f;
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) {
                        c01[rt] = sym_codes8(u32x4{yv[rt][0][0], yv[rt][0][1], yv[rt][1][0], yv[rt][1][1]}, sp, rs, fs);
                        c23[rt] = sym_codes8(u32x4{yv[rt][2][0], yv[rt][2][1], yv[rt][3][0], yv[rt][3][1]}, sp, rs, fs);
                    }
                }
                // piece (g, c) -> lane c: first the halves of the wave (g and g ^ 2), then neighbouring rows of 16 lanes;
                // a lane ends with 16 consecutive codes of row k' = 16 rt + l16: columns 64 wave + 16 g ..
                u32x2* qrow = (u32x2*)(q + row * (int64_t)nchunks);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    const auto s1 = __builtin_amdgcn_permlane32_swap(c01[rt], c23[rt], false, false);
                    const u32 ev = __builtin_amdgcn_perm(s1[1], s1[0], 0x05040100u);
                    const u32 od = __builtin_amdgcn_perm(s1[1], s1[0], 0x07060302u);
                    const auto s2 = __builtin_amdgcn_permlane16_swap(ev, od, false, false);
                    const u32x2 outv = {__builtin_amdgcn_perm(s2[1], s2[0], 0x05040100u), __builtin_amdgcn_perm(s2[1], s2[0], 0x07060302u)};
                    if (dval[rt]) qrow[(rt * 16 + l16) * (M_ / 16) + wave * 4 + g] = outv;
                }
                // Tl is next written after the next barrier (the one behind the next row's phase 1 comes after these
                // reads); red[] is next written after that barrier too
                continue;
            }
        }
        // ---- stage 2: Y^T = T^T . hadK^T (the row's largest magnitude is taken on the way: packed unsigned maxima
        // of the fp16 bit patterns without their signs, so that a NaN still wins)
        u16x2 mx2 = {0, 0};
        for (int ct = wave * (CT / NW); ct < (wave + 1) * (CT / NW); ++ct) {
            f16x8 th[KS2];
#pragma unroll
            for (int ks = 0; ks < KS2; ++ks) th[ks] = __builtin_bit_cast(f16x8, Tl[((ks * 4 + g) * CT + ct) * TS + l16]);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                if (rt * 16 < K) {
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < KS2; ++ks)
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(th[ks], hf[rt][ks], acc, 0, 0, 0);
                    const int kp = rt * 16 + l16;
                    if (kp < K) {
                        u32x2 o;
                        o[0] = narrow_f16x2(acc[0], acc[1]);
                        o[1] = narrow_f16x2(acc[2], acc[3]);
                        *(u32x2*)(Yl + kp * YS + ct * 16 + g * 4) = o;
                        if (QUANT) {
                            mx2 = __builtin_elementwise_max(mx2, __builtin_bit_cast(u16x2, o[0] & 0x7fff7fffu));
                            mx2 = __builtin_elementwise_max(mx2, __builtin_bit_cast(u16x2, o[1] & 0x7fff7fffu));
                        }
                    }
                }
            }
        }
        u32 mx = 0;
        if (QUANT) {
            mx = mx2[0] > mx2[1] ? mx2[0] : mx2[1];
            mx = wave_max_u32(mx);
            if (lane == 0) red[wave] = mx;          // (last read before the barrier that follows the previous row's phase 1)
        }
        __syncthreads();
        // ---- stage 3
        if (QUANT) {
#pragma unroll
            for (int w = 0; w < NW; ++w) mx = mx > red[w] ? mx : red[w];
            const f16 sh = quantizer_scale(f16_from_bits((unsigned short)mx), clip);
            if (tid == 0) scales[row] = sh;
            const float s = (float)sh;
            const bool lean = fast_quant_ok(mx, s);
            const FastRecip fq = make_fast_recip(lean ? s : 1.0f);
            // (three loops rather than a choice per chunk: the forms differ in length, the choice is the row's)
            auto codes_of_row = [&](auto form) {
                for (int c = tid; c < nchunks; c += BT) {
                    const u32x4 h = *(const u32x4*)(Yl + ((c * 8) >> LOG2M) * YS + ((c * 8) & (M_ - 1)));
                    q[row * (int64_t)nchunks + c] = form(h);
                    if (y) __builtin_nontemporal_store(h, (u32x4*)(y + row * (int64_t)n) + c);
                }
            };
            if (lean && clamp_cannot_act(clip, s)) {
                codes_of_row([&](u32x4 h) { return sym_codes8_fast<false>(h, fq); });
            } else if (lean) {
                codes_of_row([&](u32x4 h) { return sym_codes8_fast<true>(h, fq); });
            } else {
                const bool fast = scale_fast_ok(s);
                const float rs = fast ? 1.0f / s : 0.0f;
                codes_of_row([&](u32x4 h) { return sym_codes8(h, s, rs, fast); });
            }
        } else {
            for (int c = tid; c < nchunks; c += BT) {
                const u32x4 h = *(const u32x4*)(Yl + ((c * 8) >> LOG2M) * YS + ((c * 8) & (M_ - 1)));
                __builtin_nontemporal_store(h, (u32x4*)(y + row * (int64_t)n) + c);
            }
        }
        // the next row's phase 1 writes Tl (last read before the barrier above) and its stage 2 writes
        // Yl only after the barrier that follows that phase 1
    }
}

bool bm_applies(int n, int K) {
    if (K <= 1 || (K & 3) != 0) return false;                        // hadK is fetched four columns at a time
    const int m = n / K;
    return (m == 512 && K <= 64) || (m == 1024 && K <= 32);
}

template <bool QUANT>
int launch_hadamard_bm(const void* x, void* y, int64_t rows, int n, int K, const void* hadK, float scale, float clip,
                       void* q, void* scales, hipStream_t st) {
    const int m = n / K;
    const int cpl = m / 512;
    const size_t lds = (size_t)(cpl == 1 ? 2 : 1) * 4 * (m / 16) * 17 * 16 + (size_t)K * (m + 8) * 2;
    const unsigned grid = (unsigned)(rows < 256 ? rows : 256);
#define QR_BM(CPL)                                                                                                     \
    do {                                                                                                               \
        auto kern = hadamard_bm_kernel<QUANT, CPL>;                                                                    \
        hipError_t e = qr_allow_dynamic_lds((const void*)kern, lds);   \
        if (e != hipSuccess) return (int)e;                                                                            \
        kern<<<dim3(grid), dim3(1024), lds, st>>>((const f16*)x, (f16*)y, rows, n, K, (const f16*)hadK, scale, clip,   \
                                                  (u32*)q, (f16*)scales);                                              \
    } while (0)
    if (cpl == 1) QR_BM(1);
    else QR_BM(2);
#undef QR_BM
    return qr_launch_status();
}

template <typename IO, bool MODE32, bool QUANT>
int launch_hadamard(const void* x, void* y, int64_t rows, int n, int K, const void* hadK, float scale, float clip,
                    void* q, void* scales, hipStream_t st) {
    const int m = n / K;
    int log2m = 0;
    while ((1 << log2m) < m) ++log2m;
    const int Kr = (K + 15) & ~15;
    const int hs_stride = K > 1 ? ((K + 31) & ~31) + 8 : 0;
    const size_t lds = (size_t)n * 4 + (size_t)Kr * hs_stride * 2;
    if (lds > 160 * 1024 - 64) return QR_E_UNSUPPORTED;
    auto kern = hadamard_kernel<IO, MODE32, QUANT>;
    if (lds > 48 * 1024) {
        hipError_t e = qr_allow_dynamic_lds((const void*)kern, lds);
        if (e != hipSuccess) return (int)e;
    }
    // persistent workgroups: as many as fit the CUs' LDS at once (256 CUs, 160 KB each), so that the
    // hadK staging is paid once per resident workgroup
    const int64_t cap = (int64_t)qr_device().cus * qr_blocks_per_cu((const void*)kern, HT, lds);
    const int64_t grid = rows < cap ? rows : cap;
    kern<<<dim3((unsigned)grid), dim3(HT), lds, st>>>((const IO*)x, (IO*)y, rows, n, K, log2m, hadK, scale, clip,
                                                      (u32*)q, (f16*)scales, hs_stride);
    return qr_launch_status();
}

// Short power-of-two rows (8 ... 64 elements, e.g. the transform across 32 or 64 attention heads on
// a transposed copy, e2e/quantized_llama/modeling_llama.py:108): many rows per workgroup.  A lane
// holds 8 consecutive elements of a row (one 16-byte load, consecutive lanes = consecutive memory),
// n / 8 neighbouring lanes hold a row; three butterfly stages run in the lane, the others between
// lanes (DPP quad permutes for lane distance 1 and 2, a cross-lane read for 4).  fp32 inside, the
// scale applied at the end, rounded to fp16 once.
template <int LPR>
__global__ __launch_bounds__(256) void hadamard_small_kernel(const u32x4* __restrict__ x, u32x4* __restrict__ y,
                                                             int64_t chunks, float scale) {
    const int lane = threadIdx.x & 63;
    const int64_t stride = (int64_t)gridDim.x * 256;
    // every lane of a wave runs the same number of turns: chunks beyond the end are zeros, not stored
    const int64_t turns = (chunks + stride - 1) / stride;
    int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    for (int64_t t = 0; t < turns; ++t, idx += stride) {
        const bool live = idx < chunks;
        const u32x4 v = live ? __builtin_nontemporal_load(x + idx) : u32x4{0, 0, 0, 0};
        float f[8];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const f16x2 h = as_f16x2(v[w]);
            f[2 * w] = (float)h[0];
            f[2 * w + 1] = (float)h[1];
        }
#pragma unroll
        for (int b = 1; b < 8; b <<= 1)
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if ((e & b) == 0) {
                    const float lo = f[e], hi = f[e | b];
                    f[e] = lo + hi;
                    f[e | b] = lo - hi;
                }
#pragma unroll
        for (int d = 1; d < LPR; d <<= 1) {
            const bool upper = (lane & d) != 0;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int own = __builtin_bit_cast(int, f[e]);
                int other;
                if (d == 1) other = __builtin_amdgcn_update_dpp(0, own, 0xB1, 0xF, 0xF, true);        // quad_perm [1,0,3,2]
                else if (d == 2) other = __builtin_amdgcn_update_dpp(0, own, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
                else other = __shfl_xor(own, d, QR_WAVE);
                const float p = __builtin_bit_cast(float, other);
                f[e] = upper ? p - f[e] : f[e] + p;
            }
        }
        if (live) {
            u32x4 o;
#pragma unroll
            for (int w = 0; w < 4; ++w) o[w] = narrow_f16x2(f[2 * w] * scale, f[2 * w + 1] * scale);
            __builtin_nontemporal_store(o, y + idx);
        }
    }
}

int launch_hadamard_small(const void* x, void* y, int64_t rows, int n, float scale, hipStream_t st) {
    const int64_t chunks = rows * (n / 8);
    int64_t blocks = (chunks + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    const dim3 grid((unsigned)blocks), block(256);
    if (n == 8) hadamard_small_kernel<1><<<grid, block, 0, st>>>((const u32x4*)x, (u32x4*)y, chunks, scale);
    else if (n == 16) hadamard_small_kernel<2><<<grid, block, 0, st>>>((const u32x4*)x, (u32x4*)y, chunks, scale);
    else if (n == 32) hadamard_small_kernel<4><<<grid, block, 0, st>>>((const u32x4*)x, (u32x4*)y, chunks, scale);
    else hadamard_small_kernel<8><<<grid, block, 0, st>>>((const u32x4*)x, (u32x4*)y, chunks, scale);
    return qr_launch_status();
}

// Rows whose power-of-two factor is 1, 2 or 4 (e.g. OnlineHadamard(40) across the 40 attention heads
// of Llama-2-13B on a transposed copy: had_40 alone), n <= 128.  A workgroup takes 64 consecutive rows:
// they are staged in LDS as floats, the m-point butterflies run in place with the scale applied (and,
// for fp16 I/O, the rounding to fp16 that the reference's two-step form has between its steps,
// quarot/functional/hadamard.py:99-100), then thread (row, part) forms outputs part, part + 4, ... as
// dot products of hadK rows (LDS broadcast reads) with the staged row, and the results leave through
// LDS as one contiguous block.  fp32 accumulation, one rounding at the end.
template <typename IO>
__global__ __launch_bounds__(256) void hadamard_tiny_kernel(const IO* __restrict__ x, IO* __restrict__ y, int64_t rows,
                                                            int n, int K, const IO* __restrict__ hadK, float scale) {
    constexpr int RW = 64;
    extern __shared__ float tiny_lds[];
    const int m = n / K, ld = n + 1;                        // odd row stride in floats: lanes = rows hit distinct banks
    float* T = tiny_lds;                                    // [RW][ld]
    float* Y = T + RW * ld;                                 // [RW][ld]
    float* H = Y + RW * ld;                                 // [K][K]
    const int tid = threadIdx.x;
    const int64_t row0 = (int64_t)blockIdx.x * RW;
    const int live = (int)((rows - row0) < RW ? (rows - row0) : RW);
    // m == 1: hadK is kept transposed, so that four consecutive outputs read their four coefficients
    // of one k with a single 16-byte broadcast (K % 4 == 0 for every table of the reference)
    const bool blocked = m == 1 && (K & 3) == 0;
    for (int i = tid; i < K * K; i += 256) {
        const float hv = K > 1 ? (float)hadK[i] : 1.0f;
        if (blocked) H[(i % K) * K + i / K] = hv;
        else H[i] = hv;
    }
    const IO* xb = x + row0 * n;
    for (int i = tid; i < live * n; i += 256) T[(i / n) * ld + i % n] = (float)xb[i];
    __syncthreads();
    // m-point Walsh-Hadamard transform of every (row, k) group, scaled
    for (int u = tid; u < live * K; u += 256) {
        float* t = T + (u / K) * ld + (u % K) * m;
        float v[4] = {t[0], m > 1 ? t[1] : 0.f, m > 2 ? t[2] : 0.f, m > 2 ? t[3] : 0.f};
        if (m > 1) {
            const float a = v[0] + v[1], b = v[0] - v[1], c = v[2] + v[3], d = v[2] - v[3];
            v[0] = a; v[1] = b; v[2] = c; v[3] = d;
        }
        if (m > 2) {
            const float a = v[0] + v[2], b = v[1] + v[3], c = v[0] - v[2], d = v[1] - v[3];
            v[0] = a; v[1] = b; v[2] = c; v[3] = d;
        }
        for (int e = 0; e < m; ++e) {
            const float sv = v[e] * scale;
            t[e] = sizeof(IO) == 2 ? (float)narrow_f16(sv) : sv;
        }
    }
    __syncthreads();
    const int r = tid & 63, part = tid >> 6;
    if (r < live && blocked) {
        const float* t = T + r * ld;
        for (int j0 = part * 4; j0 < n; j0 += 16) {
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
            for (int k = 0; k < K; ++k) {
                const f32x4 h4 = *(const f32x4*)(H + k * K + j0);
                const float tv = t[k];
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[e] = __builtin_fmaf(h4[e], tv, acc[e]);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) Y[r * ld + j0 + e] = acc[e];
        }
    } else if (r < live) {
        const float* t = T + r * ld;
        for (int j = part; j < n; j += 4) {
            const int kp = j / m, rr = j - kp * m;
            const float* h = H + kp * K;
            float acc = 0.f;
            for (int k = 0; k < K; ++k) acc = __builtin_fmaf(h[k], t[k * m + rr], acc);
            Y[r * ld + j] = acc;
        }
    }
    __syncthreads();
    IO* yb = y + row0 * n;
    for (int i = tid; i < live * n; i += 256) yb[i] = (IO)Y[(i / n) * ld + i % n];
}

template <typename IO>
int launch_hadamard_tiny(const void* x, void* y, int64_t rows, int n, int K, const void* hadK, float scale, hipStream_t st) {
    const size_t lds = ((size_t)2 * 64 * (n + 1) + (size_t)K * K) * sizeof(float);
    auto kern = hadamard_tiny_kernel<IO>;
    if (lds > 48 * 1024) {
        hipError_t e = qr_allow_dynamic_lds((const void*)kern, lds);
        if (e != hipSuccess) return (int)e;
    }
    const int64_t grid = (rows + 63) / 64;
    if (grid > 0x7fffffffLL) return QR_E_SHAPE;
    kern<<<dim3((unsigned)grid), dim3(256), lds, st>>>((const IO*)x, (IO*)y, rows, n, K, (const IO*)hadK, scale);
    return qr_launch_status();
}

bool tiny_applies(int n, int K) { return n / K < 8 && n <= 128; }

int check_shape(int64_t rows, int n, int K) {
    if (rows < 0 || n <= 0 || K <= 0) return QR_E_SHAPE;
    if (n % K != 0) return QR_E_SHAPE;
    const int m = n / K;
    if ((m & (m - 1)) != 0) return QR_E_SHAPE;
    if ((m < 8 && n > 128) || n > 32768 || K > 32 * KS_MAX) return QR_E_UNSUPPORTED;
    return QR_OK;
}

}  // namespace

extern "C" int qr_hadamard(const void* x, void* y, int64_t rows, int n, int K, const void* hadK, int dtype, float scale,
                           void* stream) {
    int rc = check_shape(rows, n, K);
    if (rc != QR_OK) return rc;
    if (rows == 0) return QR_OK;
    if (!x || !y || (K > 1 && !hadK)) return QR_E_NULL;
    if (((uintptr_t)x & 15) || ((uintptr_t)y & 15)) return QR_E_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    if (tiny_applies(n, K)) {
        if (dtype == QR_DTYPE_F16) return launch_hadamard_tiny<f16>(x, y, rows, n, K, hadK, scale, st);
        if (dtype == QR_DTYPE_F32) return launch_hadamard_tiny<float>(x, y, rows, n, K, hadK, scale, st);
        return QR_E_DTYPE;
    }
    // head-dimension rows: the kernel whose arithmetic the K-cache quantiser shares
    if (dtype == QR_DTYPE_F16 && K == 1 && n == 128) return qr_internal_hadamard128_f16(x, y, rows, scale, st);
    if (dtype == QR_DTYPE_F16 && K == 1 && n <= 64) return launch_hadamard_small(x, y, rows, n, scale, st);
    if (dtype == QR_DTYPE_F16 && K == 1 && pow2_split(n))
        return launch_hadamard_mm<true, false>(x, y, rows, n, pow2_split(n), nullptr, scale, 1.f, nullptr, nullptr, st);
    if (dtype == QR_DTYPE_F16 && bm_applies(n, K))
        return launch_hadamard_bm<false>(x, y, rows, n, K, hadK, scale, 1.f, nullptr, nullptr, st);
    if (dtype == QR_DTYPE_F16 && mm_applies(n, K))
        return launch_hadamard_mm<false, false>(x, y, rows, n, K, hadK, scale, 1.f, nullptr, nullptr, st);
    if (dtype == QR_DTYPE_F16 && km_applies(n, K, false)) {
        int log2m = 0;
        while ((1 << log2m) < n / K) ++log2m;
        return launch_hadamard_km<false, false>(x, y, rows, n, K, log2m, hadK, scale, 1.f, nullptr, nullptr, st);
    }
    if (dtype == QR_DTYPE_F16) return launch_hadamard<f16, false, false>(x, y, rows, n, K, hadK, scale, 1.f, nullptr, nullptr, st);
    if (dtype == QR_DTYPE_F32) return launch_hadamard<float, true, false>(x, y, rows, n, K, hadK, scale, 1.f, nullptr, nullptr, st);
    return QR_E_DTYPE;
}

extern "C" int qr_hadamard_quantize_f16_i4(const void* x, int64_t rows, int n, int K, const void* hadK, int mode,
                                           float scale, float clip, void* q, void* scales, void* y_or_null,
                                           void* stream) {
    int rc = check_shape(rows, n, K);
    if (rc != QR_OK) return rc;
    if (rows == 0) return QR_OK;
    if (!x || !q || !scales || (K > 1 && !hadK)) return QR_E_NULL;
    if (((uintptr_t)x & 15) || ((uintptr_t)y_or_null & 15) || ((uintptr_t)q & 7)) return QR_E_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    const int signs = (mode & QR_HADK_SIGNS) ? 1 : 0;
    mode &= ~QR_HADK_SIGNS;
    if (mode != QR_DTYPE_F16 && mode != QR_DTYPE_F32) return QR_E_DTYPE;
    if (signs) {
        // hadK as sign words: the lean kernel of the m = 64 widths behind a table of order 97 .. 192 only (nothing is
        // launched otherwise: the caller passes the table itself)
        if (K <= 96 || y_or_null || !mm_applies(n, K) || n / K != 64 || ((uintptr_t)hadK & 3)) return QR_E_UNSUPPORTED;
        if (mode == QR_DTYPE_F16) return launch_hadamard_mm<false, true>(x, nullptr, rows, n, K, hadK, scale, clip, q, scales, st, 0, 1);
        return launch_hadamard_mm<true, true>(x, nullptr, rows, n, K, hadK, scale, clip, q, scales, st, 0, 1);
    }
    if (tiny_applies(n, K)) return QR_E_UNSUPPORTED;       // rows this short: qr_hadamard, then qr_quantize_rows_f16_i4
    if (mode == QR_DTYPE_F16 && K == 1 && n == 128) {
        // head-dimension rows: qr_hadamard's kernel for this length adds in another order than the general kernel below
        // (results one fp16 step apart now and then), so the transformed rows are written by THAT kernel and quantised
        // from memory: this call and qr_hadamard followed by the quantiser stay on the same bits.  Without a place for
        // the transformed rows nothing is launched.
        if (!y_or_null) return QR_E_UNSUPPORTED;
        rc = qr_internal_hadamard128_f16(x, y_or_null, rows, scale, st);
        if (rc != QR_OK) return rc;
        return qr_quantize_rows_f16_i4(y_or_null, clip, rows, n, q, scales, stream);
    }
    if (K == 1 && pow2_split(n))
        return launch_hadamard_mm<true, true>(x, y_or_null, rows, n, pow2_split(n), nullptr, scale, clip, q, scales, st);
    if (mode == QR_DTYPE_F16 && bm_applies(n, K))
        return launch_hadamard_bm<true>(x, y_or_null, rows, n, K, hadK, scale, clip, q, scales, st);
    if (mm_applies(n, K)) {
        if (mode == QR_DTYPE_F16) return launch_hadamard_mm<false, true>(x, y_or_null, rows, n, K, hadK, scale, clip, q, scales, st);
        return launch_hadamard_mm<true, true>(x, y_or_null, rows, n, K, hadK, scale, clip, q, scales, st);
    }
    if (km_applies(n, K, mode == QR_DTYPE_F32)) {
        int log2m = 0;
        while ((1 << log2m) < n / K) ++log2m;
        if (mode == QR_DTYPE_F16) return launch_hadamard_km<false, true>(x, y_or_null, rows, n, K, log2m, hadK, scale, clip, q, scales, st);
        return launch_hadamard_km<true, true>(x, y_or_null, rows, n, K, log2m, hadK, scale, clip, q, scales, st);
    }
    if (mode == QR_DTYPE_F16) return launch_hadamard<f16, false, true>(x, y_or_null, rows, n, K, hadK, scale, clip, q, scales, st);
    if (mode == QR_DTYPE_F32) return launch_hadamard<f16, true, true>(x, y_or_null, rows, n, K, hadK, scale, clip, q, scales, st);
    return QR_E_DTYPE;
}

// quant.hip: Hadamard across `heads` groups of 128 + quantiser for head counts that are orders of the
// reference's tables: the fused two-stage kernel with the identity as inner factor
__attribute__((visibility("hidden"))) int qr_internal_heads_matrix_quantize(const void* x, int64_t rows, int heads,
                                                                            const void* hadK, float clip, void* q,
                                                                            void* scales, void* y_or_null, hipStream_t st) {
    const int n = heads * 128;
    if (!mm_applies(n, heads)) return QR_E_UNSUPPORTED;
    return launch_hadamard_mm<false, true>(x, y_or_null, rows, n, heads, hadK, 1.0f / __builtin_sqrtf((float)heads), clip, q,
                                           scales, st, 1);
}
