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
    const bool upper = (lane & MASK) != 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float p = lane_xor<MASK>(v[e]);
        v[e] = upper ? p - v[e] : v[e] + p;
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
    u32x4 raw = __builtin_nontemporal_load((const u32x4*)p);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = (float)f16_from_bits((unsigned short)(raw[i] & 0xffffu));
        v[2 * i + 1] = (float)f16_from_bits((unsigned short)(raw[i] >> 16));
    }
}
__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
    f32x4 a = __builtin_nontemporal_load((const f32x4*)p);
    f32x4 b = __builtin_nontemporal_load((const f32x4*)p + 1);
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
        o[i] = (u32)f16_bits(narrow_f16(v[2 * i])) | ((u32)f16_bits(narrow_f16(v[2 * i + 1])) << 16);
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
        // ---- phase 1
        for (int c0 = 0; c0 < nchunks; c0 += HT) {
            const int c = c0 + tid;             // whole waves share the predicate: nchunks % 64 may be != 0 only
            float v[8];                         // when m < 512, and then exchanges stay inside a segment's lanes
            const bool live = c < nchunks;
            if (live) load8(xr + (int64_t)c * 8, v);
            else {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = 0.f;
            }
            reg_fwht8(v);
            if (lane_stages > 0) lane_stage<1>(v, lane);
            if (lane_stages > 1) lane_stage<2>(v, lane);
            if (lane_stages > 2) lane_stage<4>(v, lane);
            if (lane_stages > 3) lane_stage<8>(v, lane);
            if (lane_stages > 4) lane_stage<16>(v, lane);
            if (lane_stages > 5) lane_stage<32>(v, lane);
            if (live) {
                *(f32x4*)(buf + c * 8) = f32x4{v[0], v[1], v[2], v[3]};
                *(f32x4*)(buf + c * 8 + 4) = f32x4{v[4], v[5], v[6], v[7]};
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
            const bool fast = scale_fast_ok(s);
            const float rs = fast ? 1.0f / s : 0.0f;
            for (int c = tid; c < nchunks; c += HT) {
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = buf[c * 8 + e] * osc;
                u32x4 h = to_f16x8(v);
                q[row * (int64_t)nchunks + c] = sym_codes8(h, s, rs, fast);
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
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
    }
    // persistent workgroups: as many as fit the CUs' LDS at once (256 CUs, 160 KB each), so that the
    // hadK staging is paid once per resident workgroup
    int per_cu = (int)((160 * 1024) / (lds + 1024));
    per_cu = per_cu < 1 ? 1 : (per_cu > 8 ? 8 : per_cu);
    const int64_t cap = 256LL * per_cu;
    const int64_t grid = rows < cap ? rows : cap;
    kern<<<dim3((unsigned)grid), dim3(HT), lds, st>>>((const IO*)x, (IO*)y, rows, n, K, log2m, hadK, scale, clip,
                                                      (u32*)q, (f16*)scales, hs_stride);
    return qr_launch_status();
}

int check_shape(int64_t rows, int n, int K) {
    if (rows < 0 || n <= 0 || K <= 0) return QR_E_SHAPE;
    if (n % K != 0) return QR_E_SHAPE;
    const int m = n / K;
    if ((m & (m - 1)) != 0) return QR_E_SHAPE;
    if (m < 8 || n > 32768 || K > 32 * KS_MAX) return QR_E_UNSUPPORTED;
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
    if (((uintptr_t)x & 15) || ((uintptr_t)y_or_null & 15) || ((uintptr_t)q & 3)) return QR_E_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    if (mode == QR_DTYPE_F16) return launch_hadamard<f16, false, true>(x, y_or_null, rows, n, K, hadK, scale, clip, q, scales, st);
    if (mode == QR_DTYPE_F32) return launch_hadamard<f16, true, true>(x, y_or_null, rows, n, K, hadK, scale, clip, q, scales, st);
    return QR_E_DTYPE;
}
