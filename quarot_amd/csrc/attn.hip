// Paged int4 KV cache: appending quantised vectors to their pages, and single-query (decode) attention
// over the cache with the dequantisation done in registers.
#include "qr_paged.h"

namespace {

// ---- append: pure data movement --------------------------------------------------------------------
// One 16-byte piece per thread: four threads move the 64 code bytes of a (token, head) vector of K and of
// V; the first of them also moves the two {scale, zero} words.
__global__ __launch_bounds__(256) void paged_append_i4_kernel(PagedKV c, const u32x4* __restrict__ key,
                                                              const u32x4* __restrict__ value,
                                                              const u32* __restrict__ kparam, const u32* __restrict__ vparam,
                                                              const int32_t* __restrict__ append_indptr, int64_t tokens) {
    const int64_t pieces = tokens * c.num_heads * 4;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < pieces; i += (int64_t)gridDim.x * 256) {
        const int piece = (int)(i & 3);
        const int64_t vec = i >> 2, token = vec / c.num_heads;
        const int head = (int)(vec - token * c.num_heads);
        int64_t page;
        int entry;
        if (!paged_locate(c, append_indptr, token, page, entry)) continue;
        const int64_t ks = paged_slot(c, page, 0, head, entry), vs = paged_slot(c, page, 1, head, entry);
        ((u32x4*)c.data)[ks * 4 + piece] = key[i];
        ((u32x4*)c.data)[vs * 4 + piece] = value[i];
        if (piece == 0) {
            c.param[ks] = kparam[vec];
            c.param[vs] = vparam[vec];
        }
    }
}

// ---- decode attention --------------------------------------------------------------------------------
// o[b, h, :] = sum_j softmax_j( q[b, h, :] . k_j / sqrt(128) ) v_j over the sequence's cached vectors, with
// k_j[i] = float(code) * scale_j - zero_j formed in fp32 (quantization.cuh:59-84, decode.cuh:492-689).
// HBM-bound: 128 code bytes + 8 parameter bytes per cached position and head.
//
// A workgroup of four waves serves one (sequence, head) -- or one of `splits` interleaved parts of it.
// A wave takes 16 consecutive positions per step, four lanes per position, so that a lane's 16-byte load
// is one quarter (32 dimensions) of a K or V vector and a wave's load instruction covers 1 KB of
// consecutive cache bytes.  Because  q . k_j = scale_j (q . codes_j) - zero_j sum(q)  the inner loop works on
// the codes themselves: byte-to-float conversions of the masked nibbles (the high nibbles come out
// times 16: folded into the multiplier) and one fma per element, in fp32.  Every group of four lanes
// keeps its own running maximum, denominator and 32-dimension accumulator for the positions it visits
// (U of them per step, so the accumulator is rescaled once per U positions); the 64 partial states of
// the workgroup are merged through LDS at the end.
constexpr int AT = 256;
constexpr int AU = 4;                 // positions per lane group and step

__device__ __forceinline__ float quad_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // lanes ^ 1
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // lanes ^ 2
    return v;
}

__device__ __forceinline__ float byte_f32(u32 w, int k) {
    switch (k) {
        case 0: return (float)(w & 0xffu);
        case 1: return (float)((w >> 8) & 0xffu);
        case 2: return (float)((w >> 16) & 0xffu);
        default: return (float)(w >> 24);
    }
}

// ALIGNED: page_size is a multiple of 16, so the 16 positions of a wave step lie in one page
template <bool ALIGNED>
__global__ __launch_bounds__(AT, 4) void paged_decode_i4_kernel(const f16* __restrict__ q, PagedKV c, f16* __restrict__ o,
                                                            float sm_scale_log2, int splits, float* __restrict__ part) {
    __shared__ float st[64 * 4 * 36];                      // [wave * 16 + slot][quarter][m, d, -, -, acc[32]]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int slot = lane >> 2, c4 = lane & 3;
    const int bh = blockIdx.x / splits, sp = blockIdx.x - bh * splits;
    const int b = bh / c.num_heads, h = bh - b * c.num_heads;
    const int p0 = c.indptr[b], npages = c.indptr[b + 1] - p0;
    const int seq_len = npages > 0 ? (npages - 1) * c.page_size + c.last_page_offset[b] : 0;

    // this lane's 32 query values, in the order the code bytes are consumed: word j, byte k holds
    // dimensions 8 j + 2 k (low nibble) and 8 j + 2 k + 1 (high nibble, converted times 16)
    float qlo[4][4], qhi[4][4], qs = 0.f;
    {
        const u32x4* qp = (const u32x4*)(q + (int64_t)bh * 128 + c4 * 32);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const u32x4 w = qp[j];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const f16x2 pr = as_f16x2(w[k]);
                qlo[j][k] = (float)pr[0];
                qhi[j][k] = (float)pr[1] * 0.0625f;
                qs += (float)pr[0] + (float)pr[1];
            }
        }
    }
    qs = quad_sum(qs);                                     // sum of all 128 query values

    float m = -5e4f, d = 0.f, pz = 0.f, acc[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) acc[i] = 0.f;

    const int chunks = (seq_len + 15) >> 4;
    const int cpp = ALIGNED ? c.page_size >> 4 : 1;        // chunks per page
    for (int g0 = sp * 4 + wave; g0 < chunks; g0 += 4 * splits * AU) {
        u32x4 kw[AU], vw[AU];
        u32 kp[AU], vp[AU];
        bool ok[AU];
#pragma unroll
        for (int u = 0; u < AU; ++u) {
            const int g = g0 + u * 4 * splits, pos = g * 16 + slot;
            int it, entry;
            if (ALIGNED) {
                it = g / cpp;                              // wave-uniform
                entry = (g - it * cpp) * 16 + slot;
            } else {
                it = pos / c.page_size;
                entry = pos - it * c.page_size;
            }
            ok[u] = pos < seq_len && it < npages;
            int64_t page = ok[u] ? c.indices[p0 + it] : 0;
            ok[u] = ok[u] && page >= 0 && page < c.num_pages;
            page = ok[u] ? page : 0;
            entry = ok[u] ? entry : 0;
            const int64_t ks = paged_slot(c, page, 0, h, entry), vs = paged_slot(c, page, 1, h, entry);
            kw[u] = __builtin_nontemporal_load((const u32x4*)c.data + ks * 4 + c4);
            vw[u] = __builtin_nontemporal_load((const u32x4*)c.data + vs * 4 + c4);
            kp[u] = c.param[ks];
            vp[u] = c.param[vs];
        }
        float lg[AU], mx = m;
#pragma unroll
        for (int u = 0; u < AU; ++u) {
            float a0 = 0.f, a1 = 0.f;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const u32 lo = kw[u][j] & 0x0F0F0F0Fu, hi = kw[u][j] & 0xF0F0F0F0u;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    a0 = __builtin_fmaf(qlo[j][k], byte_f32(lo, k), a0);
                    a1 = __builtin_fmaf(qhi[j][k], byte_f32(hi, k), a1);
                }
            }
            const float dot = quad_sum(a0 + a1);
            const f16x2 prm = as_f16x2(kp[u]);
            const float x = (dot * (float)prm[0] - (float)prm[1] * qs) * sm_scale_log2;
            lg[u] = ok[u] ? x : -__builtin_inff();
            mx = __builtin_fmaxf(mx, lg[u]);
        }
        const float alpha = __builtin_amdgcn_exp2f(m - mx);
        m = mx;
        d *= alpha;
        pz *= alpha;
#pragma unroll
        for (int i = 0; i < 32; ++i) acc[i] *= alpha;
#pragma unroll
        for (int u = 0; u < AU; ++u) {
            const float p = __builtin_amdgcn_exp2f(lg[u] - m);
            const f16x2 prm = as_f16x2(vp[u]);
            const float ps = p * (float)prm[0], ps16 = ps * 0.0625f;
            d += p;
            pz = __builtin_fmaf(p, (float)prm[1], pz);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const u32 lo = vw[u][j] & 0x0F0F0F0Fu, hi = vw[u][j] & 0xF0F0F0F0u;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    acc[8 * j + 2 * k] = __builtin_fmaf(ps, byte_f32(lo, k), acc[8 * j + 2 * k]);
                    acc[8 * j + 2 * k + 1] = __builtin_fmaf(ps16, byte_f32(hi, k), acc[8 * j + 2 * k + 1]);
                }
            }
        }
    }
    // ---- merge the 64 lane-group states of the workgroup
    float* mine = st + ((wave * 16 + slot) * 4 + c4) * 36;
    mine[0] = m;
    mine[1] = d;
#pragma unroll
    for (int i = 0; i < 32; ++i) mine[4 + i] = acc[i] - pz;          // sum p (code scale - zero)
    __syncthreads();
    if (threadIdx.x < 128) {
        const int dim = threadIdx.x, qd = dim >> 5, r = dim & 31;
        float M = -5e4f;
        for (int s = 0; s < 64; ++s) M = __builtin_fmaxf(M, st[(s * 4 + qd) * 36]);
        float D = 0.f, O = 0.f;
        for (int s = 0; s < 64; ++s) {
            const float* src = st + (s * 4 + qd) * 36;
            const float w = __builtin_amdgcn_exp2f(src[0] - M);
            D = __builtin_fmaf(src[1], w, D);
            O = __builtin_fmaf(src[4 + r], w, O);
        }
        if (splits == 1) {
            o[(int64_t)bh * 128 + dim] = (f16)(O / D);     // an empty sequence gives 0 / 0, as the reference's kernel does
        } else {
            float* dst = part + (int64_t)blockIdx.x * 132;
            if (dim == 0) {
                dst[0] = M;
                dst[1] = D;
            }
            dst[4 + dim] = O;
        }
    }
}

// combines the `splits` partial states of every (sequence, head)
__global__ __launch_bounds__(128) void paged_decode_merge_kernel(const float* __restrict__ part, int splits,
                                                                 f16* __restrict__ o) {
    const int64_t bh = blockIdx.x;
    const int dim = threadIdx.x;
    const float* src = part + bh * splits * 132;
    float M = -5e4f;
    for (int s = 0; s < splits; ++s) M = __builtin_fmaxf(M, src[s * 132]);
    float D = 0.f, O = 0.f;
    for (int s = 0; s < splits; ++s) {
        const float w = __builtin_amdgcn_exp2f(src[s * 132] - M);
        D = __builtin_fmaf(src[s * 132 + 1], w, D);
        O = __builtin_fmaf(src[s * 132 + 4 + dim], w, O);
    }
    o[bh * 128 + dim] = (f16)(O / D);
}

int check_cache(const void* kv_data, const void* kv_param, const void* kv_indptr, const void* kv_indices,
                const void* last_page_offset, int64_t num_pages, int num_layers, int layer_idx, int num_heads,
                int page_size, int head_dim, int64_t batch_size) {
    if (num_pages < 0 || num_layers <= 0 || layer_idx < 0 || layer_idx >= num_layers || num_heads <= 0 || page_size <= 0 ||
        batch_size < 0 || batch_size > 0x7fffffff || head_dim <= 0)
        return QR_E_SHAPE;
    if (head_dim != 128) return QR_E_UNSUPPORTED;          // as the reference's bindings (CHECK_EQ(head_dim, 128))
    if (batch_size == 0) return QR_OK;
    if (!kv_data || !kv_param || !kv_indptr || !kv_indices || !last_page_offset) return QR_E_NULL;
    if (((uintptr_t)kv_data & 15) || ((uintptr_t)kv_param & 3)) return QR_E_ALIGN;
    return QR_OK;
}

}  // namespace

__attribute__((visibility("hidden"))) PagedKV qr_internal_paged_kv(void* kv_data, void* kv_param, const void* kv_indptr,
                                                                    const void* kv_indices, const void* last_page_offset,
                                                                    int64_t num_pages, int num_layers, int layer_idx,
                                                                    int num_heads, int page_size, int64_t batch_size) {
    PagedKV c;
    c.data = (uint8_t*)kv_data;
    c.param = (u32*)kv_param;
    c.indptr = (const int32_t*)kv_indptr;
    c.indices = (const int32_t*)kv_indices;
    c.last_page_offset = (const int32_t*)last_page_offset;
    c.num_pages = num_pages;
    c.num_layers = num_layers;
    c.layer_idx = layer_idx;
    c.num_heads = num_heads;
    c.page_size = page_size;
    c.batch_size = (int)batch_size;
    return c;
}

extern "C" int qr_kv_append_i4(void* kv_data, void* kv_param, const void* kv_indptr, const void* kv_indices,
                               const void* last_page_offset, int64_t num_pages, const void* k, const void* v,
                               const void* k_param, const void* v_param, const void* append_indptr_or_null,
                               int64_t tokens, int num_layers, int layer_idx, int num_heads, int page_size, int head_dim,
                               int64_t batch_size, void* stream) {
    if (tokens < 0) return QR_E_SHAPE;
    const int rc = check_cache(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, num_pages, num_layers, layer_idx,
                               num_heads, page_size, head_dim, batch_size);
    if (rc != QR_OK) return rc;
    if (batch_size == 0 || tokens == 0) return QR_OK;
    if (!append_indptr_or_null && tokens != batch_size) return QR_E_SHAPE;     // one new token per sequence
    if (!k || !v || !k_param || !v_param) return QR_E_NULL;
    if (((uintptr_t)k & 15) || ((uintptr_t)v & 15) || ((uintptr_t)k_param & 3) || ((uintptr_t)v_param & 3)) return QR_E_ALIGN;
    const PagedKV c = qr_internal_paged_kv(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, num_pages, num_layers,
                                           layer_idx, num_heads, page_size, batch_size);
    const int64_t pieces = tokens * num_heads * 4;
    int64_t blocks = (pieces + 255) / 256;
    blocks = blocks > 256 * 32 ? 256 * 32 : blocks;
    paged_append_i4_kernel<<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(
        c, (const u32x4*)k, (const u32x4*)v, (const u32*)k_param, (const u32*)v_param, (const int32_t*)append_indptr_or_null,
        tokens);
    return qr_launch_status();
}

namespace {
// Parts per (sequence, head): enough workgroups to fill the GPU four deep, each with at least 256
// positions, when the caller says how long the sequences can be and provides room for the partial states.
int decode_splits(int64_t batch_size, int num_heads, int64_t max_seq_len) {
    if (max_seq_len <= 0) return 1;
    const int64_t bh = batch_size * num_heads;
    int64_t s = (1024 + bh - 1) / bh, cap = max_seq_len / 256;
    s = s > cap ? cap : s;
    s = s > 64 ? 64 : s;
    return s < 1 ? 1 : (int)s;
}
}  // namespace

extern "C" size_t qr_batch_decode_workspace_bytes(int64_t batch_size, int num_heads, int64_t max_seq_len) {
    if (batch_size <= 0 || num_heads <= 0) return 0;
    const int s = decode_splits(batch_size, num_heads, max_seq_len);
    return s > 1 ? (size_t)batch_size * num_heads * s * 132 * sizeof(float) : 0;
}

extern "C" int qr_batch_decode_i4(void* o, const void* q, const void* kv_data, const void* kv_param, const void* kv_indptr,
                                  const void* kv_indices, const void* last_page_offset, int64_t num_pages, int num_layers,
                                  int layer_idx, int num_heads, int page_size, int head_dim, int64_t batch_size,
                                  int64_t max_seq_len, void* workspace, size_t workspace_bytes, void* stream) {
    const int rc = check_cache(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, num_pages, num_layers, layer_idx,
                               num_heads, page_size, head_dim, batch_size);
    if (rc != QR_OK) return rc;
    if (batch_size == 0) return QR_OK;
    if (!o || !q) return QR_E_NULL;
    if (((uintptr_t)q & 15) || ((uintptr_t)o & 1)) return QR_E_ALIGN;
    if (batch_size * num_heads > 0x3fffffff / 64) return QR_E_SHAPE;
    const PagedKV c = qr_internal_paged_kv((void*)kv_data, (void*)kv_param, kv_indptr, kv_indices, last_page_offset, num_pages,
                                           num_layers, layer_idx, num_heads, page_size, batch_size);
    int splits = decode_splits(batch_size, num_heads, max_seq_len);
    if (splits > 1 && (!workspace || ((uintptr_t)workspace & 15) ||
                       workspace_bytes < (size_t)batch_size * num_heads * splits * 132 * sizeof(float)))
        splits = 1;                                        // no room for partial states: one workgroup per (sequence, head)
    const float sm = (float)(1.4426950408889634 / __builtin_sqrt((double)head_dim));
    const unsigned grid = (unsigned)(batch_size * num_heads * splits);
    hipStream_t st = (hipStream_t)stream;
    if (page_size % 16 == 0)
        paged_decode_i4_kernel<true><<<dim3(grid), dim3(AT), 0, st>>>((const f16*)q, c, (f16*)o, sm, splits, (float*)workspace);
    else
        paged_decode_i4_kernel<false><<<dim3(grid), dim3(AT), 0, st>>>((const f16*)q, c, (f16*)o, sm, splits, (float*)workspace);
    int lrc = qr_launch_status();
    if (lrc != QR_OK || splits == 1) return lrc;
    paged_decode_merge_kernel<<<dim3((unsigned)(batch_size * num_heads)), dim3(128), 0, st>>>((const float*)workspace, splits,
                                                                                             (f16*)o);
    return qr_launch_status();
}
