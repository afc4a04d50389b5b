// The paged KV cache with fp16 pages (the reference's disable_quant mode: quarot/transformers/kv_cache.py:134-151,189-193,
// quarot/kernels/bindings.cpp:247-374): the same page tables and the same parameter tensor as the int4 cache, a vector
// of 128 halves (256 bytes) per (page, layer, K/V, head, entry) instead of 64 code bytes.  Appending is data movement;
// decode attention is the plain softmax(q . K^T / sqrt(128)) . V over the sequence's cached vectors in fp32.
// The parameters {scale, zero} are stored with the vectors (the cache class passes ones and zeros) and never read:
// the reference's kernel for this page type loads the halves as they are.
#include "qr_paged.h"

namespace {

// ---- append: one 16-byte piece per thread, sixteen threads per (token, head) vector of K and of V
__global__ __launch_bounds__(256) void paged_append_f16_kernel(PagedKV c, const u32x4* __restrict__ key,
                                                               const u32x4* __restrict__ value,
                                                               const u32* __restrict__ kparam, const u32* __restrict__ vparam,
                                                               const int32_t* __restrict__ append_indptr, int64_t tokens) {
    const int64_t pieces = tokens * c.num_heads * 16;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < pieces; i += (int64_t)gridDim.x * 256) {
        const int piece = (int)(i & 15);
        const int64_t vec = i >> 4, token = vec / c.num_heads;
        const int head = (int)(vec - token * c.num_heads);
        int64_t page;
        int entry;
        if (!paged_locate(c, append_indptr, token, page, entry)) continue;
        const int64_t ks = paged_slot(c, page, 0, head, entry), vs = paged_slot(c, page, 1, head, entry);
        ((u32x4*)c.data)[ks * 16 + piece] = key[i];
        ((u32x4*)c.data)[vs * 16 + piece] = value[i];
        if (piece == 0) {
            c.param[ks] = kparam[vec];
            c.param[vs] = vparam[vec];
        }
    }
}

template <int CTRL>
__device__ __forceinline__ float row_ror(float v) {      // DPP rotation within each row of 16 lanes
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float row_sum(float v) {      // every lane of a row ends with the row's sum
    v += row_ror<0x128>(v);
    v += row_ror<0x124>(v);
    v += row_ror<0x122>(v);
    v += row_ror<0x121>(v);
    return v;
}

// ---- decode attention: a workgroup of NW waves per (sequence, head).  A row of 16 lanes takes one cached position at
// a time, a lane 8 of its 128 dimensions (one 16-byte load each of K and V: a row reads the vector's 256 consecutive
// bytes); the NW * 4 rows walk the sequence U positions at a time, each with its own running maximum, denominator
// and accumulator (online softmax in the base-2 domain), merged through LDS at the end.  HBM-bound: 512 bytes per
// cached position and head.
constexpr int FU = 4;                 // positions per row and step: their loads are issued together

template <int NW>
__global__ __launch_bounds__(64 * NW) void paged_decode_f16_kernel(const f16* __restrict__ q, PagedKV c, f16* __restrict__ o,
                                                                    float sm_scale_log2) {
    __shared__ float st[NW * 4 * 16 * 10];                 // [row][lane of the row][m, d, acc[8]]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l16 = lane & 15, row = wave * 4 + (lane >> 4);
    const int bh = blockIdx.x, b = bh / c.num_heads, h = bh - b * c.num_heads;
    const int p0 = c.indptr[b], npages = c.indptr[b + 1] - p0;
    if (npages <= 0) {
        // a sequence without pages: the empty softmax, 0 / 0, as the int4 kernel (and the reference's) gives
        if (threadIdx.x < 128) o[(int64_t)bh * 128 + threadIdx.x] = (f16)__builtin_nanf("");
        return;
    }
    const int seq_len = (npages - 1) * c.page_size + c.last_page_offset[b];
    const u32x4 qw = ((const u32x4*)(q + (int64_t)bh * 128))[l16];
    f16x2 qp[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) qp[j] = as_f16x2(qw[j]);
    const int64_t kv_slots = (int64_t)c.num_heads * c.page_size;
    float m = -5e4f, d = 0.f, acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    constexpr int ROWS = NW * 4;
    for (int pos0 = row * FU; pos0 < seq_len; pos0 += ROWS * FU) {
        u32x4 kw[FU], vw[FU];
        bool ok[FU];
#pragma unroll
        for (int u = 0; u < FU; ++u) {
            const int pos = pos0 + u;
            const int it = pos / c.page_size, entry = pos - it * c.page_size;
            const bool in = pos < seq_len && it < npages;
            const int64_t page = c.indices[p0 + (in ? it : 0)];
            ok[u] = in && page >= 0 && page < c.num_pages;
            // a position outside the sequence reads entry 0 of page 0 and is masked: no branch around the loads
            const int64_t ks = paged_slot(c, ok[u] ? page : 0, 0, h, ok[u] ? entry : 0);
            kw[u] = __builtin_nontemporal_load((const u32x4*)c.data + ks * 16 + l16);
            vw[u] = __builtin_nontemporal_load((const u32x4*)c.data + (ks + kv_slots) * 16 + l16);
        }
        float lg[FU], mx = m;
#pragma unroll
        for (int u = 0; u < FU; ++u) {
            float a = 0.f;
#pragma unroll
            for (int j = 0; j < 4; ++j) a = __builtin_amdgcn_fdot2(qp[j], as_f16x2(kw[u][j]), a, false);
            const float x = row_sum(a) * sm_scale_log2;
            lg[u] = ok[u] ? x : -__builtin_inff();
            mx = __builtin_fmaxf(mx, lg[u]);
        }
        const float alpha = __builtin_amdgcn_exp2f(m - mx);
        m = mx;
        d *= alpha;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] *= alpha;
#pragma unroll
        for (int u = 0; u < FU; ++u) {
            const float p = __builtin_amdgcn_exp2f(lg[u] - m);
            d += p;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f16x2 pr = as_f16x2(vw[u][j]);
                // (a masked position may hold anything, a NaN included: its weight is an exact zero, so select)
                acc[2 * j] = ok[u] ? __builtin_fmaf(p, (float)pr[0], acc[2 * j]) : acc[2 * j];
                acc[2 * j + 1] = ok[u] ? __builtin_fmaf(p, (float)pr[1], acc[2 * j + 1]) : acc[2 * j + 1];
            }
        }
    }
    float* mine = st + (row * 16 + l16) * 10;
    mine[0] = m;
    mine[1] = d;
#pragma unroll
    for (int i = 0; i < 8; ++i) mine[2 + i] = acc[i];
    __syncthreads();
    if (threadIdx.x < 128) {
        const int dim = threadIdx.x, l = dim >> 3, i = dim & 7;
        float M = -5e4f;
        for (int r = 0; r < ROWS; ++r) M = __builtin_fmaxf(M, st[(r * 16 + l) * 10]);
        float D = 0.f, O = 0.f;
        for (int r = 0; r < ROWS; ++r) {
            const float* src = st + (r * 16 + l) * 10;
            const float w = __builtin_amdgcn_exp2f(src[0] - M);
            D = __builtin_fmaf(src[1], w, D);
            O = __builtin_fmaf(src[2 + i], w, O);
        }
        o[(int64_t)bh * 128 + dim] = (f16)(O / D);
    }
}

}  // namespace

extern "C" int qr_kv_append_f16(void* kv_data, void* kv_param, const void* kv_indptr, const void* kv_indices,
                                const void* last_page_offset, int64_t num_pages, const void* k, const void* v,
                                const void* k_param, const void* v_param, const void* append_indptr_or_null,
                                int64_t tokens, int num_layers, int layer_idx, int num_heads, int page_size, int head_dim,
                                int64_t batch_size, void* stream) {
    if (tokens < 0) return QR_E_SHAPE;
    const int rc = qr_internal_check_paged_cache(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, num_pages,
                                                 num_layers, layer_idx, num_heads, page_size, head_dim, batch_size);
    if (rc != QR_OK) return rc;
    if (batch_size == 0 || tokens == 0) return QR_OK;
    if (!append_indptr_or_null && tokens != batch_size) return QR_E_SHAPE;     // one new token per sequence
    if (!k || !v || !k_param || !v_param) return QR_E_NULL;
    if (((uintptr_t)k & 15) || ((uintptr_t)v & 15) || ((uintptr_t)k_param & 3) || ((uintptr_t)v_param & 3)) return QR_E_ALIGN;
    const PagedKV c = qr_internal_paged_kv(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, num_pages, num_layers,
                                           layer_idx, num_heads, page_size, batch_size);
    const int64_t pieces = tokens * num_heads * 16;
    int64_t blocks = (pieces + 255) / 256;
    blocks = blocks > 256 * 32 ? 256 * 32 : blocks;
    paged_append_f16_kernel<<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(
        c, (const u32x4*)k, (const u32x4*)v, (const u32*)k_param, (const u32*)v_param, (const int32_t*)append_indptr_or_null,
        tokens);
    return qr_launch_status();
}

extern "C" int qr_batch_decode_f16(void* o, const void* q, const void* kv_data, const void* kv_param, const void* kv_indptr,
                                   const void* kv_indices, const void* last_page_offset, int64_t num_pages, int num_layers,
                                   int layer_idx, int num_heads, int page_size, int head_dim, int64_t batch_size,
                                   void* stream) {
    const int rc = qr_internal_check_paged_cache(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, num_pages,
                                                 num_layers, layer_idx, num_heads, page_size, head_dim, batch_size);
    if (rc != QR_OK) return rc;
    if (batch_size == 0) return QR_OK;
    if (!o || !q) return QR_E_NULL;
    if (((uintptr_t)q & 15) || ((uintptr_t)o & 1)) return QR_E_ALIGN;
    if (batch_size * num_heads > 0x7fffffff) return QR_E_SHAPE;
    const PagedKV c = qr_internal_paged_kv((void*)kv_data, (void*)kv_param, kv_indptr, kv_indices, last_page_offset, num_pages,
                                           num_layers, layer_idx, num_heads, page_size, batch_size);
    const float sm = (float)(1.4426950408889634 / __builtin_sqrt((double)head_dim));
    const unsigned grid = (unsigned)(batch_size * num_heads);
    // few (sequence, head) pairs: more waves each
    if ((int64_t)grid >= 2 * (int64_t)qr_device().cus)
        paged_decode_f16_kernel<4><<<dim3(grid), dim3(256), 0, (hipStream_t)stream>>>((const f16*)q, c, (f16*)o, sm);
    else
        paged_decode_f16_kernel<16><<<dim3(grid), dim3(1024), 0, (hipStream_t)stream>>>((const f16*)q, c, (f16*)o, sm);
    return qr_launch_status();
}
