// Paged int4 KV cache: layout arithmetic shared by the append kernels, the quantise-and-append
// kernels and decode attention.
//   kv_data  uint8 [pages, layers, 2 (K, V), heads, page_size, 64]    packed int4 codes of 128-wide vectors
//   kv_param half2 [pages, layers, 2 (K, V), heads, page_size]         {scale, zero} of each vector
//   kv_indptr  int32 [batch + 1]   page-list bounds of every sequence
//   kv_indices int32 [...]         page numbers
//   last_page_offset int32 [batch] entries in use in a sequence's last page (1 .. page_size)
// (quarot/kernels/include/flashinfer/page.cuh:19-113).
#pragma once
#include "qr_common.h"

struct PagedKV {
    uint8_t* data;
    u32* param;                       // half2 {scale, zero} as one word
    const int32_t* indptr;
    const int32_t* indices;
    const int32_t* last_page_offset;
    int64_t num_pages;                // first dimension of kv_data: page numbers beyond it are never touched
    int num_layers, layer_idx, num_heads, page_size, batch_size;
};

// index of a vector in kv_param (and, times 64 bytes, in kv_data): page.cuh:75-103
__device__ __forceinline__ int64_t paged_slot(const PagedKV& c, int64_t page, int kv, int head, int entry) {
    return (((page * c.num_layers + c.layer_idx) * 2 + kv) * c.num_heads + head) * (int64_t)c.page_size + entry;
}

// tokens held by sequence b (page.cuh:131-133, decode.cuh:516)
__device__ __forceinline__ int paged_seq_len(const PagedKV& c, int b) {
    const int np = c.indptr[b + 1] - c.indptr[b];
    return np > 0 ? (np - 1) * c.page_size + c.last_page_offset[b] : 0;
}

// Where appended token `token` goes: its sequence, and through it page and entry.  append_indptr ==
// nullptr: one new token per sequence, token = sequence index, position seq_len - 1 (page.cuh:120-166);
// else the tokens of sequence b are append_indptr[b] .. append_indptr[b + 1] - 1 and fill the LAST
// positions of the sequence (page.cuh:168-219).  Returns false when the token has no valid place (a
// page list too short for the sequence, a page number outside kv_data): nothing is written then.
__device__ __forceinline__ bool paged_locate(const PagedKV& c, const int32_t* __restrict__ append_indptr, int64_t token,
                                             int64_t& page, int& entry) {
    int b, pos;
    if (append_indptr == nullptr) {
        if (token >= c.batch_size) return false;
        b = (int)token;
        pos = paged_seq_len(c, b) - 1;
    } else {
        int lo = 0, hi = c.batch_size;                 // largest b with append_indptr[b] <= token
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if ((int64_t)append_indptr[mid] <= token) lo = mid;
            else hi = mid;
        }
        b = lo;
        const int first = append_indptr[b], count = append_indptr[b + 1] - first;
        pos = paged_seq_len(c, b) - count + (int)(token - first);
    }
    if (pos < 0) return false;
    const int it = pos / c.page_size;
    if (it >= c.indptr[b + 1] - c.indptr[b]) return false;
    page = c.indices[c.indptr[b] + it];
    entry = pos - it * c.page_size;
    return page >= 0 && page < c.num_pages;
}

// destination of a quantise-and-append kernel: the cache, which tokens the vectors belong to, K or V
struct PagedDst {
    PagedKV c;
    const int32_t* append_indptr;     // nullptr: one new token per sequence
    int kv;                           // 0: K, 1: V
};

__device__ __forceinline__ u32 pack_scale_zero(f16 scale, f16 zero) {
    return (u32)f16_bits(scale) | ((u32)f16_bits(zero) << 16);
}

// attn.hip
PagedKV qr_internal_paged_kv(void* kv_data, void* kv_param, const void* kv_indptr, const void* kv_indices,
                             const void* last_page_offset, int64_t num_pages, int num_layers, int layer_idx,
                             int num_heads, int page_size, int64_t batch_size);
int qr_internal_check_paged_cache(const void* kv_data, const void* kv_param, const void* kv_indptr, const void* kv_indices,
                                  const void* last_page_offset, int64_t num_pages, int num_layers, int layer_idx,
                                  int num_heads, int page_size, int head_dim, int64_t batch_size);
