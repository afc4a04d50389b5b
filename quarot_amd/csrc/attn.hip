// Paged int4 KV cache: appending quantised vectors to their pages, and single-query (decode) attention
// over the cache with the dequantisation done in registers.
#include "qr_kvq.h"

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
constexpr int AU = 2;                 // positions per lane group and step (two steps are in flight)

__device__ __forceinline__ float quad_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // lanes ^ 1
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // lanes ^ 2
    return v;
}

// float(byte k of w): one instruction each (v_cvt_f32_ubyte0..3).  Spelled as asm because the compiler,
// seeing the nibble mask applied before, prefers a 4-bit field extract per element plus ubyte0, which
// doubles the instruction count of the inner loops.
__device__ __forceinline__ float byte_f32(u32 w, int k) {
    float f;
    switch (k) {
        case 0: asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(w)); break;
        case 1: asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(w)); break;
        case 2: asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(w)); break;
        default: asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(w)); break;
    }
    return f;
}

// Codes of one 32-bit word (eight nibbles) as four fp16 pairs, exponent bits or-ed in so that no integer
// to float conversion is needed: pair i holds codes i and i + 4 as BIAS + code, BIAS = 1024 for i = 0, 2
// (code in mantissa bits 0..3 under exponent 25) and 64 for i = 1, 3 (code in mantissa bits 4..7 under
// exponent 21).  One shift and four and-or instructions per word.
struct CodePairs {
    u32 p[4];
};
__device__ __forceinline__ CodePairs code_pairs(u32 w, u32 mask_lo, u32 bias_lo, u32 mask_hi, u32 bias_hi) {
    CodePairs r;
    const u32 w8 = w >> 8;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r.p[0]) : "v"(w), "v"(mask_lo), "v"(bias_lo));
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r.p[1]) : "v"(w), "v"(mask_hi), "v"(bias_hi));
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r.p[2]) : "v"(w8), "v"(mask_lo), "v"(bias_lo));
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r.p[3]) : "v"(w8), "v"(mask_hi), "v"(bias_hi));
    return r;
}
constexpr float kBiasEven = 1024.0f, kBiasOdd = 64.0f;

template <int CTRL>
__device__ __forceinline__ float row_rotate(float v) {   // DPP row_ror within each row of 16 lanes
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// ALIGNED: page_size is a multiple of 16, so the 16 positions of a wave step lie in one page.
// NW: waves per workgroup (4 or 16): a (sequence, head) gets NW * splits waves in all.
// APPEND: the sequence's LAST position is the token of this step, and its key and value arrive as fp16 vectors
// (knew, vnew: [batch, heads, 128]) instead of lying in the cache already: the first wave of the (sequence, head)
// quantises them itself (kv_quant_one_vector: the bits of the quantise-and-append kernel), writes codes and parameters
// to the position's page slot, and takes the position into its softmax state from its own registers; the walk over
// the cache stops one position short.  A decode step is then ONE launch instead of append + attention.
template <bool ALIGNED, int NW, bool APPEND = false>
__global__ __launch_bounds__(64 * NW, (NW == 16 ? 1 : NW == 8 ? 2 : 4)) void paged_decode_i4_kernel(
    const f16* __restrict__ q, PagedKV c, f16* __restrict__ o, float sm_scale_log2, int splits, float* __restrict__ part,
    int q_had, const u32x4* __restrict__ knew = nullptr, const u32x4* __restrict__ vnew = nullptr, int k_had = 0) {
    __shared__ float st[NW * 4 * 4 * 36];                  // [wave * 4 + row][quarter][m, d, -, -, acc[32]]
    __shared__ float st2[(NW / 2) * 128 * 3];              // second merge level: [part][dimension][m, d, o]
    __shared__ u32x4 fresh[APPEND ? 26 : 1];               // APPEND: staging [16], the new key's codes [4], the value's [4], parameters
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int slot = lane >> 2, c4 = lane & 3;
    const int bh = blockIdx.x / splits, sp = blockIdx.x - bh * splits;
    const int b = bh / c.num_heads, h = bh - b * c.num_heads;
    const int p0 = c.indptr[b], npages = c.indptr[b + 1] - p0;
    const int seq_all = npages > 0 ? (npages - 1) * c.page_size + c.last_page_offset[b] : 0;
    const int seq_len = APPEND ? seq_all - 1 : seq_all;     // positions read from the cache
    if (npages <= 0) {
        // A sequence without pages (uniform over the workgroup): nothing may be read -- its slice of kv_indices is
        // empty, and so may be the whole list and the page pool.  The result is the empty softmax state, i.e. the
        // 0 / 0 that the loop below would arrive at (and the reference's kernel does).
        if (threadIdx.x < 128) {
            if (splits == 1) {
                o[(int64_t)bh * 128 + threadIdx.x] = (f16)__builtin_nanf("");
            } else {
                float* dst = part + (int64_t)blockIdx.x * 132;
                if (threadIdx.x == 0) {
                    dst[0] = -5e4f;
                    dst[1] = 0.f;
                }
                dst[4 + threadIdx.x] = 0.f;
            }
        }
        return;
    }

    const bool appends = APPEND && sp == 0 && wave == 0;    // wave-uniform
    if (APPEND && appends) {
        const int64_t vec = (int64_t)bh * 16;
        u32 W[8];
        f16 sc, zp;
        const int pos = seq_all - 1, it = pos / c.page_size, entry = pos - it * c.page_size;
        const int64_t page = c.indices[p0 + it];
        const bool page_ok = page >= 0 && page < c.num_pages;
        const float hs = 0.08838834764831845f;                 // 1 / sqrt(128)
        const u32x4 piece[2] = {knew[vec + (lane & 15)], vnew[vec + (lane & 15)]};      // both in flight at once
#pragma unroll
        for (int kv = 0; kv < 2; ++kv) {
            if (kv == 0 && k_had) kv_quant_one_vector<true>(piece[0], fresh, hs, W, sc, zp);
            else kv_quant_one_vector<false>(piece[kv], fresh, hs, W, sc, zp);
            const u32 prm = pack_scale_zero(sc, zp);
            const int hh = lane >> 5;
            if (page_ok && (lane & 31) == 0) {
                const int64_t s = paged_slot(c, page, kv, h, entry);
                u32x4* dst = (u32x4*)c.data + s * 4 + 2 * hh;
                dst[0] = u32x4{W[0], W[1], W[2], W[3]};
                dst[1] = u32x4{W[4], W[5], W[6], W[7]};
                if (hh == 0) c.param[s] = prm;
            }
            // for the position's own turn after the walk: pieces 2 hh, 2 hh + 1 of the 64 code bytes, and the parameters
            if ((lane & 31) == 0) {
                fresh[16 + 4 * kv + 2 * hh] = u32x4{W[0], W[1], W[2], W[3]};
                fresh[16 + 4 * kv + 2 * hh + 1] = u32x4{W[4], W[5], W[6], W[7]};
                if (hh == 0) ((u32*)(fresh + 24))[kv] = page_ok ? prm : 0u;
                if (hh == 0 && kv == 0) ((u32*)(fresh + 24))[2] = page_ok ? 1u : 0u;
            }
            __builtin_amdgcn_wave_barrier();
        }
    }

    // this lane's 32 query values as fp16 pairs in the order the codes are consumed: word j of a 16-byte
    // piece holds dimensions 8 j .. 8 j + 7, and (word >> 4 i) & 0x000F000F isolates codes i and i + 4
    f16x2 qp[4][4];
    float ql = 0.f;                                        // sum of this lane's 32 values
    {
        const u32x4* qsrc = (const u32x4*)(q + (int64_t)bh * 128 + c4 * 32);
        u32x4 qw[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) qw[j] = qsrc[j];
        if (q_had) {
            // The query's Hadamard over the head dimension (matmul_had_cuda on q, kv_cache.py:30-33,113) here instead of
            // in a launch of its own: 128-point transform in fp32 -- five butterfly levels over the lane's 32 values,
            // two across the four lanes of a position group -- times 1 / sqrt(128), rounded to fp16 like that
            // function's result.
            float t[32];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const f16x2 pr = as_f16x2(qw[j][k]);
                    t[8 * j + 2 * k] = (float)pr[0];
                    t[8 * j + 2 * k + 1] = (float)pr[1];
                }
#pragma unroll
            for (int hb = 1; hb < 32; hb <<= 1)
#pragma unroll
                for (int i = 0; i < 32; ++i)
                    if ((i & hb) == 0) {
                        const float a = t[i], b = t[i + hb];
                        t[i] = a + b;
                        t[i + hb] = a - b;
                    }
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                const float o1 = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, t[i]), 0xB1, 0xF, 0xF, true));
                t[i] = (c4 & 1) ? o1 - t[i] : t[i] + o1;                // lanes ^ 1: index bit 5
                const float o2 = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, t[i]), 0x4E, 0xF, 0xF, true));
                t[i] = (c4 & 2) ? o2 - t[i] : t[i] + o2;                // lanes ^ 2: index bit 6
            }
            const float hs = 0.08838834764831845f;                       // 1 / sqrt(128)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int k = 0; k < 4; ++k) qw[j][k] = narrow_f16x2(t[8 * j + 2 * k] * hs, t[8 * j + 2 * k + 1] * hs);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const u32x4 w = qw[j];
            f16 e[8];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const f16x2 pr = as_f16x2(w[k]);
                e[2 * k] = pr[0];
                e[2 * k + 1] = pr[1];
                ql += (float)pr[0] + (float)pr[1];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) qp[j][i] = f16x2{e[i], e[i + 4]};
        }
    }
    const float qs = quad_sum(ql);                         // sum of all 128 query values
    float qbias = 0.f;                                     // sum over this lane's values of q * (bias of its code)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
            qbias = __builtin_fmaf((float)qp[j][i][0] + (float)qp[j][i][1], (i & 1) ? kBiasOdd : kBiasEven, qbias);
    u32 mask_lo = 0x000F000Fu, bias_lo = 0x64006400u, mask_hi = 0x00F000F0u, bias_hi = 0x54005400u;
    asm volatile("" : "+v"(mask_lo), "+v"(bias_lo), "+v"(mask_hi), "+v"(bias_hi));     // kept in registers for v_and_or_b32

    float m = -5e4f, d = 0.f, pz = 0.f, psum = 0.f, acc[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) acc[i] = 0.f;

    const int chunks = (seq_len + 15) >> 4;
    // a vector's place: slot = page * page_slots + head_slots + entry (K), + kv_slots (V); 64 code bytes and
    // one parameter word per slot
    const int64_t page_slots = (int64_t)c.num_layers * 2 * c.num_heads * c.page_size;
    const int64_t head_slots = ((int64_t)c.layer_idx * 2 * c.num_heads + h) * c.page_size;
    const int64_t kv_slots = (int64_t)c.num_heads * c.page_size;
    const int stride = NW * splits;                         // chunks between the steps of one wave
    // ALIGNED: chunk g lies in page g / cpp at entry 16 (g % cpp); both advance without divisions
    const int cpp = ALIGNED ? c.page_size >> 4 : 1;
    const int it_step = stride / cpp, r_step = stride - it_step * cpp;
    // APPEND: the wave that quantises the new token leaves its first two chunks (one step's worth) to its two
    // neighbours, which take one each after their own walk: its extra work would otherwise stand at the launch's end
    const int g_first = sp * NW + wave;
    int g = g_first + ((APPEND && appends) ? stride * AU : 0);
    int it_u = g / cpp, r_u = g - it_u * cpp;
    // Two sets of AU positions per lane group: the loads of the next set are issued before the current
    // one is consumed, so their latency hides under the arithmetic.  Loads are unconditional (a position
    // beyond the sequence reads entry 0 of a valid page and is masked), which keeps the loop free of
    // branches around memory operations.
    struct Step {
        u32x4 kw[AU], vw[AU];
        u32 kp[AU], vp[AU];
        bool ok[AU];
    };
    auto issue = [&](Step& t, int g0) {
        int64_t page[AU];
        int entry[AU];
        // page numbers first (scalar loads when ALIGNED), then every vector load of the step
#pragma unroll
        for (int u = 0; u < AU; ++u) {
            const int pos = (g0 + u * stride) * 16 + slot;
            int it;
            if (ALIGNED) {
                it = __builtin_amdgcn_readfirstlane(it_u);  // wave-uniform: the page number comes by a scalar load
                entry[u] = r_u * 16 + slot;
                it_u += it_step;
                r_u += r_step;
                if (r_u >= cpp) {
                    r_u -= cpp;
                    ++it_u;
                }
            } else {
                it = pos / c.page_size;
                entry[u] = pos - it * c.page_size;
            }
            t.ok[u] = pos < seq_len && it < npages;
            const int32_t* pp = c.indices + p0 + (it < npages ? it : 0);
            if (ALIGNED) {
                // a scalar load, spelled out: behind the scheduling barriers of the loop the compiler falls back
                // to a vector load plus a wait for EVERY outstanding vector load, which would drain the pipeline
                int pg;
                asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(pg) : "s"(pp) : "memory");
                page[u] = pg;
            } else {
                page[u] = *pp;
            }
        }
#pragma unroll
        for (int u = 0; u < AU; ++u) {
            const bool page_ok = page[u] >= 0 && page[u] < c.num_pages;
            t.ok[u] = t.ok[u] && page_ok;
            // the page part of the address is wave-uniform when ALIGNED (scalar base, 32-bit lane offsets)
            const int64_t kbase = (page_ok ? page[u] : 0) * page_slots + head_slots;
            const u32 e = t.ok[u] ? (u32)entry[u] : 0u;
            const uint8_t* kd = c.data + kbase * 64;
            const uint8_t* vd = c.data + (kbase + kv_slots) * 64;
            t.kw[u] = __builtin_nontemporal_load((const u32x4*)(kd + (e * 64u + (u32)c4 * 16u)));
            t.vw[u] = __builtin_nontemporal_load((const u32x4*)(vd + (e * 64u + (u32)c4 * 16u)));
            t.kp[u] = *(const u32*)((const uint8_t*)(c.param + kbase) + e * 4u);
            t.vp[u] = *(const u32*)((const uint8_t*)(c.param + kbase + kv_slots) + e * 4u);
        }
    };
    auto consume = [&](const Step& t) {
        float lg[AU], mx = m;
#pragma unroll
        for (int u = 0; u < AU; ++u) {
            // q . (bias + codes) with fp32 accumulation of exact products, minus sum(q * bias)
            float a0 = 0.f, a1 = 0.f;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const CodePairs cp = code_pairs(t.kw[u][j], mask_lo, bias_lo, mask_hi, bias_hi);
                a0 = __builtin_amdgcn_fdot2(qp[j][0], as_f16x2(cp.p[0]), a0, false);
                a1 = __builtin_amdgcn_fdot2(qp[j][1], as_f16x2(cp.p[1]), a1, false);
                a0 = __builtin_amdgcn_fdot2(qp[j][2], as_f16x2(cp.p[2]), a0, false);
                a1 = __builtin_amdgcn_fdot2(qp[j][3], as_f16x2(cp.p[3]), a1, false);
            }
            const float dot = quad_sum((a0 + a1) - qbias);
            const f16x2 prm = as_f16x2(t.kp[u]);
            const float x = (dot * (float)prm[0] - (float)prm[1] * qs) * sm_scale_log2;
            lg[u] = t.ok[u] ? x : -__builtin_inff();
            mx = __builtin_fmaxf(mx, lg[u]);
        }
        const float alpha = __builtin_amdgcn_exp2f(m - mx);
        m = mx;
        d *= alpha;
        pz *= alpha;
        psum *= alpha;
#pragma unroll
        for (int i = 0; i < 32; ++i) acc[i] *= alpha;
#pragma unroll
        for (int u = 0; u < AU; ++u) {
            const float p = __builtin_amdgcn_exp2f(lg[u] - m);
            const f16x2 prm = as_f16x2(t.vp[u]);
            const float ps = p * (float)prm[0];
            d += p;
            pz = __builtin_fmaf(p, (float)prm[1], pz);
            psum += ps;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const CodePairs cp = code_pairs(t.vw[u][j], mask_lo, bias_lo, mask_hi, bias_hi);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const f16x2 pr = as_f16x2(cp.p[i]);
                    acc[8 * j + i] = __builtin_fmaf(ps, (float)pr[0], acc[8 * j + i]);
                    acc[8 * j + i + 4] = __builtin_fmaf(ps, (float)pr[1], acc[8 * j + i + 4]);
                }
            }
        }
    };
    Step sa, sb;
    const int gs = stride * AU;
    issue(sa, g);
    for (; g < chunks; g += 2 * gs) {
        issue(sb, g + gs);
        __builtin_amdgcn_sched_barrier(0);                 // the compiler would otherwise sink the loads below the arithmetic
        consume(sa);
        __builtin_amdgcn_sched_barrier(0);
        issue(sa, g + 2 * gs);
        __builtin_amdgcn_sched_barrier(0);
        if (g + gs < chunks) consume(sb);                  // (no loads inside: the branch does not disturb the wait counts)
        __builtin_amdgcn_sched_barrier(0);
    }
    if (APPEND && sp == 0 && (wave == 1 || wave == 2)) {
        const int extra = sp * NW + (wave == 2 ? stride : 0);           // the quantising wave's first or second chunk
        if (extra < chunks) {
            it_u = extra / cpp;
            r_u = extra - it_u * cpp;
            issue(sb, extra);
            sb.ok[1] = false;                                           // (the step's second chunk is not this wave's)
            consume(sb);
        }
    }
    if (APPEND && appends) {
        // the new position, from the codes this wave made: lane group 0 takes it, the others sit the turn out
        Step tn;
        const u32* prm = (const u32*)(fresh + 24);
        const bool valid = prm[2] != 0u;
#pragma unroll
        for (int u = 0; u < AU; ++u) {
            tn.kw[u] = fresh[16 + c4];
            tn.vw[u] = fresh[20 + c4];
            tn.kp[u] = prm[0];
            tn.vp[u] = prm[1];
            tn.ok[u] = u == 0 && slot == 0 && valid;
        }
        consume(tn);
    }
    // ---- merge: first the four lane groups of each row of 16 lanes (two DPP rotations: every lane ends
    // with its row's state), then the NW * 4 row states of the workgroup through LDS
#pragma unroll
    for (int i = 0; i < 32; ++i) acc[i] -= __builtin_fmaf(psum, (i & 1) ? kBiasOdd : kBiasEven, pz);     // sum p (code scale - zero)
#pragma unroll
    for (int step = 0; step < 2; ++step) {
        const float om = step == 0 ? row_rotate<0x124>(m) : row_rotate<0x128>(m);
        const float od = step == 0 ? row_rotate<0x124>(d) : row_rotate<0x128>(d);
        const float M = __builtin_fmaxf(m, om);
        const float ws = __builtin_amdgcn_exp2f(m - M), wo = __builtin_amdgcn_exp2f(om - M);
        d = __builtin_fmaf(d, ws, od * wo);
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const float oa = step == 0 ? row_rotate<0x124>(acc[i]) : row_rotate<0x128>(acc[i]);
            acc[i] = __builtin_fmaf(acc[i], ws, oa * wo);
        }
        m = M;
    }
    if ((lane & 12) == 0) {                                           // the first lane group of every row writes
        float* mine = st + ((wave * 4 + (lane >> 4)) * 4 + c4) * 36;
        mine[0] = m;
        mine[1] = d;
#pragma unroll
        for (int i = 0; i < 32; ++i) mine[4 + i] = acc[i];
    }
    __syncthreads();
    // two levels, so that no thread walks more than eight states: thread (part, dimension) merges the row
    // states part, part + PARTS, ...; then 128 threads merge the PARTS partial results
    constexpr int PARTS = NW / 2, PER = NW * 4 / PARTS;              // 8 states per thread
    {
        const int dim = threadIdx.x & 127, prt = threadIdx.x >> 7, qd = dim >> 5, r = dim & 31;
        float sm_[PER], sd_[PER], so_[PER], M = -5e4f;
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const float* src = st + ((prt + k * PARTS) * 4 + qd) * 36;
            sm_[k] = src[0];
            sd_[k] = src[1];
            so_[k] = src[4 + r];
            M = __builtin_fmaxf(M, sm_[k]);
        }
        float D = 0.f, O = 0.f;
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const float w = __builtin_amdgcn_exp2f(sm_[k] - M);
            D = __builtin_fmaf(sd_[k], w, D);
            O = __builtin_fmaf(so_[k], w, O);
        }
        float* dst = st2 + (prt * 128 + dim) * 3;
        dst[0] = M;
        dst[1] = D;
        dst[2] = O;
    }
    __syncthreads();
    if (threadIdx.x < 128) {
        const int dim = threadIdx.x;
        float M = -5e4f;
#pragma unroll
        for (int k = 0; k < PARTS; ++k) M = __builtin_fmaxf(M, st2[(k * 128 + dim) * 3]);
        float D = 0.f, O = 0.f;
#pragma unroll
        for (int k = 0; k < PARTS; ++k) {
            const float* src = st2 + (k * 128 + dim) * 3;
            const float w = __builtin_amdgcn_exp2f(src[0] - M);
            D = __builtin_fmaf(src[1], w, D);
            O = __builtin_fmaf(src[2], w, O);
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
    if (num_pages == 0) return QR_E_SHAPE;                 // sequences but no page pool: nothing a page number could name
    if (!kv_data || !kv_param || !kv_indptr || !kv_indices || !last_page_offset) return QR_E_NULL;
    if (((uintptr_t)kv_data & 15) || ((uintptr_t)kv_param & 3)) return QR_E_ALIGN;
    return QR_OK;
}

}  // namespace

// paged_f16.hip: the same argument checks for the cache with fp16 pages
__attribute__((visibility("hidden"))) int qr_internal_check_paged_cache(const void* kv_data, const void* kv_param,
                                                                        const void* kv_indptr, const void* kv_indices,
                                                                        const void* last_page_offset, int64_t num_pages,
                                                                        int num_layers, int layer_idx, int num_heads,
                                                                        int page_size, int head_dim, int64_t batch_size) {
    return check_cache(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, num_pages, num_layers, layer_idx, num_heads,
                       page_size, head_dim, batch_size);
}

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
// Waves per (sequence, head): enough to fill the GPU's wave slots (16 per CU), each with at least four steps of 16
// positions when the caller says how long the sequences can be.  Up to 16 of them form one workgroup;
// beyond that the sequence is split over several workgroups, which needs room for their partial states.
struct DecodePlan {
    int nw, splits;
};
DecodePlan decode_plan(int64_t batch_size, int num_heads, int64_t max_seq_len) {
    const int64_t bh = batch_size * num_heads, cus = qr_device().cus;
    if (max_seq_len <= 0) return DecodePlan{bh >= 4 * cus ? 4 : bh >= cus ? 8 : 16, 1};
    const int64_t chunks = (max_seq_len + 15) / 16;
    int64_t wp = (16 * cus + bh - 1) / bh, cap = chunks / 4;
    wp = wp > cap ? cap : wp;
    if (wp <= 4) return DecodePlan{4, 1};
    if (wp <= 16) return DecodePlan{8, 1};                  // (measured a few percent ahead of 16 waves at 256 (sequence, head) pairs)
    int64_t s = (wp + 15) / 16;
    return DecodePlan{16, (int)(s > 16 ? 16 : s)};
}
}  // namespace

extern "C" size_t qr_batch_decode_workspace_bytes(int64_t batch_size, int num_heads, int64_t max_seq_len) {
    if (batch_size <= 0 || num_heads <= 0) return 0;
    const int s = decode_plan(batch_size, num_heads, max_seq_len).splits;
    return s > 1 ? (size_t)batch_size * num_heads * s * 132 * sizeof(float) : 0;
}

namespace {
int batch_decode(void* o, const void* q, const void* kv_data, const void* kv_param, const void* kv_indptr,
                 const void* kv_indices, const void* last_page_offset, int64_t num_pages, int num_layers, int layer_idx,
                 int num_heads, int page_size, int head_dim, int64_t batch_size, int64_t max_seq_len, void* workspace,
                 size_t workspace_bytes, void* stream, int q_had, const void* knew = nullptr, const void* vnew = nullptr,
                 int k_had = 0) {
    const int rc = check_cache(kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, num_pages, num_layers, layer_idx,
                               num_heads, page_size, head_dim, batch_size);
    if (rc != QR_OK) return rc;
    if (batch_size == 0) return QR_OK;
    if (!o || !q) return QR_E_NULL;
    if (((uintptr_t)q & 15) || ((uintptr_t)o & 1)) return QR_E_ALIGN;
    if (batch_size * num_heads > 0x3fffffff / 64) return QR_E_SHAPE;
    const PagedKV c = qr_internal_paged_kv((void*)kv_data, (void*)kv_param, kv_indptr, kv_indices, last_page_offset, num_pages,
                                           num_layers, layer_idx, num_heads, page_size, batch_size);
    DecodePlan plan = decode_plan(batch_size, num_heads, max_seq_len);
    int splits = plan.splits;
    if (splits > 1 && (!workspace || ((uintptr_t)workspace & 15) ||
                       workspace_bytes < (size_t)batch_size * num_heads * splits * 132 * sizeof(float)))
        splits = 1;                                        // no room for partial states: one workgroup per (sequence, head)
    const float sm = (float)(1.4426950408889634 / __builtin_sqrt((double)head_dim));
    const unsigned grid = (unsigned)(batch_size * num_heads * splits);
    hipStream_t st = (hipStream_t)stream;
#define QR_DECODE(AL, NWV)                                                                                              \
    do {                                                                                                                \
        if (knew)                                                                                                       \
            paged_decode_i4_kernel<AL, NWV, true><<<dim3(grid), dim3(64 * NWV), 0, st>>>(                               \
                (const f16*)q, c, (f16*)o, sm, splits, (float*)workspace, q_had, (const u32x4*)knew, (const u32x4*)vnew, k_had); \
        else                                                                                                            \
            paged_decode_i4_kernel<AL, NWV><<<dim3(grid), dim3(64 * NWV), 0, st>>>((const f16*)q, c, (f16*)o, sm, splits, \
                                                                                  (float*)workspace, q_had);           \
    } while (0)
    if (page_size % 16 == 0) {
        if (plan.nw == 16) QR_DECODE(true, 16);
        else if (plan.nw == 8) QR_DECODE(true, 8);
        else QR_DECODE(true, 4);
    } else {
        if (plan.nw == 16) QR_DECODE(false, 16);
        else if (plan.nw == 8) QR_DECODE(false, 8);
        else QR_DECODE(false, 4);
    }
#undef QR_DECODE
    int lrc = qr_launch_status();
    if (lrc != QR_OK || splits == 1) return lrc;
    paged_decode_merge_kernel<<<dim3((unsigned)(batch_size * num_heads)), dim3(128), 0, st>>>((const float*)workspace, splits,
                                                                                             (f16*)o);
    return qr_launch_status();
}
}  // namespace

extern "C" int qr_batch_decode_i4(void* o, const void* q, const void* kv_data, const void* kv_param, const void* kv_indptr,
                                  const void* kv_indices, const void* last_page_offset, int64_t num_pages, int num_layers,
                                  int layer_idx, int num_heads, int page_size, int head_dim, int64_t batch_size,
                                  int64_t max_seq_len, void* workspace, size_t workspace_bytes, void* stream) {
    return batch_decode(o, q, kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, num_pages, num_layers, layer_idx,
                        num_heads, page_size, head_dim, batch_size, max_seq_len, workspace, workspace_bytes, stream, 0);
}

extern "C" int qr_batch_decode_qhad_i4(void* o, const void* q, const void* kv_data, const void* kv_param, const void* kv_indptr,
                                       const void* kv_indices, const void* last_page_offset, int64_t num_pages, int num_layers,
                                       int layer_idx, int num_heads, int page_size, int head_dim, int64_t batch_size,
                                       int64_t max_seq_len, void* workspace, size_t workspace_bytes, void* stream) {
    return batch_decode(o, q, kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, num_pages, num_layers, layer_idx,
                        num_heads, page_size, head_dim, batch_size, max_seq_len, workspace, workspace_bytes, stream, 1);
}

// One decode step in one launch: the new token's key and value (fp16 [batch, heads, 128], one token per sequence, its
// place the LAST position of the sequence as the page tables already count it) are quantised inside the attention kernel
// -- the codes and parameters of qr_kv_quant_append_f16_i4, written to the same page slots -- and attended to along with
// the cached positions: qr_kv_quant_append_f16_i4 followed by qr_batch_decode_i4 / _qhad_i4
// (MultiLayerPagedKVCache4Bit.update and the callable it returns, quarot/transformers/kv_cache.py:104-129,224-251).
extern "C" int qr_kv_quant_append_batch_decode_f16_i4(void* o, const void* q, int q_had_mode, const void* k, const void* v,
                                                      int k_had_mode, void* kv_data, void* kv_param, const void* kv_indptr,
                                                      const void* kv_indices, const void* last_page_offset, int64_t num_pages,
                                                      int num_layers, int layer_idx, int num_heads, int page_size, int head_dim,
                                                      int64_t batch_size, int64_t max_seq_len, void* workspace,
                                                      size_t workspace_bytes, void* stream) {
    if ((q_had_mode != 0 && q_had_mode != 1) || (k_had_mode != 0 && k_had_mode != 1)) return QR_E_DTYPE;
    if (batch_size > 0 && (!k || !v)) return QR_E_NULL;
    if (((uintptr_t)k & 15) || ((uintptr_t)v & 15)) return QR_E_ALIGN;
    return batch_decode(o, q, kv_data, kv_param, kv_indptr, kv_indices, last_page_offset, num_pages, num_layers, layer_idx,
                        num_heads, page_size, head_dim, batch_size, max_seq_len, workspace, workspace_bytes, stream, q_had_mode,
                        k, v, k_had_mode);
}
