// A decode step's whole linear layer in ONE launch: one or two tokens through OnlineHadamard -> Quantizer -> Linear4bit
// (bm_gemv_kernel) or through Quantizer -> Linear4bit (quant_gemv_kernel, quant_gemv_mt_kernel)
// (quarot/nn/hadamard.py:17-23, quarot/nn/quantization.py:10, quarot/nn/linear.py:42-56 on one or two rows).
// A decode step at one token is latency: the transform of a 57 KB row keeps one CU busy for a few microseconds
// while the others wait, and only then does the weight stream start.  Here EVERY workgroup transforms and
// quantises the row itself (the row comes out of L2; the arithmetic is that of hadamard_bm_kernel's register
// path, operation for operation, so codes and scale are the same bits) with its first weight segments already
// requested, keeps the codes in LDS and goes on as the dot-product kernel does (v_dot8_i32_i4 over 1 KB segments of
// the weight rows, gemv_i4_kernel's arithmetic and epilogue).  Nothing is exchanged between workgroups.
#include "qr_common.h"

namespace {

// Weight segments a wave requests at each point of the front (after the first barrier, after its part of the power-of-two
// factor, after the table stage, after the codes); their sum is the depth of the ring.  A CU's memory pipeline takes
// requests only as fast as it drains (the stream runs at the HBM rate from the first request on), so a wave that asks for
// its whole ring at once stands at the load instructions for microseconds while the row's transform waits; spread out,
// the front finishes earlier and the ring is still full when the dot products start.  Alternating runs, one token,
// 8192 x 28672: {5,0,0,0} 22.0 us, {3,1,1,0} 21.4, {2,1,1,1} 20.9, {2,1,2,0} 20.7, {1,2,2,0} 20.6, {0,3,2,0} 21.3; deeper
// rings are slower ({1,2,2,1} 21.0, {1,2,2,2} 22.2: more requests queue ahead of what the front waits for).
constexpr int F0 = 1, F1 = 2, F2 = 2, F3 = 0, RING = F0 + F1 + F2 + F3;

// The dot products that all kernels of this file end in: a wave takes `ng` consecutive pairs of weight rows as one
// flattened sequence of 1 KB segments (lane l: bytes [16 l, 16 l + 16) of each row's segment), a ring of segments in
// flight, against the MB tokens' codes in LDS (v_dot8_i32_i4: eight signed 4-bit products per lane and instruction).
// The kernels place the first requests between the phases of their fronts (fetch) and consume the ring once the codes
// are in LDS (run).  A row's last segment may be short: the lanes past its end re-read the row's start against zero
// codes.  The 64 partial sums of each (row, token) pair are added across the wave by a halving exchange, and the lane
// that ends up with a pair's sum applies Linear4bit's epilogue: y = fp16(fp16(sA sW) fp16(sum)) (+ bias).
template <int MB>
struct RowPairStream {
    static constexpr int R = 2, NS = R * MB, LV = NS == 2 ? 1 : NS == 4 ? 2 : NS == 8 ? 3 : 4;
    struct Seg {
        u32x4 w[R];
        f16 sb, bi;                              // scale and bias of the output this lane will store
    };
    const uint8_t* B;
    const f16* sB;
    const f16* bias;
    int N, Kb, nseg, g0, gcount, lane, my_m, my_r, fg, fs;

    __device__ __forceinline__ void init(const uint8_t* B_, const f16* sB_, const f16* bias_, int N_, int Kb_, int ng, int wave,
                                         int lane_) {
        B = B_, sB = sB_, bias = bias_, N = N_, Kb = Kb_, lane = lane_;
        nseg = (Kb + 1023) >> 10;
        const int groups = (N + R - 1) / R;
        g0 = ((int)blockIdx.x * 16 + wave) * ng;
        gcount = g0 >= groups ? 0 : (groups - g0 < ng ? groups - g0 : ng);
        const int vidx = lane >> (6 - LV);       // which of a pair's NS sums this lane stores at the end of the exchange
        my_m = vidx / R, my_r = vidx % R;
        fg = fs = 0;
    }
    __device__ __forceinline__ void fetch(Seg& s) {
        const int off = (fs * 1024 + lane * 16 < Kb) ? fs * 1024 + lane * 16 : 0;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int nr = (g0 + fg) * R + r;
            nr = nr < N ? nr : N - 1;
            s.w[r] = __builtin_nontemporal_load((const u32x4*)(B + (int64_t)nr * Kb + off));
        }
        // every segment carries its pair's scale along: loading it at the pair's end would make the wave wait for
        // everything it has in flight
        int col = (g0 + fg) * R + my_r;
        col = col < N ? col : N - 1;
        s.sb = sB[col];
        s.bi = (bias ? bias : sB)[col];          // (no bias: a harmless second read of the scale)
        if (fs + 1 < nseg) ++fs;
        else if (fg + 1 < gcount) { ++fg; fs = 0; }
    }
    // xq: the tokens' codes in LDS, nseg * 1024 bytes per token (zero-filled past the row's end); my_sa: the scale of
    // the token whose sums this lane stores; M: tokens that exist
    template <int RD>
    __device__ __forceinline__ void run(Seg (&ring)[RD], const void* xq, f16 my_sa, int M, f16* __restrict__ Y) {
        if (gcount == 0) return;
        const u32x4* xs = (const u32x4*)xq + lane;
        const int total = gcount * nseg;
        int acc[NS];
#pragma unroll
        for (int i = 0; i < NS; ++i) acc[i] = 0;
        int cg = 0, cs = 0;
        auto consume = [&](const Seg& sg) {
#pragma unroll
            for (int mt = 0; mt < MB; ++mt) {
                const u32x4 xv = xs[(mt * nseg + cs) * 64];
#pragma unroll
                for (int d = 0; d < 4; ++d)
#pragma unroll
                    for (int r = 0; r < R; ++r)
                        acc[mt * R + r] = __builtin_amdgcn_sdot8((int)sg.w[r][d], (int)xv[d], acc[mt * R + r], false);
            }
            if (++cs < nseg) return;
            // end of a pair of rows: each step of the exchange gives away half of the values a lane still holds
            int vals[NS];
#pragma unroll
            for (int i = 0; i < NS; ++i) vals[i] = acc[i];
            int off = 32;
#pragma unroll
            for (int cur = NS; cur > 1; cur >>= 1) {
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
                    f16 yo = (f16)(my_sa * sg.sb) * (f16)(float)sum;
                    if (bias) yo = yo + sg.bi;
                    Y[(int64_t)my_m * N + col] = yo;
                }
            }
#pragma unroll
            for (int i = 0; i < NS; ++i) acc[i] = 0;
            cs = 0;
            ++cg;
        };
        int it = 0;
        for (; it + RD <= total; it += RD) {                    // whole turns of the ring: no branch around the loads
#pragma unroll
            for (int r = 0; r < RD; ++r) {
                consume(ring[r]);
                fetch(ring[r]);
            }
        }
#pragma unroll
        for (int r = 0; r < RD - 1; ++r)
            if (it + r < total) consume(ring[r]);
    }
};

// n = 1024 K (K = order of the table, a multiple of 4, at most 32), MB = 1 or 2 tokens (the rows are transformed one
// after the other, the second row's pieces requested when the first's are consumed).  A wave takes `ng` consecutive pairs of weight
// rows as one flattened sequence of 1 KB segments, RD segments in flight (first requested while the row is transformed).
template <int MB>
__global__ __launch_bounds__(1024) void bm_gemv_kernel(const f16* __restrict__ x, int K, const f16* __restrict__ hadK,
                                                       float scale, float clip, const uint8_t* __restrict__ B,
                                                       const f16* __restrict__ sB, const f16* __restrict__ bias, int N,
                                                       int ng, f16* __restrict__ Y) {
    constexpr int RD = RING;
    constexpr int NW = 16, M_ = 1024, CT = M_ / 16, RT = 2, TS = 17;
    extern __shared__ f32x4 smem_raw[];
    __shared__ u32 red[NW];
    __shared__ f16 sc[MB];
    u32x4* Tl = (u32x4*)smem_raw;                // [4][CT][TS]
    u32x2* xq = (u32x2*)(Tl + 4 * CT * TS);      // codes of the transformed rows, K * 512 bytes each
    u32x4* hk = (u32x4*)(xq + MB * K * 64);      // the table, K * K halves
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int Kb = K * (M_ / 2);

    // the table as it lies in memory, one piece per thread (eight copies over the workgroup, no branch: it is the
    // oldest request, so waiting for it leaves everything else in flight); fragments are read from LDS later
    const u32x4 hpiece = *((const u32x4*)hadK + ((tid & 127) < K * K / 8 ? (tid & 127) : 0));

    // ---- the row (requested first: it is what the workgroup waits for) --------------------------------------
    const bool works = wave * 2 < K;
    const int pair = works ? wave : 0;
    u32x4 raw[4];
    auto request = [&](int row) {
#pragma unroll
        for (int sg = 0; sg < 2; ++sg)
#pragma unroll
            for (int bt = 0; bt < 2; ++bt)
                raw[sg * 2 + bt] = *((const u32x4*)x + (int64_t)row * (K * 128) + (pair * 2 + sg) * 128 + bt * 64 + l16 * 4 + g);
    };
    request(0);
    // (Lanes take the pieces in the order the matrix instruction wants them, neighbouring lanes 64 bytes apart; loading
    // them as they lie and swapping lanes through LDS was measured 0.1 us slower.)

    // ---- the weight stream of this wave ----------------------------------------------------------------------
    RowPairStream<MB> ws;
    ws.init(B, sB, bias, N, Kb, ng, wave, lane);
    auto fetch = [&](typename RowPairStream<MB>::Seg& sg) { ws.fetch(sg); };
    using Seg = typename RowPairStream<MB>::Seg;

    // ---- fragments: Sylvester factors of both stages -----------------------------------------------------------
    f16x8 ha[2], hb[2];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
#pragma unroll
        for (int cth = 0; cth < 2; ++cth) ha[cth][t] = (__builtin_popcount((g * 8 + t) & (cth * 16 + l16)) & 1) ? (f16)-1.0f : (f16)1.0f;
        const int b = 16 * (t >> 2) + 4 * g + (t & 3);
#pragma unroll
        for (int bt = 0; bt < 2; ++bt) hb[bt][t] = (__builtin_popcount(b & (bt * 16 + l16)) & 1) ? (f16)-1.0f : (f16)1.0f;
    }
    for (int i = tid; i < 4 * CT * TS; i += 1024) Tl[i] = u32x4{0, 0, 0, 0};
    __syncthreads();
    // every wave's requests for the row now stand before every weight request in the CU's memory queue
    Seg ring[RD];
    static_assert(F0 == 1 && F1 == 2 && F2 == 2 && F3 == 0 && RD == 5, "the request points below spell this schedule out");
    fetch(ring[0]);
    if (tid < 128) hk[tid] = hpiece;        // (read after the next barrier)
    f16 sh_one = (f16)0;                         // MB == 1: the row's scale stays in a register

#pragma unroll
    for (int row = 0; row < MB; ++row) {
    // ---- H_1024 of the wave's two segments as H_32 (x) H_32, into the fragment order of the table stage ------
    if (works) {
#pragma unroll
        for (int cth = 0; cth < 2; ++cth) {
            u32 o[2][2][2];
#pragma unroll
            for (int sg = 0; sg < 2; ++sg) {
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
            u32* const dst = (u32*)(Tl + ((pair >> 2) * CT + cth) * TS + l16) + (pair & 3);
#pragma unroll
            for (int bt = 0; bt < 2; ++bt)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const u32 sel = (e & 1) ? 0x07060302u : 0x05040100u;
                    dst[(2 * (16 * bt + 4 * g + e)) * TS * 4] = __builtin_amdgcn_perm(o[1][bt][e >> 1], o[0][bt][e >> 1], sel);
                }
        }
    }
    if (row + 1 < MB) request(row + 1);          // (the row's pieces are consumed: the next row's take their registers)
    // (two tokens: one segment at each of the four points of the two fronts instead of two at each of the two)
    if constexpr (MB == 1) {
        fetch(ring[1]);
        fetch(ring[2]);
    } else {
        fetch(ring[1 + 2 * row]);
    }
    __syncthreads();

    // ---- the table stage, the row's maximum, the codes (into LDS) -------------------------------------------
    // the table's fragments (second operand of the table stage): column k' = 16 rt + l16, contraction k = 8 g + j
    f16x8 hf[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        u32x4 v;
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
            const int hr = rt * 16 + l16, hc = g * 8 + hh * 4;
            const bool in = hr < K && hc < K;
            const u32x2 w = *((const u32x2*)hk + (in ? (hr * K + hc) >> 2 : 0));
            v[hh * 2] = in ? w[0] : 0u;
            v[hh * 2 + 1] = in ? w[1] : 0u;
        }
        hf[rt] = __builtin_bit_cast(f16x8, v);
    }
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
            const f32x4 acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(th4[c], hf[rt], f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
            if (c == 0 && rt == 0) probe = acc[0];
            yv[rt][c][0] = cvt_f16x2(acc[0], acc[1]);
            yv[rt][c][1] = cvt_f16x2(acc[2], acc[3]);
            mxf = __builtin_fmaxf(__builtin_fmaxf(mxf, __builtin_fabsf(acc[0])), __builtin_fabsf(acc[1]));
            mxf = __builtin_fmaxf(__builtin_fmaxf(mxf, __builtin_fabsf(acc[2])), __builtin_fabsf(acc[3]));
        }
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
    if (lane == 0) red[wave] = mx;
    if constexpr (MB == 1) {
        fetch(ring[3]);
        fetch(ring[4]);
    } else {
        fetch(ring[2 + 2 * row]);
    }
    __syncthreads();
#pragma unroll
    for (int w = 0; w < NW; ++w) mx = mx > red[w] ? mx : red[w];
    const f16 sh = quantizer_scale(f16_from_bits((unsigned short)mx), clip);
    const float sp = (float)sh;
    if (MB > 1 && tid == 0) sc[row] = sh;
    sh_one = sh;
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
        const bool fs_ok = scale_fast_ok(sp);
        const float rs = fs_ok ? 1.0f / sp : 0.0f;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            c01[rt] = sym_codes8(u32x4{yv[rt][0][0], yv[rt][0][1], yv[rt][1][0], yv[rt][1][1]}, sp, rs, fs_ok);
            c23[rt] = sym_codes8(u32x4{yv[rt][2][0], yv[rt][2][1], yv[rt][3][0], yv[rt][3][1]}, sp, rs, fs_ok);
        }
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const auto s1 = __builtin_amdgcn_permlane32_swap(c01[rt], c23[rt], false, false);
        const u32 ev = __builtin_amdgcn_perm(s1[1], s1[0], 0x05040100u);
        const u32 od = __builtin_amdgcn_perm(s1[1], s1[0], 0x07060302u);
        const auto s2 = __builtin_amdgcn_permlane16_swap(ev, od, false, false);
        const u32x2 outv = {__builtin_amdgcn_perm(s2[1], s2[0], 0x05040100u), __builtin_amdgcn_perm(s2[1], s2[0], 0x07060302u)};
        if (dval[rt]) xq[row * (K * 64) + (rt * 16 + l16) * (M_ / 16) + wave * 4 + g] = outv;
    }
    // (the next row's first stage writes the table stage's operand only after the barrier above, behind every wave's
    // reads of it; the maxima are next written behind the next barrier)
    }
    __syncthreads();

    // ---- the dot products -----------------------------------------------------------------------------------
    ws.run(ring, xq, MB == 1 ? sh_one : sc[ws.my_m], MB, Y);
}

// ---- Quantizer -> Linear4bit for one token (no Hadamard in front) ---------------------------------------------
// The same construction with quant_rows_kernel's arithmetic as the front: every workgroup takes the row's largest
// magnitude, the scale and the codes itself (element-wise work on the row out of L2: the scale and every code are the
// bits of the separate quantiser), keeps the codes in LDS and takes its dot products.  NV: 16-byte pieces of the row
// per thread (rows of up to 8192 NV halves).  The last segment of a row may be short: its missing codes are zeros in
// LDS and the lanes past the row's end re-read the row's start.
template <int NV>
__global__ __launch_bounds__(1024) void quant_gemv_kernel(const u32x4* __restrict__ x, int cols8, float clip,
                                                          const uint8_t* __restrict__ B, const f16* __restrict__ sB,
                                                          const f16* __restrict__ bias, int N, int ng, f16* __restrict__ Y) {
    constexpr int NW = 16, RD = 5;
    extern __shared__ f32x4 smem_raw[];
    __shared__ u32 red[NW];
    u32* xq = (u32*)smem_raw;                    // codes of the row, a word per piece, zero-filled to whole segments
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int Kb = cols8 * 4, nseg = (Kb + 1023) >> 10;
    u32x4 v[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = tid + i * 1024;
        v[i] = x[c < cols8 ? c : 0];
    }
    RowPairStream<1> ws;
    ws.init(B, sB, bias, N, Kb, ng, wave, lane);
    auto fetch = [&](RowPairStream<1>::Seg& sg) { ws.fetch(sg); };
    using Seg = RowPairStream<1>::Seg;
    Seg ring[RD];
    fetch(ring[0]);
    fetch(ring[1]);
    u32 m = 0;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const u32 mi = tid + i * 1024 < cols8 ? absmax_bits8(v[i]) : 0u;
        m = m > mi ? m : mi;
    }
    m = wave_max_u32(m);
    if (lane == 0) red[wave] = m;
    fetch(ring[2]);
    fetch(ring[3]);
    __syncthreads();
#pragma unroll
    for (int w = 0; w < NW; ++w) m = m > red[w] ? m : red[w];
    const f16 sh = quantizer_scale(f16_from_bits((unsigned short)m), clip);
    const float s = (float)sh;
    auto codes_of_row = [&](auto form) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = tid + i * 1024;
            if (c < nseg * 256) xq[c] = c < cols8 ? form(v[i]) : 0u;
        }
    };
    if (fast_quant_ok(m, s)) {
        const FastRecip fr = make_fast_recip(s);
        if (clamp_cannot_act(clip, s)) codes_of_row([&](u32x4 h) { return sym_codes8_fast<false>(h, fr); });
        else codes_of_row([&](u32x4 h) { return sym_codes8_fast<true>(h, fr); });
    } else {
        const bool fast = scale_fast_ok(s);
        const float rs = fast ? 1.0f / s : 0.0f;
        codes_of_row([&](u32x4 h) { return sym_codes8(h, s, rs, fast); });
    }
    fetch(ring[4]);
    __syncthreads();
    ws.run(ring, xq, sh, 1, Y);
}

// ---- Quantizer -> Linear4bit for two tokens -------------------------------------------------------------------------
// MB tokens: 16 / MB waves quantise each row (a lane keeps up to eight 16-byte pieces of its row in registers: rows of up
// to 65536 / MB halves) and every wave then takes its pairs of weight rows against all tokens.  Built for MB = 2 only:
// with four and eight tokens every workgroup pulls 64 / 128 KB of rows through its CU's memory path before its weight
// stream can be consumed, and the launch (70B gate_up: 43.7 / 41.8 us) is no faster than the quantiser kernel followed
// by the shared-token decode kernel (43.5 / 43.7 us); with two tokens it is 38.2 against 43.4 us.  (Eight tokens once more
// on the present form of this kernel, no spills, ring depths 3 to 6, alternating runs on one GPU: 44.1 .. 45.4 us against
// 44.0 for the two launches.)
template <int MB>
__global__ __launch_bounds__(1024) void quant_gemv_mt_kernel(const u32x4* __restrict__ x, int M, int cols8, float clip,
                                                             const uint8_t* __restrict__ B, const f16* __restrict__ sB,
                                                             const f16* __restrict__ bias, int N, int ng, f16* __restrict__ Y) {
    constexpr int NW = 16, RD = 5, WPR = NW / MB, NV = 8;
    extern __shared__ f32x4 smem_raw[];
    __shared__ u32 red[NW];
    __shared__ f16 sc[MB];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int Kb = cols8 * 4, nseg = (Kb + 1023) >> 10;
    u32* xq = (u32*)smem_raw;                    // [MB][nseg * 256] words: codes of the rows, zero-filled to whole segments
    const int row = wave / WPR, part = wave % WPR;
    const u32x4* xr = x + (int64_t)(row < M ? row : M - 1) * cols8;
    u32x4 v[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = (i * WPR + part) * 64 + lane;
        v[i] = xr[c < cols8 ? c : 0];
    }
    RowPairStream<MB> ws;
    ws.init(B, sB, bias, N, Kb, ng, wave, lane);
    auto fetch = [&](typename RowPairStream<MB>::Seg& sg) { ws.fetch(sg); };
    using Seg = typename RowPairStream<MB>::Seg;
    Seg ring[RD];
    fetch(ring[0]);
    fetch(ring[1]);
    u32 m = 0;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const u32 mi = (i * WPR + part) * 64 + lane < cols8 ? absmax_bits8(v[i]) : 0u;
        m = m > mi ? m : mi;
    }
    m = wave_max_u32(m);
    if (lane == 0) red[wave] = m;
    fetch(ring[2]);
    fetch(ring[3]);
    __syncthreads();
#pragma unroll
    for (int w = 0; w < WPR; ++w) m = m > red[row * WPR + w] ? m : red[row * WPR + w];
    const f16 sh = quantizer_scale(f16_from_bits((unsigned short)m), clip);
    const float s = (float)sh;
    if (part == 0 && lane == 0) sc[row] = sh;
    u32* xrow = xq + row * (nseg * 256);
    auto codes_of_row = [&](auto form) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = (i * WPR + part) * 64 + lane;
            if (c < nseg * 256) xrow[c] = c < cols8 ? form(v[i]) : 0u;
        }
    };
    if (fast_quant_ok(m, s)) {                   // (uniform over the waves of a row)
        const FastRecip fr = make_fast_recip(s);
        if (clamp_cannot_act(clip, s)) codes_of_row([&](u32x4 h) { return sym_codes8_fast<false>(h, fr); });
        else codes_of_row([&](u32x4 h) { return sym_codes8_fast<true>(h, fr); });
    } else {
        const bool fast = scale_fast_ok(s);
        const float rs = fast ? 1.0f / s : 0.0f;
        codes_of_row([&](u32x4 h) { return sym_codes8(h, s, rs, fast); });
    }
    fetch(ring[4]);
    __syncthreads();
    ws.run(ring, xq, sc[ws.my_m < M ? ws.my_m : M - 1], M, Y);
}

}  // namespace

// api.hip: the whole layer for one or two tokens whose rows are 1024 K halves behind a table of order K <= 32.
// QR_E_UNSUPPORTED (nothing launched) for every other shape: the caller then chains the two kernels.
__attribute__((visibility("hidden"))) int qr_internal_token_hadamard_linear(const void* x, int64_t M, int n, int K,
                                                                            const void* hadK, float scale, float clip,
                                                                            const void* W, const void* sW, const void* bias,
                                                                            int64_t N, void* y, hipStream_t st) {
    if (M < 1 || M > 2 || K < 4 || K > 32 || (K & 3) != 0 || n != 1024 * K || N <= 0 || N > (1 << 30)) return QR_E_UNSUPPORTED;
    if (((uintptr_t)x & 15) || ((uintptr_t)W & 15) || ((uintptr_t)hadK & 15)) return QR_E_UNSUPPORTED;
    const int cus = qr_device().cus;
    const int64_t groups = (N + 1) / 2;
    const int ng = (int)((groups + (int64_t)cus * 16 - 1) / ((int64_t)cus * 16));
    const unsigned grid = (unsigned)(((groups + ng - 1) / ng + 15) / 16);
    const size_t lds = (size_t)4 * 64 * 17 * 16 + (size_t)M * K * 512 + 128 * 16;
#define QR_BG(MBV)                                                                                                        \
    do {                                                                                                                  \
        auto kern = bm_gemv_kernel<MBV>;                                                                                  \
        hipError_t e = qr_allow_dynamic_lds((const void*)kern, lds);                                                      \
        if (e != hipSuccess) return (int)e;                                                                               \
        kern<<<dim3(grid), dim3(1024), lds, st>>>((const f16*)x, K, (const f16*)hadK, scale, clip, (const uint8_t*)W,     \
                                                  (const f16*)sW, (const f16*)bias, (int)N, ng, (f16*)y);                 \
    } while (0)
    if (M == 1) QR_BG(1);
    else QR_BG(2);
#undef QR_BG
    return qr_launch_status();
}

// api.hip: Quantizer + Linear4bit for one or two tokens in one launch (rows of up to 32768 halves, a multiple of 64).
__attribute__((visibility("hidden"))) int qr_internal_token_quant_linear(const void* x, int64_t M, int64_t K, float clip,
                                                                         const void* W, const void* sW, const void* bias,
                                                                         int64_t N, void* y, hipStream_t st) {
    if (M < 1 || M > 2 || K <= 0 || K % 64 != 0 || K > 32768 || N <= 0 || N > (1 << 30)) return QR_E_UNSUPPORTED;
    if (((uintptr_t)x & 15) || ((uintptr_t)W & 15)) return QR_E_UNSUPPORTED;
    const int cols8 = (int)(K / 8), nseg = (cols8 * 4 + 1023) / 1024;
    const int cus = qr_device().cus;
    const int64_t groups = (N + 1) / 2;
    const int ng = (int)((groups + (int64_t)cus * 16 - 1) / ((int64_t)cus * 16));
    const unsigned grid = (unsigned)(((groups + ng - 1) / ng + 15) / 16);
    const size_t lds = (size_t)nseg * 1024 * (size_t)M;
    if (M == 2) {
        quant_gemv_mt_kernel<2><<<dim3(grid), dim3(1024), lds, st>>>((const u32x4*)x, 2, cols8, clip, (const uint8_t*)W,
                                                                     (const f16*)sW, (const f16*)bias, (int)N, ng, (f16*)y);
        return qr_launch_status();
    }
#define QR_QG(NV)                                                                                                          \
    quant_gemv_kernel<NV><<<dim3(grid), dim3(1024), lds, st>>>((const u32x4*)x, cols8, clip, (const uint8_t*)W, (const f16*)sW, \
                                                               (const f16*)bias, (int)N, ng, (f16*)y)
    if (cols8 <= 1024) QR_QG(1);
    else if (cols8 <= 2048) QR_QG(2);
    else QR_QG(4);
#undef QR_QG
    return qr_launch_status();
}
