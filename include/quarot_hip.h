/*
 * quarot_hip.h - C ABI of libquarot_hip.so: QuaRot's quantized-linear hot path on gfx950 (MI355X).
 *
 * Conventions
 *   - Every pointer except `stream` and `hadK`-when-K==1 is a DEVICE pointer owned by the caller.
 *     The library never allocates, frees or synchronises; kernels are enqueued on `stream`
 *     (a hipStream_t passed as void*, NULL = the default stream).
 *   - Matrices are dense row-major.  "int4 packed" means two two's-complement nibbles per byte,
 *     even column in the LOW nibble (reference: quarot/kernels/include/int4.h:86-98,
 *     quarot/functional/quantization.py:42-49).
 *   - fp16 is IEEE binary16.  Every fp16 operation the reference performs is performed here as one
 *     correctly rounded operation in the same order, so codes and dequantised values are bit-exact.
 *   - Return value: 0 = success; < 0 = argument error (QR_E_*), nothing was launched;
 *     > 0 = a hipError_t reported by the launch.  qr_strerror() explains either.
 *
 * Reference paths are relative to the spcl/QuaRot source tree.
 */
#ifndef QUAROT_HIP_H
#define QUAROT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QR_OK            0
#define QR_E_NULL       -1   /* a required pointer is NULL */
#define QR_E_SHAPE      -2   /* a size is negative, zero where it may not be, or violates a divisibility rule */
#define QR_E_UNSUPPORTED -3  /* valid for the reference but outside what this build implements */
#define QR_E_ALIGN      -4   /* a pointer is not aligned as the entry point requires */
#define QR_E_DTYPE      -5   /* unknown dtype / mode code */
#define QR_E_WORKSPACE  -6   /* the workspace is NULL, misaligned or smaller than the entry point needs */
#define QR_E_SCRATCH_LIMIT -7 /* the shape needs more scratch than the library's built-in buffer holds */

#define QR_DTYPE_F16 0
#define QR_DTYPE_F32 1
/* or-ed into the `mode` of qr_hadamard_quantize_f16_i4 / qr_quantized_linear_f16: hadK points to SIGN WORDS instead of
 * the table -- uint32 [K][ceil(K / 32)] row-major, 4-byte aligned, bit j of word w of row r set where hadK[r][32 w + j]
 * is -1 and clear where it is +1 (bits past column K clear).  A prepared operand like a packed weight: built once per
 * table by the caller, 4 KB where the fp16 table of order 172 is 59 KB that every workgroup would fetch.  Only for
 * tables of +-1 (all of the reference's are); taken where the lean kernel applies (n / K = 64, K = 97 .. 192, no copy
 * of the transformed rows), QR_E_UNSUPPORTED with nothing launched otherwise: pass the table then. */
#define QR_HADK_SIGNS 0x100

/* Library version (major*10000 + minor*100 + patch). */
int qr_version(void);

/* Human-readable text for a return code of any entry point (static storage). */
const char* qr_strerror(int code);

/*
 * Online Hadamard transform along the last axis:  y = x . (hadK (x) H_{n/K})^T * scale.
 * Replaces fast_hadamard_transform.hadamard_transform + `hadK @ input` as called by
 * matmul_hadU_cuda (quarot/functional/hadamard.py:92-101) and matmul_had_cuda
 * (quarot/transformers/kv_cache.py:30-33).
 *   x, y    [rows, n] of `dtype` (QR_DTYPE_F16 or QR_DTYPE_F32); y may alias x.
 *   K       1, or the order of hadK; n % K == 0 and n / K a power of two; n <= 32768, and n <= 128
 *           when n / K < 8 (e.g. had_40 alone across the 40 attention heads of Llama-2-13B).
 *   hadK    [K, K] row-major of `dtype` (the module's had_rem_dim buffer), ignored when K == 1.
 *           Entries must be exactly representable in fp16 (the reference's tables are +-1).
 *   scale   applied in fp32 after the butterflies (the reference passes 1/sqrt(n)).
 * Numerics: butterflies and scale in fp32.  QR_DTYPE_F16: the power-of-two stage is rounded to fp16
 * before the hadK stage, whose fp32 accumulation is rounded to fp16 (the reference's staging).
 * QR_DTYPE_F32: fp32 throughout.
 */
int qr_hadamard(const void* x, void* y, int64_t rows, int n, int K, const void* hadK,
                int dtype, float scale, void* stream);

/*
 * Symmetric int4 quantisation with given per-row scales.
 * Replaces sym_quant_host / sym_quantize_f16_i4_kernel (quarot/kernels/quant.cu:11-61), bound as
 * quarot._CUDA.sym_quant (quarot/kernels/bindings.cpp:27-44).
 *   x fp16 [rows, cols], scale fp16 [rows]  ->  q uint8 [rows, ceil(cols/2)]
 *   q = clamp(round_half_even(fp16(x / scale)), -8, 7); 0/0 gives code 0; odd cols leave the last
 *   high nibble 0.
 */
int qr_sym_quant_f16_i4(const void* x, const void* scale, int64_t rows, int64_t cols, void* q,
                        void* stream);

/*
 * Per-token quantiser: row abs-max -> scale -> codes, one pass over x.
 * Replaces Quantizer.forward (quarot/nn/quantization.py:9-13) = four torch kernels + sym_quant.
 *   scales[r] = fp16( float(fp16(amax_r / 7)) * clip ),  q as qr_sym_quant_f16_i4.
 *   x fp16 [rows, cols] -> q uint8 [rows, ceil(cols/2)], scales fp16 [rows]
 */
int qr_quantize_rows_f16_i4(const void* x, float clip, int64_t rows, int64_t cols, void* q,
                            void* scales, void* stream);

/*
 * Fused OnlineHadamard + Quantizer (quarot/nn/hadamard.py:17-23 then quarot/nn/quantization.py:9-13):
 * the transformed row is rounded to fp16 exactly as qr_hadamard(QR_DTYPE_F16 input) would store it
 * and quantised from there, without the fp16 tensor making a round trip through HBM.
 *   x fp16 [rows, n]; mode QR_DTYPE_F16 (fp16 staging) or QR_DTYPE_F32 (OnlineHadamard force_fp32:
 *   hadK is then fp32 [K,K]), optionally | QR_HADK_SIGNS (hadK is then the table's sign words, see above);
 *   y_or_null: optional fp16 [rows, n] copy of the transformed rows.
 *   x and y 16-byte aligned, q 8-byte aligned.
 *   Rows of 128 in fp16 mode need y_or_null (qr_hadamard's kernel for that length writes them and the quantiser reads
 *   them back: two launches); without it, and for rows shorter than 8 K, QR_E_UNSUPPORTED: call qr_hadamard and
 *   qr_quantize_rows_f16_i4.
 */
int qr_hadamard_quantize_f16_i4(const void* x, int64_t rows, int n, int K, const void* hadK,
                                int mode, float scale, float clip, void* q, void* scales,
                                void* y_or_null, void* stream);

/*
 * Fused RMSNorm + Quantizer: the chain in front of q/k/v_proj and gate/up_proj
 * (quarot/nn/normalization.py:15-21 then quarot/nn/quantization.py:9-13; chained in
 * e2e/quantized_llama/modeling_llama.py:40-44,108-110).
 *   y = fp16( float(x) * rsqrt( sum(float(x)^2) / mean_dim + eps ) ), computed in fp32 and rounded to
 *   fp16 once, as the unfused module returns it; q and scales as qr_quantize_rows_f16_i4(y).
 *   x fp16 [rows, cols], cols % 8 == 0 and cols <= 32768 (else QR_E_UNSUPPORTED: use the two
 *   separate steps); y_or_null: optional fp16 [rows, cols] copy of the normalised rows.
 *   x and y 16-byte aligned, q 4-byte aligned.
 */
int qr_rmsnorm_quantize_f16_i4(const void* x, int64_t rows, int64_t cols, int mean_dim, float eps,
                               float clip, void* q, void* scales, void* y_or_null, void* stream);

/*
 * Fused Hadamard across attention heads + Quantizer: the chain in front of o_proj
 * (e2e/quantized_llama/modeling_llama.py:108-110: quarot.nn.OnlineHadamard(num_heads) applied to
 * attn_output.transpose(-1, -2), transposed back and reshaped to [.., hidden], then o_proj's
 * quarot.nn.Quantizer; the transform itself is quarot/nn/hadamard.py:17-23 with K = 1, i.e.
 * quarot/functional/hadamard.py:92-101 on a last axis of length num_heads).
 *   x fp16 [rows, heads * head_dim], a row being [heads, head_dim] as attention writes it;
 *   y[r, g, d] = fp16( (1 / sqrt(heads)) * sum_h Had[g, h] * x[r, h, d] ), Had the Sylvester matrix of
 *   size heads, summed in fp32 and rounded to fp16 once; q and scales as qr_quantize_rows_f16_i4(y)
 *   over the whole row.  No transposed copies are made.
 *   head_dim == 128 and heads in {16, 32, 64}, hadK_or_null ignored; or heads the order of one of
 *   the reference's tables (12, 20, 28, 36, 40, 52, 60: Llama-2-13B has 40 heads, Llama-30B 52) with
 *   hadK_or_null = that table, fp16 [heads, heads] (the module's had_rem_dim buffer): OnlineHadamard
 *   is then hadK alone and y[r, g, d] = fp16( sum_h hadK[g, h] * fp16(x[r, h, d] / sqrt(heads)) ), the
 *   reference's two-step rounding (quarot/functional/hadamard.py:99-100).  Anything else returns
 *   QR_E_UNSUPPORTED (use qr_hadamard on a transposed copy and qr_quantize_rows_f16_i4).
 *   y_or_null: optional fp16 copy of the transformed rows.  x and y 16-byte aligned, q 4-byte aligned.
 */
int qr_heads_hadamard_quantize_f16_i4(const void* x, int64_t rows, int heads, int head_dim,
                                      const void* hadK_or_null, float clip, void* q, void* scales,
                                      void* y_or_null, void* stream);

/*
 * int4 x int4 -> int32 GEMM:  C[M, N] = unpack(A)[M, K] . unpack(B)[N, K]^T.
 * Replaces matmul_host (quarot/kernels/gemm.cu:7-46), bound as quarot._CUDA.matmul
 * (quarot/kernels/bindings.cpp:9-25).
 *   A uint8 [M, K/2], B uint8 [N, K/2], C int32 [M, N]; K % 64 == 0 (quarot/__init__.py:38),
 *   K <= 131008; A and B 16-byte aligned.
 */
int qr_matmul_i4_i32(const void* A, const void* B, int64_t M, int64_t N, int64_t K, void* C,
                     void* stream);

/*
 * y[r, c] = fp16( fp16(scale_row[r] * scale_col[c]) * fp16_rn(q[r, c]) ).
 * Replaces sym_dequant_host / sym_dequantize_i32_f16_kernel (quarot/kernels/quant.cu:64-97), bound
 * as quarot._CUDA.sym_dequant with bits == 32 (quarot/kernels/bindings.cpp:47-87).
 */
int qr_sym_dequant_i32_f16(const void* q, const void* scale_row, const void* scale_col,
                           int64_t rows, int64_t cols, void* y, void* stream);

/*
 * Linear4bit.forward in one kernel (quarot/nn/linear.py:42-56): the GEMM above with the dequant
 * (and the optional fp16 bias add, a fourth rounded operation) applied to the accumulators.
 *   A uint8 [M, K/2], sA fp16 [M], W uint8 [N, K/2], sW fp16 [N], bias fp16 [N] or NULL -> y fp16 [M, N]
 */
int qr_linear_i4_f16(const void* A, const void* sA, const void* W, const void* sW,
                     const void* bias_or_null, int64_t M, int64_t N, int64_t K, void* y,
                     void* stream);

/*
 * The same with a caller-provided scratch buffer, for shapes whose output tiles would occupy only a
 * fraction of the CUs (decode batches of 40..64 tokens against a narrow weight with K >= 16384,
 * prompts of a few hundred tokens): K is then split across workgroups, each slice leaves its int32 partial sums in
 * `workspace` and a second kernel adds and dequantises them (two launches on `stream`).  The library never
 * allocates (the reference's bindings allocate their outputs with torch::empty,
 * quarot/kernels/bindings.cpp:20,39,74; here the caller does).
 *   qr_workspace_bytes: bytes that qr_linear_i4_f16_ws can use for this shape (0: none; any M, N, K).
 *   workspace: device memory, 16-byte aligned, at least qr_workspace_bytes(M, N, K) bytes; NULL or a
 *   smaller size selects the single-launch path of qr_linear_i4_f16.  Results are identical bit for
 *   bit either way (integer partial sums).  Calls that share a workspace must not overlap.
 */
size_t qr_workspace_bytes(int64_t M, int64_t N, int64_t K);
int qr_linear_i4_f16_ws(const void* A, const void* sA, const void* W, const void* sW,
                        const void* bias_or_null, int64_t M, int64_t N, int64_t K, void* y,
                        void* workspace, size_t workspace_bytes, void* stream);

/*
 * qr_linear_i4_f16_ws without a workspace argument and without any allocation.  It has NO counterpart
 * in the reference (whose bindings allocate with torch::empty on every call); it exists for callers
 * that cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  The K-split slabs live in a buffer of QR_STATIC_SCRATCH_BYTES that is part
 * of the library's device image (one copy per GPU, held until the process ends); the call itself
 * performs no hipMalloc / hipFree and no allocating library call.
 *   Same operands and bit-identical results as qr_linear_i4_f16_ws with a sufficient workspace.
 *   A shape whose qr_workspace_bytes(M, N, K) exceeds QR_STATIC_SCRATCH_BYTES returns
 *   QR_E_SCRATCH_LIMIT and launches nothing (use qr_linear_i4_f16 or the _ws form); shapes that need
 *   no scratch run the single-launch kernels.
 *   All calls on one GPU share that GPU's buffer: calls that overlap in time on one GPU (different
 *   streams or host threads) race.  The first call on a device looks the buffer's address up
 *   (hipGetSymbolAddress); make that call outside graph capture.  The buffer is the CURRENT device's
 *   (hipGetDevice at the time of the call): `stream` must belong to the current device.  A failure
 *   of that look-up comes back as the positive hipError_t, like a launch error.
 */
#define QR_STATIC_SCRATCH_BYTES (32u << 20)
int qr_linear_i4_f16_static(const void* A, const void* sA, const void* W, const void* sW,
                            const void* bias_or_null, int64_t M, int64_t N, int64_t K, void* y,
                            void* stream);

/*
 * Linear4bit.forward (quarot/nn/linear.py:42-56) for prefill shapes on the FP6 matrix path: the same
 * product and the same fp16 epilogue as qr_linear_i4_f16, bit for bit (every int4 code is a value of
 * FP6 E3M2, products and sums stay integers below 2^24, so the fp32 accumulators are exact), at a higher
 * matrix-instruction rate.  Both operands must first be converted to the 6-bit stage-major layout this
 * kernel reads; the reference has no counterpart (its CUTLASS call takes the packed nibbles,
 * quarot/kernels/gemm.cu:16-41).
 *   qr_f6_bytes(rows, K): bytes of a converted operand (rows * K * 3 / 4; K % 64 == 0).
 *   qr_convert_i4_f6: codes uint8 [rows, K/2] (16-byte aligned) -> out (8-byte aligned, qr_f6_bytes bytes).
 *     Weights are converted once after loading, activations after the quantiser.
 *   qr_linear_f6_f16: A6 = converted codes of x [M, K], W6 = converted weight [N, K] (both 16-byte
 *     aligned, each below 4 GiB, else QR_E_UNSUPPORTED), sA fp16 [M], sW fp16 [N], bias fp16 [N] or NULL
 *     -> y fp16 [M, N] (8-byte aligned).  Any M, N; meant for long prompts (256 x 256 tiles, or 128 x 256 when
 *     those fill the compute units in fewer rounds).
 */
size_t qr_f6_bytes(int64_t rows, int64_t K);
int qr_convert_i4_f6(const void* codes, int64_t rows, int64_t K, void* out, void* stream);
int qr_linear_f6_f16(const void* A6, const void* sA, const void* W6, const void* sW,
                     const void* bias_or_null, int64_t M, int64_t N, int64_t K, void* y, void* stream);

/*
 * A whole quantised linear layer in one host call: the module chain
 *   torch.nn.Sequential(OnlineHadamard(K), Quantizer(clip), Linear4bit)        (had_K >= 1)
 *   torch.nn.Sequential(Quantizer(clip), Linear4bit)                           (had_K == 0)
 * of e2e/quantized_llama/modeling_llama.py:99-102,111-115 (quarot/nn/hadamard.py:17-23,
 * quarot/nn/quantization.py:9-13, quarot/nn/linear.py:42-56).  It enqueues exactly the launches of
 * qr_hadamard_quantize_f16_i4 (or qr_quantize_rows_f16_i4) and qr_linear_i4_f16_ws on `stream`, with
 * the codes and scales between them in `workspace`: same results bit for bit, one call instead of
 * two for hosts whose per-call cost matters (a decode step launched from Python).
 * ONE or TWO tokens (M <= 2) behind a 1024-point factor (K == 1024 * had_K, had_K a multiple of 4 up to 32:
 * the 70B down_proj, 28672 = 1024 x 28), mode QR_DTYPE_F16: a single kernel in which every workgroup
 * transforms and quantises the rows itself and goes straight on to its dot products -- the same codes,
 * scales, sums and epilogue, so y carries the same bits, and the weight stream starts while the rows are
 * still being transformed.  ONE or TWO tokens with had_K == 0 (K up to 32768): likewise one kernel, every
 * workgroup quantising the rows itself.  The workspace is checked as always; what it holds afterwards
 * is unspecified.
 *   x fp16 [M, K]; had_K, hadK, mode, scale as in qr_hadamard_quantize_f16_i4; W uint8 [N, K/2],
 *   sW fp16 [N], bias fp16 [N] or NULL -> y fp16 [M, N].
 *   workspace: device memory, 16-byte aligned, at least qr_quantized_linear_workspace_bytes(M, N, K)
 *   bytes (never 0 for M > 0), else QR_E_WORKSPACE.  Calls that share a workspace must not overlap.
 */
size_t qr_quantized_linear_workspace_bytes(int64_t M, int64_t N, int64_t K);
int qr_quantized_linear_f16(const void* x, int64_t M, int64_t K, int had_K, const void* hadK, int mode,
                            float scale, float clip, const void* W, const void* sW,
                            const void* bias_or_null, int64_t N, void* y, void* workspace,
                            size_t workspace_bytes, void* stream);

/*
 * KV-cache path: optional Hadamard over the head dimension, then per-vector asymmetric int4.
 * Replaces matmul_had_cuda + asym_quantize_and_pack_i4 (quarot/transformers/kv_cache.py:10-33).
 *   x fp16 [vectors, dim], dim a power of two in [16, 256].
 *   had_mode: 0 = none (V), 1 = FWHT * 1/sqrt(dim) rounded to fp16 (K).
 *   q uint8 [vectors, dim/2]; scale, zero fp16 [vectors]:
 *   scale = max(fp16(max - min), fp16(1e-5)) / 15, zero = -min,
 *   q = clamp(round_half_even(fp16(fp16(x + zero) / scale)), 0, 15).
 */
int qr_kv_quant_f16_i4(const void* x, int64_t vectors, int dim, int had_mode, void* q,
                       void* scale, void* zero, void* stream);

/*
 * Inverse of the above: y = fp16( fp16(nibble * scale) - zero )
 * (unpack_i4_and_asym_dequantize, quarot/transformers/kv_cache.py:24-28).
 */
int qr_kv_dequant_i4_f16(const void* q, const void* scale, const void* zero, int64_t vectors,
                         int dim, void* y, void* stream);

/*
 * Paged int4 KV cache (quarot/kernels/include/flashinfer/page.cuh:19-113), head_dim 128:
 *   kv_data   uint8 [num_pages, num_layers, 2 (K, V), num_heads, page_size, 64]   packed codes
 *   kv_param  fp16  [num_pages, num_layers, 2 (K, V), num_heads, page_size, 2]    {scale, zero} per vector
 *   kv_indptr int32 [batch_size + 1], kv_indices int32 [kv_indptr[batch_size]], last_page_offset int32 [batch_size]:
 *   sequence b owns pages kv_indices[kv_indptr[b] .. kv_indptr[b + 1] - 1] and holds
 *   (pages - 1) * page_size + last_page_offset[b] tokens.  All five are device pointers.
 * The index arrays cannot be checked on the host: a token whose place lies outside the sequence's page
 * list, or on a page number outside [0, num_pages), is skipped on the device instead of written / read.
 */

/*
 * Copy already quantised K and V vectors of new tokens into their pages.
 * Replaces quarot._CUDA.init_kv_i4 and append_kv_i4 (quarot/kernels/bindings.cpp:155-245 ->
 * AppendPagedKVCachePrefillKernel / AppendPagedKVCacheDecodeKernel, page.cuh:120-219).
 *   k, v uint8 [tokens, num_heads, 64]; k_param, v_param fp16 [tokens, num_heads, 2] = {scale, zero}.
 *   append_indptr_or_null: int32 [batch_size + 1] (init_kv_i4's seqlen_indptr): the tokens of sequence b
 *   are append_indptr[b] .. append_indptr[b + 1] - 1 and become the LAST positions of the sequence, whose
 *   length (from kv_indptr / last_page_offset) already includes them.  NULL: one token per sequence
 *   (append_kv_i4), tokens == batch_size, written at position length - 1.
 *   k, v, kv_data 16-byte aligned.
 */
int qr_kv_append_i4(void* kv_data, void* kv_param, const void* kv_indptr, const void* kv_indices,
                    const void* last_page_offset, int64_t num_pages, const void* k, const void* v,
                    const void* k_param, const void* v_param, const void* append_indptr_or_null,
                    int64_t tokens, int num_layers, int layer_idx, int num_heads, int page_size,
                    int head_dim, int64_t batch_size, void* stream);

/*
 * The same from fp16 K and V, quantising on the way: what MultiLayerPagedKVCache4Bit.update runs as
 * matmul_had_cuda(K), asym_quantize_and_pack_i4 (K and V), two torch.cat of {scale, zero} and
 * init_kv_i4 / append_kv_i4 (quarot/transformers/kv_cache.py:174-251).  Codes, scales and zeros are those
 * of qr_kv_quant_f16_i4 bit for bit; they go straight to their pages (one launch for keys and values).
 *   k, v fp16 [tokens, num_heads, 128]; k_had_mode as qr_kv_quant_f16_i4's had_mode (1: Hadamard over the
 *   head dimension first); append_indptr_or_null as above.
 */
int qr_kv_quant_append_f16_i4(const void* k, const void* v, int64_t tokens, const void* append_indptr_or_null,
                              int k_had_mode, void* kv_data, void* kv_param, const void* kv_indptr,
                              const void* kv_indices, const void* last_page_offset, int64_t num_pages,
                              int num_layers, int layer_idx, int num_heads, int page_size, int head_dim,
                              int64_t batch_size, void* stream);

/*
 * Single-query attention over the paged int4 cache:
 *   o[b, h, :] = sum_j softmax_j( q[b, h, :] . k_j / sqrt(head_dim) ) v_j,   j over the tokens of sequence b,
 *   k_j[i] = float(code) * scale_j - zero_j in fp32 (quarot/kernels/include/flashinfer/quantization.cuh:59-84).
 * Replaces quarot._CUDA.batch_decode_i4 (quarot/kernels/bindings.cpp:118-153 ->
 * BatchDecodeWithPagedKVCacheKernel, decode.cuh:492-689; no rotary embedding, as the reference calls it).
 *   q, o fp16 [batch_size, num_heads, 128] (q 16-byte aligned).  fp32 arithmetic, results within
 *   rtol 1e-3 / atol 1e-3 of the exact softmax over the dequantised cache.
 *   max_seq_len: an upper bound of the sequences' lengths if the caller knows one, else 0.  With it and a
 *   workspace of qr_batch_decode_workspace_bytes(batch_size, num_heads, max_seq_len) bytes (16-byte
 *   aligned) a small batch is split along the sequence over several workgroups per (sequence, head) and
 *   a second launch merges them; without, one workgroup serves each (sequence, head).
 */
size_t qr_batch_decode_workspace_bytes(int64_t batch_size, int num_heads, int64_t max_seq_len);
int qr_batch_decode_i4(void* o, const void* q, const void* kv_data, const void* kv_param,
                       const void* kv_indptr, const void* kv_indices, const void* last_page_offset,
                       int64_t num_pages, int num_layers, int layer_idx, int num_heads, int page_size,
                       int head_dim, int64_t batch_size, int64_t max_seq_len, void* workspace,
                       size_t workspace_bytes, void* stream);

/*
 * qr_batch_decode_i4 with the query's Hadamard inside: what the reference's decode step does as two calls,
 * matmul_had_cuda(q, torch.float16) (quarot/transformers/kv_cache.py:30-33,113: fast_hadamard_transform over
 * the head dimension, scale 1 / sqrt(128), result in fp16) and then batch_decode_i4, in ONE launch -- every
 * workgroup transforms its own query vector (128 values, fp32 butterflies, rounded to fp16 as that function's
 * result is) before it walks the cache.  Same arguments and tolerance as qr_batch_decode_i4; q is the
 * untransformed query.
 */
int qr_batch_decode_qhad_i4(void* o, const void* q, const void* kv_data, const void* kv_param,
                            const void* kv_indptr, const void* kv_indices, const void* last_page_offset,
                            int64_t num_pages, int num_layers, int layer_idx, int num_heads, int page_size,
                            int head_dim, int64_t batch_size, int64_t max_seq_len, void* workspace,
                            size_t workspace_bytes, void* stream);

/*
 * One decode step of the paged cache in ONE launch: qr_kv_quant_append_f16_i4 (one new token per sequence,
 * append_indptr NULL) followed by qr_batch_decode_i4 / qr_batch_decode_qhad_i4 -- what
 * MultiLayerPagedKVCache4Bit.update and the callable it returns do for a decode step
 * (quarot/transformers/kv_cache.py:104-129,224-251).  The page tables already count the new token (it is the
 * LAST position of its sequence, as for qr_kv_quant_append_f16_i4); the first wave of every (sequence, head)
 * quantises the token's key (through H_128 when k_had_mode = 1) and value with the arithmetic of that entry
 * point -- the same codes, scales and zeros, written to the same page slots -- and attends to them from its
 * registers while the other waves walk the cached positions.
 *   k, v fp16 [batch_size, num_heads, 128] (16-byte aligned); q_had_mode 0 / 1 as the two entry points above;
 *   everything else as qr_batch_decode_i4.  A sequence whose page list is empty is skipped by the append and
 *   gets a NaN output row, as there.
 */
int qr_kv_quant_append_batch_decode_f16_i4(void* o, const void* q, int q_had_mode, const void* k, const void* v,
                                           int k_had_mode, void* kv_data, void* kv_param, const void* kv_indptr,
                                           const void* kv_indices, const void* last_page_offset,
                                           int64_t num_pages, int num_layers, int layer_idx, int num_heads,
                                           int page_size, int head_dim, int64_t batch_size, int64_t max_seq_len,
                                           void* workspace, size_t workspace_bytes, void* stream);

/*
 * The paged cache with fp16 pages (the reference's disable_quant mode, quarot/transformers/kv_cache.py:134-151,189-193):
 *   kv_data fp16 [num_pages, num_layers, 2 (K, V), num_heads, page_size, 128]; kv_param and the page tables as above.
 *
 * qr_kv_append_f16 replaces quarot._CUDA.init_kv_f16 and append_kv_f16 (quarot/kernels/bindings.cpp:287-374):
 *   k, v fp16 [tokens, num_heads, 128]; k_param, v_param fp16 [tokens, num_heads, 2] (the cache class passes
 *   {1, 0}); append_indptr_or_null, tokens and the alignment rules as qr_kv_append_i4.
 * qr_batch_decode_f16 replaces quarot._CUDA.batch_decode_f16 (quarot/kernels/bindings.cpp:247-285):
 *   o[b, h, :] = sum_j softmax_j( q[b, h, :] . k_j / sqrt(128) ) v_j over the cached fp16 vectors, fp32 arithmetic,
 *   within rtol 1e-3 / atol 1e-3 of the exact result; kv_param is not read.  q, o fp16 [batch_size, num_heads, 128].
 *   One workgroup per (sequence, head); a sequence without pages gets a NaN row, as qr_batch_decode_i4 gives.
 */
int qr_kv_append_f16(void* kv_data, void* kv_param, const void* kv_indptr, const void* kv_indices,
                     const void* last_page_offset, int64_t num_pages, const void* k, const void* v,
                     const void* k_param, const void* v_param, const void* append_indptr_or_null,
                     int64_t tokens, int num_layers, int layer_idx, int num_heads, int page_size,
                     int head_dim, int64_t batch_size, void* stream);
int qr_batch_decode_f16(void* o, const void* q, const void* kv_data, const void* kv_param,
                        const void* kv_indptr, const void* kv_indices, const void* last_page_offset,
                        int64_t num_pages, int num_layers, int layer_idx, int num_heads, int page_size,
                        int head_dim, int64_t batch_size, void* stream);

/*
 * Measurement aids.  NO counterpart in the reference and no caller in the product path: kernels whose
 * work is known exactly, run by bench.py next to the workloads to calibrate the rooflines.
 *
 * qr_calib_mfma_i8: `workgroups` workgroups of four waves, each wave `iters` turns of 16
 *   v_mfma_i32_32x32x32_i8 (four independent accumulator chains, operands and accumulators in
 *   registers, no memory access): workgroups * 4 * iters * 16 * 65536 integer operations per launch.
 *   pattern 0: all-zero operands; 1: random int4 codes as the int4 GEMMs feed them (16 * code in every
 *   byte); 2: random int8 bytes; 3: random int4 codes as sign-extended int8.  `out` (device, >= workgroups * 1024 bytes) is never written (it only
 *   keeps the loop observable).
 * qr_calib_copy: dst[0 .. bytes) = src[0 .. bytes) with 16-byte nontemporal loads and stores (bytes a
 *   multiple of 16, pointers 16-byte aligned): `bytes` read and `bytes` written per launch.
 */
int qr_calib_mfma_i8(int pattern, int iters, int workgroups, void* out, void* stream);
int qr_calib_copy(const void* src, void* dst, int64_t bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* QUAROT_HIP_H */
