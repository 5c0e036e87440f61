/*
 * astrai_q -- C ABI of the MI355X (gfx950) quantized-Linear path.
 *
 * The reference's Linear layer has no FFI: it is one Python call,
 *   y = F.linear(x, weight, bias)      astrai/model/components/linear.py:20-21
 * with weight laid out [out_dim, in_dim] (linear.py:10) and an optional bias
 * [out_dim] (linear.py:11).  Every entry point below is a stage of the
 * quantized replacement of that one call; each comment names the part of the
 * reference call it stands in for.
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer owned by the caller.  The library never
 *    allocates, frees or synchronises; work is queued on `stream` (a
 *    hipStream_t passed as void*, NULL = the null stream).
 *  - Matrices are row-major and contiguous unless a leading dimension is given.
 *    K (the reduction length, Linear's in_dim) must be a multiple of 16 and
 *    every matrix base 16-byte aligned.
 *  - dtype codes: AQ_F32 = 0, AQ_BF16 = 1.
 *  - Return value: 0 on success, a negative AQ_E_* for a rejected argument, or
 *    a positive hipError_t from the launch.  aq_error_string() names either.
 *  - Re-entrant: no mutable state outlives a call except where an entry point says so (the
 *    no-allocation variant's scratch).  (The reference calls Linear from its scheduler's
 *    daemon thread, astrai/inference/core/scheduler.py:191-196.)
 */
#ifndef ASTRAI_Q_H
#define ASTRAI_Q_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AQ_VERSION 100

enum { AQ_F32 = 0, AQ_BF16 = 1 };

enum {
  AQ_OK = 0,
  AQ_E_NULL = -1,      /* a required pointer is NULL                */
  AQ_E_SHAPE = -2,     /* negative size, K not a multiple of 16 ... */
  AQ_E_DTYPE = -3,     /* unknown dtype code                        */
  AQ_E_ALIGN = -4,     /* pointer or leading dimension not 16-byte aligned */
  AQ_E_WORKSPACE = -5, /* workspace too small                       */
  AQ_E_RANGE = -6      /* size beyond what the kernels index        */
};

int aq_version(void);
const char *aq_error_string(int code);

/* Symmetric absmax int8 per row: scale[r] = amax_r / 127 (1 when the row is all
 * zero), q = clamp(rint(x / scale), -127, 127), round-half-even, true divide.
 * Used per token on the activation x of Linear.forward (linear.py:20) and, once
 * and offline, per output channel on Linear.weight (linear.py:10).
 * x: [M, K] of x_dtype with row stride ldx elements; q: [M, K]; scale: [M]. */
int aq_quant_rowwise_i8(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                        int8_t *q, float *scale, void *stream);

/* Per-tensor FP8 (OCP e4m3fn): scale[0] = amax / 448 (1 when all zero),
 * q = e4m3fn_rne(clamp(x / scale, -448, 448)).  Stands in for the operands of
 * the same F.linear call (linear.py:21) in the FP8 variant.
 * amax_ws: device scratch of ws_bytes >= AQ_FP8_AMAX_WS_BYTES (partial maxima, one per workgroup of the first
 * pass; a smaller one is AQ_E_WORKSPACE: the size is an argument so that a buffer of a single word is refused
 * instead of written past).  It needs no initial value and carries
 * nothing from one call to the next; two calls that overlap in time must not share it.  Two launches: maximum,
 * then scale + cast. */
#define AQ_FP8_AMAX_WS_BYTES 1024
int aq_quant_tensor_fp8(const void *x, int x_dtype, int64_t numel, uint8_t *q, float *scale,
                        uint32_t *amax_ws, size_t ws_bytes, void *stream);

/* The same result in ONE launch, for callers that can keep a small piece of device state: every workgroup holds
 * its share of x in registers between the maximum and the cast (tensors up to 32 MiB on 256 compute units are read
 * from HBM once instead of twice; what does not fit is read again), and the workgroups exchange their partial
 * maxima through ws while the kernel runs.  ws: AQ_FP8_ONEPASS_WS_BYTES of device memory, 8-byte aligned, that
 * must be ZERO-FILLED before its first use and is then left, after every call, in a state the next call accepts
 * (so: fill once, reuse for every later call on that device); calls that overlap in time must not share one.
 * The wait for the other workgroups is bounded: if they cannot all run at once (a busy or partitioned device) each
 * takes the tensor's maximum itself after about a millisecond -- same codes and scale, much slower.
 * Same definition and reference call site as aq_quant_tensor_fp8 (linear.py:21, FP8 variant). */
#define AQ_FP8_ONEPASS_WS_BYTES 2048
int aq_quant_tensor_fp8_onepass(const void *x, int x_dtype, int64_t numel, uint8_t *q, float *scale,
                                void *ws, size_t ws_bytes, void *stream);

/* acc[m, n] = sum_k xq[m, k] * wq[n, k], exact int32: the matrix product inside
 * F.linear (linear.py:21) on int8 codes.  xq: [M, K], wq: [N, K], acc: [M, N]. */
int aq_gemm_i8_i32(const int8_t *xq, const int8_t *wq, int32_t *acc, int64_t M, int64_t N,
                   int64_t K, void *stream);

/* The same product with the dequantising epilogue fused:
 * y[m, n] = (float(acc) * sx[m]) * sw[n] (+ bias[n]), each step rounded to
 * fp32, then one round-to-nearest-even cast to y_dtype.  Replaces the whole
 * F.linear(x, weight, bias) of linear.py:21 for M > 16.
 * bias may be NULL (the reference never constructs a Linear with bias=True).
 * Any M: a tiled matrix-core GEMM whose tile is chosen by shape (128 x 32 up to 256 x 128), except
 * that 17..32 rows (K a multiple of 128) run on the weight-streaming kernel of the decode path
 * instead, with the same bits. */
int aq_linear_w8a8(const int8_t *xq, const float *sx, const int8_t *wq, const float *sw,
                   const void *bias, int bias_dtype, void *y, int y_dtype, int64_t M,
                   int64_t N, int64_t K, void *stream);

/* Decode path, M <= 16 rows of x: quantises x per token on the fly, streams wq
 * once and writes y in y_dtype; same arithmetic and results as
 * aq_quant_rowwise_i8 followed by aq_linear_w8a8.  Replaces F.linear
 * (linear.py:21) when the caller is the decode step (M = batch <= 16,
 * astrai/inference/core/executor.py:59-94).
 * ws: device scratch of at least aq_gemv_w8a8_workspace_bytes(M, K). */
size_t aq_gemv_w8a8_workspace_bytes(int64_t M, int64_t K);
int aq_gemv_w8a8_decode(const void *x, int x_dtype, const int8_t *wq, const float *sw,
                        const void *bias, int bias_dtype, void *y, int y_dtype, int64_t M,
                        int64_t N, int64_t K, void *ws, size_t ws_bytes, void *stream);

/* The GEMV of the decode path on codes the caller already holds (for callers
 * that quantise one activation once and feed several projections with it, as
 * q/k/v_proj and up/gate share their input: astrai/model/components/
 * attention.py:83-85, mlp.py:25).  xq: [M <= 16, K], sx: [M]. */
int aq_gemv_w8a8_codes(const int8_t *xq, const float *sx, const int8_t *wq, const float *sw,
                       const void *bias, int bias_dtype, void *y, int y_dtype, int64_t M,
                       int64_t N, int64_t K, void *stream);

/* The three entry points above with the residual connection around the Linear
 * fused into the epilogue: y = round(linear) + residual, rounded to y_dtype
 * again -- the bits of the reference's separate elementwise add
 * (`attn_output + x`, `self.mlp(...) + x`, astrai/model/components/
 * decoder_block.py:56-57), without the extra pass over [M, N].
 * residual: [M, N] contiguous in y_dtype, or NULL (then identical to the entry
 * points above).  It may be y itself: every element is read by the lane that
 * writes it. */
int aq_linear_w8a8_residual(const int8_t *xq, const float *sx, const int8_t *wq, const float *sw,
                            const void *bias, int bias_dtype, const void *residual, void *y,
                            int y_dtype, int64_t M, int64_t N, int64_t K, void *stream);
int aq_gemv_w8a8_decode_residual(const void *x, int x_dtype, const int8_t *wq, const float *sw,
                                 const void *bias, int bias_dtype, const void *residual, void *y,
                                 int y_dtype, int64_t M, int64_t N, int64_t K, void *ws,
                                 size_t ws_bytes, void *stream);

/* The same call for callers that cannot allocate.  No counterpart in the reference: it is for code under
 * HIP graph capture, tight serving loops and harnesses that forbid hipMalloc, which cannot provide the
 * workspace of the entry point above.  The workspace (activation codes and scales between the row quantiser
 * and the GEMV) is a device array that the library owns: AQ_GEMV_NOALLOC_MAX_MK + 256 bytes on every GPU the
 * library runs on, held until the process ends.  M * K beyond AQ_GEMV_NOALLOC_MAX_MK (16 rows of 16384) is
 * AQ_E_RANGE.  Allocates nothing and calls no allocating routine; the array's address is looked up on the first
 * call on each device (make that call outside a graph capture).  Every call on a GPU uses that GPU's one array:
 * calls that overlap in time on the same GPU (two streams, two threads) race on it -- serialise them or
 * use aq_gemv_w8a8_decode_residual with a workspace per stream.  Results are bit-identical to that entry point. */
#define AQ_GEMV_NOALLOC_MAX_MK 262144
int aq_gemv_w8a8_decode_noalloc(const void *x, int x_dtype, const int8_t *wq, const float *sw,
                                const void *bias, int bias_dtype, const void *residual, void *y,
                                int y_dtype, int64_t M, int64_t N, int64_t K, void *stream);
int aq_gemv_w8a8_codes_residual(const int8_t *xq, const float *sx, const int8_t *wq, const float *sw,
                                const void *bias, int bias_dtype, const void *residual, void *y,
                                int y_dtype, int64_t M, int64_t N, int64_t K, void *stream);

/* aq_gemv_w8a8_decode_residual with the RMSNorm in front of the Linear folded in:
 * y = linear(quantise(rmsnorm(x) * gamma)) (+ bias) (+ residual), the codes and
 * scales being those aq_rmsnorm_quant_rowwise_i8 gives (same fixed arithmetic),
 * so the result equals that call followed by aq_gemv_w8a8_codes_residual bit
 * for bit.  One launch for up to 8 bf16 rows of at most 2048 elements, those two
 * calls through ws otherwise.  gamma: [K] in x's dtype; residual may be NULL.
 * Replaces the norm + Linear pairs of a decode step (decoder_block.py:50-51,57
 * feeding attention.py:83-85 and mlp.py:25). */
int aq_gemv_w8a8_decode_rmsnorm(const void *x, int x_dtype, const void *gamma, float eps,
                                const int8_t *wq, const float *sw, const void *bias,
                                int bias_dtype, const void *residual, void *y, int y_dtype,
                                int64_t M, int64_t N, int64_t K, void *ws, size_t ws_bytes,
                                void *stream);

/* An MLP's up and gate projections and its activation as one launch at decode (mlp.py:25-26:
 * down(up(x) * silu(gate(x))), the part before `down`), with the norm in front folded in like
 * aq_gemv_w8a8_decode_rmsnorm when gamma is not NULL (decoder_block.py:57).
 * wq: [2F, K] codes, rows [0, F) the up projection and [F, 2F) the gate projection; sw, bias: [2F].
 * h: [M, F] = u * (g / (1 + exp(-g))) with u, g the two projections as aq_gemv_w8a8_decode would have stored them
 * in h_dtype (rounded to bf16 first for a bf16 h), the exponential and divide of aq_swiglu_quant_rowwise_i8, the
 * product rounded to h_dtype: the [M, 2F] intermediate is never written and the separate activation launch
 * disappears.  Served for bf16 x, 1 <= M <= 16, K <= 2048 a multiple of 512, F a multiple of 16
 * (aq_gemv_w8a8_decode_swiglu_ok returns 1); otherwise AQ_E_RANGE and the caller takes the separate launches. */
int aq_gemv_w8a8_decode_swiglu_ok(int x_dtype, int64_t M, int64_t F, int64_t K);
int aq_gemv_w8a8_decode_swiglu(const void *x, int x_dtype, const void *gamma, float eps,
                               const int8_t *wq, const float *sw, const void *bias, int bias_dtype,
                               void *h, int h_dtype, int64_t M, int64_t F, int64_t K, void *stream);

/* FP8 Linear: y[m, n] = (sum_k f(xq[m,k]) * f(wq[n,k])) * sx[0] * sw[0] with
 * fp32 accumulation, cast to y_dtype.  xq: [M, K], wq: [N, K] e4m3fn codes;
 * sx, sw: device scalars written by aq_quant_tensor_fp8.  Replaces F.linear
 * (linear.py:21) in the FP8 variant.  Tiles chosen by shape and 17..32 rows on the
 * weight-streaming kernel, as for aq_linear_w8a8 (the order of the fp32 sums, fixed for a
 * given shape, differs between the kernels). */
int aq_linear_fp8(const uint8_t *xq, const float *sx, const uint8_t *wq, const float *sw,
                  void *y, int y_dtype, int64_t M, int64_t N, int64_t K, void *stream);

/* The same with the optional operands of aq_linear_w8a8_residual: y = ((acc * sx) * sw + bias[n]), cast
 * to y_dtype, then + residual[m, n] (in y's type, may be y itself), rounded again -- the bits of a
 * separate add.  bias: [N] fp32 or bf16 (linear.py:11) or NULL; residual NULL: no add.  Replaces
 * F.linear(x, weight, bias) (linear.py:21) and the block's residual add (decoder_block.py:53,58) in
 * the FP8 variant. */
int aq_linear_fp8_residual(const uint8_t *xq, const float *sx, const uint8_t *wq, const float *sw,
                           const void *bias, int bias_dtype, const void *residual, void *y,
                           int y_dtype, int64_t M, int64_t N, int64_t K, void *stream);

/* The FP8 Linear at decode, M <= 16 rows (executor.py:59-94): the weight-streaming GEMV of aq_gemv_w8a8_decode
 * on e4m3 codes (one 16x16x128 matrix-core product per 128-byte line), per-tensor scales, fp32 accumulation,
 * y = ((acc * sx) * sw + bias) cast, + residual.  aq_gemv_fp8_codes_residual takes codes and scale as
 * aq_quant_tensor_fp8 writes them; aq_gemv_fp8_decode_residual takes the rows themselves and, for bf16 rows
 * of K <= 2048 (K a multiple of 512), casts them inside the GEMV kernel (one launch: the tensor's maximum goes
 * round the workgroup first), otherwise through ws (aq_gemv_fp8_workspace_bytes(M, K) bytes) by
 * aq_quant_tensor_fp8 + the codes entry.  K not a multiple of 256, or rows too long for a compute unit's
 * LDS: the tiled FP8 GEMM takes the call.  Replaces F.linear (linear.py:21) in the FP8 variant. */
size_t aq_gemv_fp8_workspace_bytes(int64_t M, int64_t K);
int aq_gemv_fp8_codes_residual(const uint8_t *xq, const float *sx, const uint8_t *wq, const float *sw,
                               const void *bias, int bias_dtype, const void *residual, void *y,
                               int y_dtype, int64_t M, int64_t N, int64_t K, void *stream);
int aq_gemv_fp8_decode_residual(const void *x, int x_dtype, const uint8_t *wq, const float *sw,
                                const void *bias, int bias_dtype, const void *residual, void *y,
                                int y_dtype, int64_t M, int64_t N, int64_t K, void *ws, size_t ws_bytes,
                                void *stream);

/* RMSNorm followed by per-token quantisation, one launch: the codes and scales
 * aq_quant_rowwise_i8 would give for y = x * rsqrt(mean(x^2) + eps) * gamma held
 * in fp32.  Fuses the reference's F.rms_norm (astrai/model/components/norm.py:14-15)
 * with the activation quantisation of the Linears that consume it
 * (q/k/v: attention.py:83-85 via decoder_block.py:50-51; up/gate: mlp.py:25 via
 * decoder_block.py:57); the normalised activations are never written.
 * x: [M, K] (row stride ldx elements), gamma: [K] in the same dtype as x.
 * Fixed arithmetic: the sum of squares is accumulated per 64-lane stripe of
 * 16-byte vectors and combined by a butterfly (see the oracle), mean = ss / K,
 * r = 1 / sqrt(mean + eps) correctly rounded, y = (x * r) * gamma.  K a
 * multiple of 16 and at most 12288 (bf16) / 6144 (fp32) elements (AQ_E_RANGE beyond). */
int aq_rmsnorm_quant_rowwise_i8(const void *x, int x_dtype, const void *gamma, int gamma_dtype,
                                float eps, int64_t M, int64_t K, int64_t ldx, int8_t *q,
                                float *scale, void *stream);

/* SwiGLU followed by per-token quantisation, one launch: ug is the output
 * [M, 2F] (row stride ld elements) of the fused up/gate projection, columns
 * [0, F) = up(x), [F, 2F) = gate(x); h = up * silu(gate) (mlp.py:25-26) is
 * formed in fp32 and quantised per row, giving the codes [M, F] and scales [M]
 * that the down projection (mlp.py:26) consumes.  h is never written.
 * Fixed arithmetic: silu(g) = g / (1 + e), e = exp(-g) from a fixed sequence of
 * fused multiply-adds (degree-5 polynomial after range reduction; the oracle
 * repeats it bit for bit), correctly rounded divide, one rounded product.
 * F a multiple of 16 and at most 8192 (bf16) / 4096 (fp32) elements. */
int aq_swiglu_quant_rowwise_i8(const void *ug, int dtype, int64_t M, int64_t F, int64_t ld,
                               int8_t *q, float *scale, void *stream);

/* ---- attention around the paged KV cache (what sits between the qkv and the
 * output projection; bf16, head dimension D = 64 or 128).
 *
 * aq_rope_kv_write: for the S new tokens of each of B sequences (S = 1 at
 * decode, the prompt length at prefill), rotate the q and k heads of
 * qkv [B, S, (Hq + 2 Hkv) * D] (q heads, then k heads, then v heads: the fused
 * projection's column order) by freqs [S, D/2, 2] = (cos, sin) pairs per sequence
 * (freqs_stride floats from one sequence's table to the next; 0 when all
 * sequences are at the same positions and share one; 16-byte aligned) --
 * interleaved pairs (x[2i], x[2i+1]), fp32, as apply_rotary_emb does
 * (astrai/model/components/rope.py:26-33) -- store q to q_out [B, S, Hq, D], the
 * rotated k to k_out [B, S, Hkv, D] when that is not NULL (for an attention over
 * the new tokens themselves), and write the rotated k and the v of token s into
 * slot (pos + s) % page_size of page page_table[b, (pos + s) / page_size] of
 * k_cache / v_cache [n_pages, page_size, Hkv, D] (Storage.write,
 * astrai/inference/core/cache.py:216-252; tokens whose page is unmapped, entry
 * < 0, are skipped there too).
 *
 * aq_paged_attn_decode: out [B, Hq, D] = softmax(scale * q K^T) V over positions
 * 0 .. total_len-1 of each sequence, read through page_table [B, P] in place --
 * replaces Storage.gather (cache.py:254-274), repeat_kv (attention.py:15-23) and
 * scaled_dot_product_attention (attention.py:98-100) for a step without padding
 * mask.  Query heads h*G .. h*G+G-1 use KV head h, G = Hq / Hkv in {1, 2, 3, 4, 6, 8}.
 * Positions whose page is unmapped count as zero keys and values (what gather's
 * zero fill gives).  fp32 scores and sums; results within bf16 rounding of the
 * reference flow, not bit-identical to it (summation order, exp2).
 * The positions of a sequence are cut into slices that run as separate
 * workgroups; with more than one slice their partial results pass through
 * `workspace` (16-byte aligned device memory of at least
 * aq_paged_attn_decode_workspace_bytes(B, Hq, Hkv, total_len) bytes, which is 0
 * when one slice suffices -- then workspace may be NULL) and a second, small
 * kernel combines them.  A workspace that is too small is AQ_E_WORKSPACE.  The size
 * grows with total_len: a caller that sizes it once uses the longest sequence
 * it will serve.
 * seq_lens (device int64 [B], or NULL: every sequence attends to all total_len positions): sequence b
 * attends to positions t < seq_lens[b] only.  This is the reference's position mask for a decode batch whose
 * sequences sit at different positions (execute_decode, executor.py:67-71, binds total_len = max position + 1
 * and process_attention_mask, transformer.py:40-46, masks t > position_ids[b]: seq_lens[b] = position_ids[b]
 * + 1); as in the reference the new token still goes to slot total_len - 1 of every sequence.  The same
 * argument has the same meaning in the three entry points below. */
int aq_rope_kv_write(const void *qkv, const float *freqs, int64_t freqs_stride,
                     const int64_t *page_table, int64_t P, int64_t pos, int64_t S,
                     int64_t page_size, void *k_cache, void *v_cache, int64_t n_pages,
                     void *q_out, void *k_out, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                     void *stream);
int aq_paged_attn_decode(const void *q, const void *k_cache, const void *v_cache,
                         const int64_t *page_table, int64_t P, int64_t total_len,
                         const int64_t *seq_lens, int64_t page_size,
                         int64_t n_pages, float scale, void *out, int64_t B, int64_t Hq, int64_t Hkv,
                         int64_t D, void *workspace, int64_t workspace_bytes, void *stream);
int64_t aq_paged_attn_decode_workspace_bytes(int64_t B, int64_t Hq, int64_t Hkv, int64_t total_len);

/* aq_rope_kv_write and aq_paged_attn_decode as one call for the usual decode
 * step: the new token sits at position total_len - 1.  Queries are rotated by
 * the workgroups that use them; the new key and value are rotated, stored into
 * their page slot and attended to from registers.  Caches and outputs are the
 * bits the two separate calls give.  freqs must be 16-byte aligned and
 * freqs_stride a multiple of 4 floats (or 0); workspace as for
 * aq_paged_attn_decode. */
int aq_rope_paged_attn_decode(const void *qkv, const float *freqs, int64_t freqs_stride,
                              const int64_t *page_table, int64_t P, int64_t total_len,
                              const int64_t *seq_lens, int64_t page_size, void *k_cache, void *v_cache, int64_t n_pages,
                              float scale, void *out, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                              void *workspace, int64_t workspace_bytes, void *stream);

/* The three rotating entry points above for attention with qk-norm (use_qk_norm: RMSNorm modules q_norm / k_norm
 * over the head dimension, applied to the rotated query and key before the key is cached and the scores are
 * taken: astrai/model/components/attention.py:62-64, 86-89).  q_gain, k_gain: the two norms' weights, bf16 [D],
 * 16-byte aligned; eps their epsilon.  The rotated head (as it would be stored, rounded to bf16) is normalised as
 * y = bf16((x * r) * gain), r = 1 / sqrt(mean(x^2) + eps), with the squares summed in a fixed order (per 8
 * elements in memory order, the chunk sums by a butterfly over the chunk index) so that the prefill and the decode
 * kernels store the same bits.  What is cached is the NORMALISED key, as in the reference; a cache filled with
 * these entry points must be read with them too.  Everything else as in the entry points without the suffix. */
int aq_rope_kv_write_qknorm(const void *qkv, const float *freqs, int64_t freqs_stride,
                            const int64_t *page_table, int64_t P, int64_t pos, int64_t S,
                            int64_t page_size, void *k_cache, void *v_cache, int64_t n_pages,
                            void *q_out, void *k_out, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                            const void *q_gain, const void *k_gain, float eps, void *stream);
int aq_rope_paged_attn_decode_qknorm(const void *qkv, const float *freqs, int64_t freqs_stride,
                                     const int64_t *page_table, int64_t P, int64_t total_len,
                                     const int64_t *seq_lens, int64_t page_size, void *k_cache, void *v_cache,
                                     int64_t n_pages, float scale, void *out, int64_t B, int64_t Hq, int64_t Hkv,
                                     int64_t D, const void *q_gain, const void *k_gain, float eps,
                                     void *workspace, int64_t workspace_bytes, void *stream);

/* The decode step's attention and output projection without the merge launch
 * in between.  aq_paged_attn_decode_partials / aq_rope_paged_attn_decode_partials
 * are the two calls above stopped before their slices are combined: `partials`
 * (16-byte aligned, at least aq_paged_attn_decode_partials_bytes(B, Hq,
 * total_len) bytes; needed for one slice too) receives, for every (sequence,
 * query head, slice), D numerators, the slice's maximum (log2 domain), its
 * denominator and 2 floats of padding: [B, Hq, n_slices, D + 4] fp32 with
 * n_slices = aq_paged_attn_decode_slices(total_len).
 * aq_gemv_w8a8_decode_attn is aq_gemv_w8a8_decode_residual (attention.py:108,
 * o_proj, plus decoder_block.py:53's add when residual is given) with the rows
 * [M = B, K = Hq * D] combined from those partial results inside the kernel, by
 * the arithmetic of the merge kernel the other path launches: outputs are the
 * bits of aq_(rope_)paged_attn_decode followed by aq_gemv_w8a8_decode_residual.
 * Limits (the kernel holds every slice of a row in registers): M <= 8, K <=
 * AQ_GEMV_ATTN_MAX_K, n_slices <= AQ_GEMV_ATTN_MAX_SLICES (1024 positions);
 * beyond them AQ_E_RANGE, and the caller takes the three-launch path. */
#define AQ_GEMV_ATTN_MAX_K 2048
#define AQ_GEMV_ATTN_MAX_SLICES 4
int64_t aq_paged_attn_decode_slices(int64_t total_len);
int64_t aq_paged_attn_decode_partials_bytes(int64_t B, int64_t Hq, int64_t total_len);
int aq_paged_attn_decode_partials(const void *q, const void *k_cache, const void *v_cache,
                                  const int64_t *page_table, int64_t P, int64_t total_len,
                                  const int64_t *seq_lens, int64_t page_size, int64_t n_pages, float scale, int64_t B,
                                  int64_t Hq, int64_t Hkv, int64_t D, void *partials,
                                  int64_t partials_bytes, void *stream);
int aq_rope_paged_attn_decode_partials(const void *qkv, const float *freqs, int64_t freqs_stride,
                                       const int64_t *page_table, int64_t P, int64_t total_len,
                                       const int64_t *seq_lens, int64_t page_size, void *k_cache, void *v_cache,
                                       int64_t n_pages, float scale, int64_t B, int64_t Hq,
                                       int64_t Hkv, int64_t D, void *partials,
                                       int64_t partials_bytes, void *stream);
/* aq_rope_paged_attn_decode_partials with qk-norm (see aq_rope_paged_attn_decode_qknorm). */
int aq_rope_paged_attn_decode_partials_qknorm(const void *qkv, const float *freqs, int64_t freqs_stride,
                                              const int64_t *page_table, int64_t P, int64_t total_len,
                                              const int64_t *seq_lens, int64_t page_size, void *k_cache,
                                              void *v_cache, int64_t n_pages, float scale, int64_t B, int64_t Hq,
                                              int64_t Hkv, int64_t D, const void *q_gain, const void *k_gain,
                                              float eps, void *partials, int64_t partials_bytes, void *stream);
int aq_gemv_w8a8_decode_attn(const float *partials, int64_t n_slices, int64_t head_dim,
                             const int8_t *wq, const float *sw, const void *bias, int bias_dtype,
                             const void *residual, void *y, int y_dtype, int64_t M, int64_t N,
                             int64_t K, void *stream);

/* Causal self-attention over a prompt, for a prefill that starts from an empty
 * cache (query and key positions coincide): out[b, s, h, :] =
 * softmax_{t <= s}(scale * q[b,s,h] . k[b,t,h/G]) v[b,t,h/G], G = Hq / Hkv.
 * Replaces repeat_kv (attention.py:15-23) + scaled_dot_product_attention with
 * is_causal (attention.py:93-100) for that case, without repeating heads.
 * Element (b, s, h, d) of q sits at q + (b*S + s)*q_stride + h*D + d, likewise
 * k and v with their own token strides (elements, multiples of 8) -- so v can be
 * read in place from the fused q/k/v projection's output; out is [B, S, Hq, D].
 * bf16, D = 64 or 128, fp32 scores and sums on the matrix core; results within
 * bf16 rounding of the reference flow (probabilities are rounded to bf16 before
 * they multiply V, as flash-attention kernels do). */
int aq_prefill_attn_causal(const void *q, int64_t q_stride, const void *k, int64_t k_stride,
                           const void *v, int64_t v_stride, void *out, float scale, int64_t B,
                           int64_t S, int64_t Hq, int64_t Hkv, int64_t D, void *stream);

/* The same attention for a chunk of S new tokens on top of `start` cached ones (a
 * prompt whose prefix was found in the cache, executor.py:32-57 with start_pos > 0):
 * query s of sequence b sits at position start + s and attends to positions
 * 0 .. start + s.  Keys and values of ALL start + S positions are read in place
 * through page_table [B, P] from k_cache / v_cache [n_pages, page_size, Hkv, D] --
 * the new tokens' rows must have been written first (aq_rope_kv_write) -- which
 * replaces Storage.gather (cache.py:254-274) + repeat_kv + scaled_dot_product_attention
 * with the explicit position mask of transformer.py:17-46 when no token is padding.
 * Positions whose page is unmapped count as zero keys and values (gather's zero
 * fill).  start = 0 gives aq_prefill_attn_causal's result on cached rows.
 * start + S <= P * page_size. */
int aq_prefill_attn_paged(const void *q, int64_t q_stride, const void *k_cache, const void *v_cache,
                          const int64_t *page_table, int64_t P, int64_t start, int64_t page_size,
                          int64_t n_pages, void *out, float scale, int64_t B, int64_t S, int64_t Hq,
                          int64_t Hkv, int64_t D, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* ASTRAI_Q_H */
