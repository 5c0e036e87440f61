/*
 * CPU oracle for the quantized-Linear path.  TEST INFRASTRUCTURE ONLY: it is
 * the checker the HIP kernels are compared against and the "port" CPU baseline
 * that the benchmark times; nothing that ships calls into it.
 *
 * What it restates.  The reference's Linear layer is a plain float
 * y = x @ W^T (+ b)  (astrai/model/components/linear.py:20-21, weight laid out
 * [out_dim, in_dim] at linear.py:10).  The reference holds no quantized
 * arithmetic, so the int8 / FP8 arithmetic below is the textbook symmetric
 * absmax scheme, frozen here and implemented a second time in HIP:
 *
 *   int8, per row r of an [R, K] matrix, all in IEEE fp32:
 *     amax_r = max_k |a_rk|;  s_r = amax_r / 127  (s_r = 1 when amax_r == 0)
 *     q_rk   = clamp(rint(a_rk / s_r), -127, 127)      rint = half-to-even,
 *                                                      '/' = true fp32 divide
 *   accumulate: acc[m,n] = sum_k xq[m,k] * wq[n,k]  in int32 (exact)
 *   epilogue:   y = (float(acc) * sx[m]) * sw[n] (+ bias[n]), each operation a
 *               separately rounded fp32 op (no FMA), then one RNE cast.
 *   FP8 (OCP e4m3fn, max 448), per tensor:
 *     s = amax / 448 (s = 1 when amax == 0);  a8 = e4m3fn_rne(clamp(a/s, +-448))
 *     acc in fp32, k ascending;  y = (acc * sx) * sw.
 *
 * Pinning status (tests/test_oracle_*.py):
 *   oq_gemm_i8_i32        pinned: exact integer identity vs torch._int_mm and
 *                         numpy int64 matmul, extreme +-127 cases.
 *   oq_f32_to_e4m3fn      pinned: element-for-element vs torch's
 *   oq_e4m3fn_to_f32      float8_e4m3fn cast over every code, every midpoint
 *                         between codes and a dense random sweep.
 *   oq_f32_to_bf16        pinned: vs torch's bfloat16 cast incl. ties.
 *   oq_quant_rowwise_i8   pinned by mathematics: exact-rational brute force on
 *                         small inputs (python fractions, correctly rounded
 *                         divide, ties-to-even), constructed tie cases,
 *                         invariants (max|q| = 127, zero rows, sign symmetry,
 *                         |a - q s| <= s/2).  No reference vector exists for it:
 *                         "parity unpinned" with respect to the reference.
 *   oq_dequant_epilogue   pinned: vs numpy float32 elementwise arithmetic and,
 *   oq_linear_w8a8        end to end, vs F.linear in fp32 (the reference's real
 *                         path) within the quantisation-error bound.
 *   oq_quant_tensor_fp8,  pinned through the cast above plus numpy float32
 *   oq_linear_fp8         restatement; accumulation order makes the GEMM a
 *                         tolerance (1e-2) comparison, never bit-exact.
 *
 *   oq_one_step_divide_mismatches   not a restatement: an exhaustive evaluation of a shortcut
 *                         the HIP quantisers take on bf16 rows, against the divide itself.
 *
 *   oq_rmsnorm_quant_i8   the norm itself restates F.rms_norm (norm.py:14-15) with a
 *                         fixed summation order; pinned against float64 and torch's
 *                         F.rms_norm within rounding, against the numpy restatement
 *                         bit for bit, and on closed forms (constant rows, unit gain).
 *                         Its quantisation half is oq_quant_rowwise_i8 above.
 *   oq_swiglu_quant_i8    up * silu(gate) (mlp.py:25-26) with an exponential built from
 *                         fused multiply-adds only; pinned against float64 / libm and
 *                         torch's F.silu within rounding, against the numpy
 *                         restatement bit for bit (numpy has no fma: the comparison
 *                         runs the polynomial in float64 products rounded once, which
 *                         is what an fma is), and on closed forms (g = 0, large |g|).
 *   oq_rope_kv_write_qknorm  the RMSNorm of the rotated heads (attention.py:86-89), pinned against
 *                         F.rms_norm applied to oq_rope_kv_write's heads (within one bf16
 *                         step), against an independent numpy restatement bit for bit,
 *                         and on closed forms (constant heads, unit gain, v untouched).
 *   oq_rope_kv_write,     restate apply_rotary_emb (rope.py:26-33), Storage.write / gather
 *   oq_paged_attn_decode  (cache.py:216-274), repeat_kv and softmax attention
 *                         (attention.py:15-23,93-103) for one new token per sequence;
 *                         pinned against torch (complex multiply, index writes,
 *                         scaled_dot_product_attention in fp32) within rounding.
 *   oq_prefill_attn_causal the same attention for a whole prompt (is_causal=True);
 *                         pinned against torch's scaled_dot_product_attention in fp32
 *                         (enable_gqa and explicit repeats) within rounding, and on
 *                         closed forms (first position = its own value row; equal keys
 *                         = running mean of the values).
 *   oq_prefill_attn_offset the same with the queries at positions start .. start + S over
 *                         start + S keys; start = 0 must reproduce oq_prefill_attn_causal
 *                         bit for bit, and it is pinned against torch's attention with the
 *                         explicit position mask.
 *
 * Build: gcc -O3 -march=native -fopenmp -ffp-contract=off -fno-fast-math
 *        -shared -fPIC (oracle/build_oracle.py).  OpenMP only parallelises over
 *        rows; every row's arithmetic is the scalar definition above.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>
#include <stdlib.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int oq_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void oq_set_num_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/* ---------------------------------------------------------------- scalars */

static inline float bits_to_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint32_t f32_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

float oq_bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

/* fp32 -> bf16, round to nearest even; NaN stays a quiet NaN. */
uint16_t oq_f32_to_bf16(float f) {
  uint32_t u = f32_to_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}

/* OCP e4m3fn: 1 sign, 4 exponent (bias 7), 3 mantissa; no infinities; only
 * S.1111.111 is NaN; largest finite 448 = 0x7e; subnormal step 2^-9. */
float oq_e4m3fn_to_f32(uint8_t b) {
  int sign = b >> 7, e = (b >> 3) & 0xf, m = b & 7;
  float v;
  if (e == 0xf && m == 7) return bits_to_f32(0x7fc00000u);
  if (e == 0)
    v = ldexpf((float)m, -9);
  else
    v = ldexpf((float)(8 + m), e - 10);
  return sign ? -v : v;
}

/* fp32 -> e4m3fn, round to nearest even.  Finite inputs beyond the range
 * saturate to +-448 and NaN gives 0x7f; callers clamp first, so saturation is
 * never what a test depends on. */
uint8_t oq_f32_to_e4m3fn(float f) {
  uint32_t u = f32_to_bits(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  uint32_t au = u & 0x7fffffffu;
  if (au > 0x7f800000u) return (uint8_t)(sign | 0x7f);
  float a = bits_to_f32(au);
  if (a >= 464.0f) return (uint8_t)(sign | 0x7e); /* 464 = midpoint past 448 */
  if (a < 0.015625f) {                            /* below 2^-6: subnormal grid 2^-9 */
    float r = rintf(a * 512.0f);                  /* exact scaling, RNE */
    return (uint8_t)(sign | (uint8_t)r);          /* r == 8 lands on 0x08 = 2^-6 */
  }
  int e;
  float fr = frexpf(a, &e); /* a = fr * 2^e, fr in [0.5,1) */
  /* a = (2 fr) * 2^(e-1); mantissa grid 1/8 on [1,2) */
  float m = rintf(fr * 16.0f); /* in [8,16] */
  int E = e - 1;
  if (m == 16.0f) {
    m = 8.0f;
    E += 1;
  }
  int be = E + 7;
  uint8_t code = (uint8_t)((be << 3) | ((int)m - 8));
  if (code > 0x7e) code = 0x7e;
  return (uint8_t)(sign | code);
}

/* ------------------------------------------------ int8 row-wise quantise */

static void quant_row_f32(const float *a, int64_t K, int8_t *q, float *s_out) {
  float amax = 0.0f;
  for (int64_t k = 0; k < K; ++k) {
    float v = fabsf(a[k]);
    if (v > amax) amax = v;
  }
  float s = amax / 127.0f;
  if (amax == 0.0f) s = 1.0f;
  for (int64_t k = 0; k < K; ++k) {
    float r = rintf(a[k] / s);
    if (r > 127.0f) r = 127.0f;
    if (r < -127.0f) r = -127.0f;
    q[k] = (int8_t)r;
  }
  *s_out = s;
}

/* x: [M, K] fp32 with row stride ldx (elements); q: [M, K] contiguous. */
void oq_quant_rowwise_i8_f32(const float *x, int64_t M, int64_t K, int64_t ldx,
                             int8_t *q, float *scale) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) quant_row_f32(x + m * ldx, K, q + m * K, scale + m);
}

/* Same with bf16 input: each element is widened to fp32 first (exact). */
void oq_quant_rowwise_i8_bf16(const uint16_t *x, int64_t M, int64_t K, int64_t ldx,
                              int8_t *q, float *scale) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    float *tmp = (float *)malloc((size_t)K * sizeof(float));
    for (int64_t k = 0; k < K; ++k) tmp[k] = oq_bf16_to_f32(x[m * ldx + k]);
    quant_row_f32(tmp, K, q + m * K, scale + m);
    free(tmp);
  }
}

/* --------------------------------------------- RMSNorm -> row-wise quantise */

/* y = x * (1 / sqrt(mean(x^2) + eps)) * gamma  (F.rms_norm with a gain:
 * astrai/model/components/norm.py:14-15), then quantised per row like any other
 * fp32 row.  The sum of squares has a fixed order: the row is cut into vectors
 * of `epv` consecutive elements (16 bytes of the input: 4 fp32 or 8 bf16);
 * stripe l = v % 64 adds the rounded products x*x of its vectors in ascending
 * order, elements in memory order; the 64 stripe sums are combined by the
 * butterfly p[l] = p[l] + p[l ^ off], off = 1, 2, 4, 8, 16, 32. */
static void rmsnorm_row(const float *a, const float *g, float eps, int64_t K, int epv, float *y) {
  float p[64], t[64];
  for (int l = 0; l < 64; ++l) p[l] = 0.0f;
  const int64_t nvec = K / epv;
  for (int64_t v = 0; v < nvec; ++v) {
    const int l = (int)(v % 64);
    for (int e = 0; e < epv; ++e) {
      const float x = a[v * epv + e];
      const float sq = x * x;
      p[l] = p[l] + sq;
    }
  }
  for (int off = 1; off < 64; off <<= 1) {
    for (int l = 0; l < 64; ++l) t[l] = p[l] + p[l ^ off];
    for (int l = 0; l < 64; ++l) p[l] = t[l];
  }
  const float mean = p[0] / (float)K;
  const float r = 1.0f / sqrtf(mean + eps);
  for (int64_t k = 0; k < K; ++k) {
    const float xr = a[k] * r;
    y[k] = xr * g[k];
  }
}

/* x: [M, K] fp32 (row stride ldx), gamma: [K] fp32; y_out (optional) receives the
 * normalised rows in fp32. */
void oq_rmsnorm_quant_i8_f32(const float *x, const float *gamma, float eps, int64_t M, int64_t K,
                             int64_t ldx, int8_t *q, float *scale, float *y_out) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    float *y = (float *)malloc((size_t)K * sizeof(float));
    rmsnorm_row(x + m * ldx, gamma, eps, K, 4, y);
    quant_row_f32(y, K, q + m * K, scale + m);
    if (y_out) memcpy(y_out + m * K, y, (size_t)K * sizeof(float));
    free(y);
  }
}

/* bf16 input and gain, widened to fp32 first (exact); vectors are 8 elements. */
void oq_rmsnorm_quant_i8_bf16(const uint16_t *x, const uint16_t *gamma, float eps, int64_t M,
                              int64_t K, int64_t ldx, int8_t *q, float *scale, float *y_out) {
  float *g = (float *)malloc((size_t)K * sizeof(float));
  for (int64_t k = 0; k < K; ++k) g[k] = oq_bf16_to_f32(gamma[k]);
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    float *a = (float *)malloc((size_t)K * 2 * sizeof(float));
    float *y = a + K;
    for (int64_t k = 0; k < K; ++k) a[k] = oq_bf16_to_f32(x[m * ldx + k]);
    rmsnorm_row(a, g, eps, K, 8, y);
    quant_row_f32(y, K, q + m * K, scale + m);
    if (y_out) memcpy(y_out + m * K, y, (size_t)K * sizeof(float));
    free(a);
  }
  free(g);
}

/* ------------------------------------------------ SwiGLU -> row-wise quantise */

/* exp(x) for |x| <= 87 from operations that round identically everywhere:
 * n = rint(x log2 e), r = x - n ln 2 in two pieces, e^r = 1 + r + r^2 P(r), then
 * the exponent field is advanced by n. */
float oq_exp_repro(float x) {
  if (x < -87.0f) x = -87.0f;
  if (x > 87.0f) x = 87.0f;
  const float t = x * 1.44269504088896341f;
  const float n = rintf(t);
  float r = fmaf(n, -0.693359375f, x);
  r = fmaf(n, 2.12194440e-4f, r);
  float p = 1.9875691500e-4f;
  p = fmaf(p, r, 1.3981999507e-3f);
  p = fmaf(p, r, 8.3334519073e-3f);
  p = fmaf(p, r, 4.1665795894e-2f);
  p = fmaf(p, r, 1.6666665459e-1f);
  p = fmaf(p, r, 5.0000001201e-1f);
  const float rr = r * r;
  const float y = fmaf(p, rr, r) + 1.0f;
  return bits_to_f32((uint32_t)((int32_t)f32_to_bits(y) + ((int32_t)n << 23)));
}

float oq_swiglu(float u, float g) {
  const float e = oq_exp_repro(-g);
  const float d = 1.0f + e;
  const float sg = g / d;
  return u * sg;
}

/* ug: [M, 2F] (row stride ld), columns [0,F) = up, [F,2F) = gate; codes [M, F]. */
void oq_swiglu_quant_i8_f32(const float *ug, int64_t M, int64_t F, int64_t ld, int8_t *q,
                            float *scale, float *h_out) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    float *h = (float *)malloc((size_t)F * sizeof(float));
    for (int64_t k = 0; k < F; ++k) h[k] = oq_swiglu(ug[m * ld + k], ug[m * ld + F + k]);
    quant_row_f32(h, F, q + m * F, scale + m);
    if (h_out) memcpy(h_out + m * F, h, (size_t)F * sizeof(float));
    free(h);
  }
}

void oq_swiglu_quant_i8_bf16(const uint16_t *ug, int64_t M, int64_t F, int64_t ld, int8_t *q,
                             float *scale, float *h_out) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    float *h = (float *)malloc((size_t)F * sizeof(float));
    for (int64_t k = 0; k < F; ++k)
      h[k] = oq_swiglu(oq_bf16_to_f32(ug[m * ld + k]), oq_bf16_to_f32(ug[m * ld + F + k]));
    quant_row_f32(h, F, q + m * F, scale + m);
    if (h_out) memcpy(h_out + m * F, h, (size_t)F * sizeof(float));
    free(h);
  }
}

/* ------------------------------------------- decode attention over paged KV */

/* One new token per sequence at logical position pos.  qkv: [B, (Hq+2Hkv)*D] bf16,
 * q heads then k heads then v heads; freqs: [B, D/2, 2] (cos, sin).  Interleaved
 * pairs are rotated in fp32 -- (x0 + i x1)(c + i s), products and sums rounded
 * one by one -- and cast to bf16 (rope.py:26-33).  q goes to q_out [B, Hq, D]; k
 * and v go to slot pos % page of page table[b, pos / page] of the caches
 * [n_pages, page, Hkv, D]; sequences whose page is unmapped are skipped
 * (cache.py:216-252). */
static void rope_kv_write(const uint16_t *qkv, const float *freqs, const int64_t *table, int64_t P,
                          int64_t pos, int64_t page, uint16_t *kc, uint16_t *vc, int64_t n_pages,
                          uint16_t *q_out, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                          const uint16_t *q_gain, const uint16_t *k_gain, float eps) {
  const int64_t heads = Hq + 2 * Hkv;
  for (int64_t b = 0; b < B; ++b) {
    const int64_t lp = pos / page;
    const int64_t phys = lp < P ? table[b * P + lp] : -1;
    for (int64_t h = 0; h < heads; ++h) {
      const uint16_t *src = qkv + (b * heads + h) * D;
      uint16_t tmp[1024];
      for (int64_t i = 0; i < D / 2; ++i) {
        if (h < Hq + Hkv) {
          const float x0 = oq_bf16_to_f32(src[2 * i]), x1 = oq_bf16_to_f32(src[2 * i + 1]);
          const float c = freqs[(b * (D / 2) + i) * 2], sn = freqs[(b * (D / 2) + i) * 2 + 1];
          const float a = x0 * c, bb = x1 * sn, cc = x0 * sn, dd = x1 * c;
          tmp[2 * i] = oq_f32_to_bf16(a - bb);
          tmp[2 * i + 1] = oq_f32_to_bf16(cc + dd);
        } else {
          tmp[2 * i] = src[2 * i];
          tmp[2 * i + 1] = src[2 * i + 1];
        }
      }
      if (q_gain && h < Hq + Hkv) {
        /* RMSNorm over the head (attention.py:62-64, 86-89; norm.py:14-15), on the rotated head as bf16 holds
         * it: y = bf16((x * r) * gain), r = 1 / sqrt(sum / D + eps).  The squares are summed per 8 elements in
         * memory order, those sums pairwise over the chunk index (c, c ^ 1, then ^ 2, ^ 4, ^ 8). */
        const uint16_t *gain = h < Hq ? q_gain : k_gain;
        float part[128];
        int64_t n = D / 8;
        for (int64_t c = 0; c < n; ++c) {
          float acc = 0.0f;
          for (int64_t e = 0; e < 8; ++e) {
            const float x = oq_bf16_to_f32(tmp[c * 8 + e]);
            const float sq = x * x;
            acc = acc + sq;
          }
          part[c] = acc;
        }
        for (; n > 1; n /= 2)
          for (int64_t c = 0; c < n / 2; ++c) part[c] = part[2 * c] + part[2 * c + 1];
        const float mean = part[0] / (float)D;
        const float r = 1.0f / sqrtf(mean + eps);
        for (int64_t i = 0; i < D; ++i) {
          const float xr = oq_bf16_to_f32(tmp[i]) * r;
          tmp[i] = oq_f32_to_bf16(xr * oq_bf16_to_f32(gain[i]));
        }
      }
      if (h < Hq) {
        memcpy(q_out + (b * Hq + h) * D, tmp, (size_t)D * 2);
      } else if (phys >= 0 && phys < n_pages) {
        const int is_k = h < Hq + Hkv;
        const int64_t kvh = is_k ? h - Hq : h - Hq - Hkv;
        uint16_t *dst = (is_k ? kc : vc) + ((phys * page + pos % page) * Hkv + kvh) * D;
        memcpy(dst, tmp, (size_t)D * 2);
      }
    }
  }
}

void oq_rope_kv_write(const uint16_t *qkv, const float *freqs, const int64_t *table, int64_t P,
                      int64_t pos, int64_t page, uint16_t *kc, uint16_t *vc, int64_t n_pages,
                      uint16_t *q_out, int64_t B, int64_t Hq, int64_t Hkv, int64_t D) {
  rope_kv_write(qkv, freqs, table, P, pos, page, kc, vc, n_pages, q_out, B, Hq, Hkv, D, NULL, NULL, 0.0f);
}

/* oq_rope_kv_write for attention with qk-norm: the rotated q and k heads go through RMSNorm modules over D
 * (gains bf16 [D]) before q is returned and k is cached; v is untouched. */
void oq_rope_kv_write_qknorm(const uint16_t *qkv, const float *freqs, const int64_t *table, int64_t P,
                             int64_t pos, int64_t page, uint16_t *kc, uint16_t *vc, int64_t n_pages,
                             uint16_t *q_out, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                             const uint16_t *q_gain, const uint16_t *k_gain, float eps) {
  rope_kv_write(qkv, freqs, table, P, pos, page, kc, vc, n_pages, q_out, B, Hq, Hkv, D, q_gain, k_gain, eps);
}

/* out[b, h, :] = softmax_t(scale * q[b,h] . K[b,t,h/G]) V[b,t,h/G], t < T, read through
 * the page table; unmapped pages are zero keys and values (cache.py:254-274 zero
 * fill).  lens (may be NULL): positions t >= lens[b] of sequence b carry the mask value that
 * process_attention_mask (transformer.py:17-46) puts on positions past position_ids[b]
 * (lens[b] = position_ids[b] + 1).  fp32, t and d ascending, libm expf. */
void oq_paged_attn_decode(const uint16_t *q, const uint16_t *kc, const uint16_t *vc,
                          const int64_t *table, int64_t P, int64_t T, const int64_t *lens, int64_t page,
                          int64_t n_pages, float scale, uint16_t *out, int64_t B, int64_t Hq, int64_t Hkv,
                          int64_t D) {
  const int64_t G = Hq / Hkv;
#pragma omp parallel for schedule(static) collapse(2)
  for (int64_t b = 0; b < B; ++b)
    for (int64_t h = 0; h < Hq; ++h) {
      const int64_t kvh = h / G;
      float *s = (float *)malloc((size_t)T * sizeof(float));
      float *acc = (float *)calloc((size_t)D, sizeof(float));
      float m = -INFINITY;
      for (int64_t t = 0; t < T; ++t) {
        const int64_t lp = t / page;
        const int64_t phys = lp < P ? table[b * P + lp] : -1;
        float d = 0.0f;
        if (phys >= 0 && phys < n_pages) {
          const uint16_t *k = kc + ((phys * page + t % page) * Hkv + kvh) * D;
          for (int64_t i = 0; i < D; ++i) d += oq_bf16_to_f32(q[(b * Hq + h) * D + i]) * oq_bf16_to_f32(k[i]);
        }
        s[t] = d * scale;
        /* a sequence shorter than T: the additive mask of transformer.py:40-46, -finfo(bfloat16).max / 2
         * on every position past the sequence's own */
        if (lens && t >= lens[b]) s[t] += -1.6947656946257676e38f;
        if (s[t] > m) m = s[t];
      }
      float l = 0.0f;
      for (int64_t t = 0; t < T; ++t) {
        const float pt = expf(s[t] - m);
        l += pt;
        const int64_t lp = t / page;
        const int64_t phys = lp < P ? table[b * P + lp] : -1;
        if (phys >= 0 && phys < n_pages) {
          const uint16_t *v = vc + ((phys * page + t % page) * Hkv + kvh) * D;
          for (int64_t i = 0; i < D; ++i) acc[i] += pt * oq_bf16_to_f32(v[i]);
        }
      }
      for (int64_t i = 0; i < D; ++i) out[(b * Hq + h) * D + i] = oq_f32_to_bf16(acc[i] / l);
      free(s);
      free(acc);
    }
}

/* Causal self-attention over a prompt: out[b, s, h, :] = softmax_{t <= s}(scale * q[b,s,h] . k[b,t,h/G])
 * v[b,t,h/G] -- repeat_kv + scaled_dot_product_attention(is_causal=True) of attention.py:15-23,93-100 when
 * query and key positions coincide.  q: [B, S, Hq, D], k, v: [B, S, Hkv, D] bf16 bit patterns; fp32, t and d
 * ascending, libm expf. */
void oq_prefill_attn_causal(const uint16_t *q, const uint16_t *k, const uint16_t *v, float scale, uint16_t *out,
                            int64_t B, int64_t S, int64_t Hq, int64_t Hkv, int64_t D) {
  const int64_t G = Hq / Hkv;
#pragma omp parallel for schedule(dynamic) collapse(3)
  for (int64_t b = 0; b < B; ++b)
    for (int64_t h = 0; h < Hq; ++h)
      for (int64_t s = 0; s < S; ++s) {
        const int64_t kvh = h / G;
        const uint16_t *qr = q + ((b * S + s) * Hq + h) * D;
        float *sc = (float *)malloc((size_t)(s + 1) * sizeof(float));
        float *acc = (float *)calloc((size_t)D, sizeof(float));
        float m = -INFINITY;
        for (int64_t t = 0; t <= s; ++t) {
          const uint16_t *kr = k + ((b * S + t) * Hkv + kvh) * D;
          float d = 0.0f;
          for (int64_t i = 0; i < D; ++i) d += oq_bf16_to_f32(qr[i]) * oq_bf16_to_f32(kr[i]);
          sc[t] = d * scale;
          if (sc[t] > m) m = sc[t];
        }
        float l = 0.0f;
        for (int64_t t = 0; t <= s; ++t) {
          const float pt = expf(sc[t] - m);
          l += pt;
          const uint16_t *vr = v + ((b * S + t) * Hkv + kvh) * D;
          for (int64_t i = 0; i < D; ++i) acc[i] += pt * oq_bf16_to_f32(vr[i]);
        }
        for (int64_t i = 0; i < D; ++i) out[((b * S + s) * Hq + h) * D + i] = oq_f32_to_bf16(acc[i] / l);
        free(sc);
        free(acc);
      }
}

/* The same with the S queries at positions start .. start + S over T = start + S keys: query s attends to
 * t <= start + s (the explicit position mask of transformer.py:17-46 for a chunk on top of cached tokens,
 * executor.py:32-57 with start_pos > 0).  q: [B, S, Hq, D], k, v: [B, T, Hkv, D]. */
void oq_prefill_attn_offset(const uint16_t *q, const uint16_t *k, const uint16_t *v, float scale, uint16_t *out,
                            int64_t B, int64_t S, int64_t start, int64_t Hq, int64_t Hkv, int64_t D) {
  const int64_t G = Hq / Hkv, T = start + S;
#pragma omp parallel for schedule(dynamic) collapse(3)
  for (int64_t b = 0; b < B; ++b)
    for (int64_t h = 0; h < Hq; ++h)
      for (int64_t s = 0; s < S; ++s) {
        const int64_t kvh = h / G, last = start + s;
        const uint16_t *qr = q + ((b * S + s) * Hq + h) * D;
        float *sc = (float *)malloc((size_t)(last + 1) * sizeof(float));
        float *acc = (float *)calloc((size_t)D, sizeof(float));
        float m = -INFINITY;
        for (int64_t t = 0; t <= last; ++t) {
          const uint16_t *kr = k + ((b * T + t) * Hkv + kvh) * D;
          float d = 0.0f;
          for (int64_t i = 0; i < D; ++i) d += oq_bf16_to_f32(qr[i]) * oq_bf16_to_f32(kr[i]);
          sc[t] = d * scale;
          if (sc[t] > m) m = sc[t];
        }
        float l = 0.0f;
        for (int64_t t = 0; t <= last; ++t) {
          const float pt = expf(sc[t] - m);
          l += pt;
          const uint16_t *vr = v + ((b * T + t) * Hkv + kvh) * D;
          for (int64_t i = 0; i < D; ++i) acc[i] += pt * oq_bf16_to_f32(vr[i]);
        }
        for (int64_t i = 0; i < D; ++i) out[((b * S + s) * Hq + h) * D + i] = oq_f32_to_bf16(acc[i] / l);
        free(sc);
        free(acc);
      }
}

/* ------------------------------------------------------------- int8 GEMM */

/* acc[m,n] = sum_k xq[m,k] * wq[n,k]; both operands K-contiguous, the layout
 * of Linear.weight (linear.py:10). */
void oq_gemm_i8_i32(const int8_t *xq, const int8_t *wq, int32_t *acc, int64_t M,
                    int64_t N, int64_t K) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    const int8_t *xr = xq + m * K;
    for (int64_t n = 0; n < N; ++n) {
      const int8_t *wr = wq + n * K;
      int32_t s = 0;
      for (int64_t k = 0; k < K; ++k) s += (int32_t)xr[k] * (int32_t)wr[k];
      acc[m * N + n] = s;
    }
  }
}

/* y = (float(acc) * sx[m]) * sw[n] (+ bias[n]) in fp32, three separately
 * rounded operations.  y_bf16 may be NULL; y_f32 may be NULL. */
void oq_dequant_epilogue(const int32_t *acc, const float *sx, const float *sw,
                         const float *bias, float *y_f32, uint16_t *y_bf16,
                         int64_t M, int64_t N) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      volatile float t = (float)acc[m * N + n] * sx[m];
      volatile float u = t * sw[n];
      float y = u;
      if (bias) {
        volatile float w = u + bias[n];
        y = w;
      }
      if (y_f32) y_f32[m * N + n] = y;
      if (y_bf16) y_bf16[m * N + n] = oq_f32_to_bf16(y);
    }
  }
}

/* Whole W8A8 Linear from float inputs: quantise x per token, GEMM, epilogue.
 * wq/sw are the already-quantised weight.  Scratch is allocated here. */
void oq_linear_w8a8_f32(const float *x, const int8_t *wq, const float *sw,
                        const float *bias, float *y_f32, uint16_t *y_bf16, int64_t M,
                        int64_t N, int64_t K) {
  int8_t *xq = (int8_t *)malloc((size_t)(M * K));
  float *sx = (float *)malloc((size_t)M * sizeof(float));
  int32_t *acc = (int32_t *)malloc((size_t)(M * N) * sizeof(int32_t));
  oq_quant_rowwise_i8_f32(x, M, K, K, xq, sx);
  oq_gemm_i8_i32(xq, wq, acc, M, N, K);
  oq_dequant_epilogue(acc, sx, sw, bias, y_f32, y_bf16, M, N);
  free(xq);
  free(sx);
  free(acc);
}

void oq_linear_w8a8_bf16(const uint16_t *x, const int8_t *wq, const float *sw,
                         const float *bias, float *y_f32, uint16_t *y_bf16, int64_t M,
                         int64_t N, int64_t K) {
  int8_t *xq = (int8_t *)malloc((size_t)(M * K));
  float *sx = (float *)malloc((size_t)M * sizeof(float));
  int32_t *acc = (int32_t *)malloc((size_t)(M * N) * sizeof(int32_t));
  oq_quant_rowwise_i8_bf16(x, M, K, K, xq, sx);
  oq_gemm_i8_i32(xq, wq, acc, M, N, K);
  oq_dequant_epilogue(acc, sx, sw, bias, y_f32, y_bf16, M, N);
  free(xq);
  free(sx);
  free(acc);
}

/* -------------------------------------------------------------------- FP8 */

static float amax_f32(const float *x, int64_t n) {
  float amax = 0.0f;
  for (int64_t i = 0; i < n; ++i) {
    float v = fabsf(x[i]);
    if (v > amax) amax = v;
  }
  return amax;
}

static void cast_fp8(const float *x, int64_t n, float s, uint8_t *q) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float v = x[i] / s;
    if (v > 448.0f) v = 448.0f;
    if (v < -448.0f) v = -448.0f;
    q[i] = oq_f32_to_e4m3fn(v);
  }
}

void oq_quant_tensor_fp8_f32(const float *x, int64_t numel, uint8_t *q, float *scale) {
  float amax = amax_f32(x, numel);
  float s = amax / 448.0f;
  if (amax == 0.0f) s = 1.0f;
  cast_fp8(x, numel, s, q);
  *scale = s;
}

void oq_quant_tensor_fp8_bf16(const uint16_t *x, int64_t numel, uint8_t *q, float *scale) {
  float *tmp = (float *)malloc((size_t)numel * sizeof(float));
  for (int64_t i = 0; i < numel; ++i) tmp[i] = oq_bf16_to_f32(x[i]);
  oq_quant_tensor_fp8_f32(tmp, numel, q, scale);
  free(tmp);
}

/*
 * Checker for a shortcut the HIP quantisers take on rows of bf16 numbers (not a restatement of anything in the
 * reference).  The definition above divides, q = fl(a / s); the kernels compute, with rs = fl(1 / s),
 *     q0 = fl(a * rs);  r = fma(-s, q0, a);  q1 = fma(r, rs, q0)
 * (one correction step; in general two are needed) and claim the CODE of q1 equals the code of q whenever a and
 * the maximum the scale comes from are bf16 numbers.  This function evaluates the claim for every bf16 maximum
 * with bit pattern in [am_lo, am_hi) whose scale s = fl(amax / divisor) lies in [2^-64, 2^64] (the range in which
 * the kernels use the shortcut) and every bf16 a with |a| <= amax, both signs, and returns the number of pairs
 * whose codes differ (*pairs = the number evaluated).  divisor 127: code = clamp(rint(.), +-127); divisor 448:
 * code = e4m3fn(clamp(., +-448)) with the quotient given the sign of a (the kernel does that too: a zero residual
 * turns a quotient of -0 into +0).  steps = 0 evaluates q0 alone, which does differ: the check has teeth.
 * steps = -1 (divisor 127) evaluates the int8 kernels' present form for bf16 rows: q0 alone, but with rs moved by
 * one unit in the last place where the 7 mantissa bits of the maximum ask for it (the table below: 0 keep, 1 up,
 * 2 down; two bits per mantissa, sixteen mantissas per word).
 */
static const uint32_t oq_rs_adjust[8] = {0x00000000u, 0x05015a02u, 0x80000000u, 0x10004480u,
                                         0x00000000u, 0x40014442u, 0x40000004u, 0x00000105u};

int64_t oq_one_step_divide_mismatches(float divisor, int steps, uint32_t am_lo, uint32_t am_hi, int64_t *pairs) {
  int64_t bad = 0, n = 0;
  const int fp8 = divisor == 448.0f;
#pragma omp parallel for schedule(dynamic, 16) reduction(+ : bad, n)
  for (uint32_t am = am_lo; am < am_hi; ++am) {
    if (am == 0 || am >= 0x7f80u) continue;
    const float amax = oq_bf16_to_f32((uint16_t)am);
    const float s = amax / divisor;
    if (!(s >= 5.421010862427522e-20f && s <= 1.8446744073709552e19f)) continue;
    float rs = 1.0f / s;
    if (steps < 0) {
      const uint32_t m = am & 127u, adj = (oq_rs_adjust[m >> 4] >> (2u * (m & 15u))) & 3u;
      uint32_t bits;
      memcpy(&bits, &rs, 4);
      bits += (adj & 1u) - (adj >> 1);
      memcpy(&rs, &bits, 4);
    }
    for (uint32_t ab = 0; ab <= am; ++ab) {
      for (int neg = 0; neg < 2; ++neg) {
        const float a = oq_bf16_to_f32((uint16_t)(ab | (neg ? 0x8000u : 0u)));
        const float q = a / s;
        const float q0 = a * rs;
        float q1 = steps > 0 ? fmaf(fmaf(-s, q0, a), rs, q0) : q0;
        ++n;
        if (fp8) {
          q1 = copysignf(q1, a);
          float c0 = q, c1 = q1;
          if (c0 > 448.0f) c0 = 448.0f;
          if (c0 < -448.0f) c0 = -448.0f;
          if (c1 > 448.0f) c1 = 448.0f;
          if (c1 < -448.0f) c1 = -448.0f;
          bad += oq_f32_to_e4m3fn(c0) != oq_f32_to_e4m3fn(c1);
        } else {
          float c0 = rintf(q), c1 = rintf(q1);
          if (c0 > 127.0f) c0 = 127.0f;
          if (c0 < -127.0f) c0 = -127.0f;
          if (c1 > 127.0f) c1 = 127.0f;
          if (c1 < -127.0f) c1 = -127.0f;
          bad += (int)c0 != (int)c1;
        }
      }
    }
  }
  if (pairs) *pairs = n;
  return bad;
}

/* y = (sum_k f(xq[m,k]) f(wq[n,k])) * sx * sw; fp32 accumulate, k ascending. */
void oq_linear_fp8(const uint8_t *xq, float sx, const uint8_t *wq, float sw, const float *bias, float *y_f32,
                   uint16_t *y_bf16, int64_t M, int64_t N, int64_t K) {
  float lut[256];
  for (int i = 0; i < 256; ++i) lut[i] = oq_e4m3fn_to_f32((uint8_t)i);
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    float *xr = (float *)malloc((size_t)K * sizeof(float));
    for (int64_t k = 0; k < K; ++k) xr[k] = lut[xq[m * K + k]];
    for (int64_t n = 0; n < N; ++n) {
      const uint8_t *wr = wq + n * K;
      float s = 0.0f;
      for (int64_t k = 0; k < K; ++k) s += xr[k] * lut[wr[k]];
      volatile float t = s * sx;
      volatile float u = t * sw;
      volatile float v = bias ? u + bias[n] : u;  /* the bias of linear.py:11,21: one more rounded add */
      float y = v;
      if (y_f32) y_f32[m * N + n] = y;
      if (y_bf16) y_bf16[m * N + n] = oq_f32_to_bf16(y);
    }
    free(xr);
  }
}

/* Float reference of the Linear itself (linear.py:20-21): fp32, k ascending. */
void oq_linear_f32(const float *x, const float *w, const float *bias, float *y, int64_t M,
                   int64_t N, int64_t K) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      double s = 0.0;
      for (int64_t k = 0; k < K; ++k) s += (double)x[m * K + k] * (double)w[n * K + k];
      if (bias) s += bias[n];
      y[m * N + n] = (float)s;
    }
}
