// Decode-step attention around the quantized projections, reading the paged KV
// cache in place: the reference gathers every page into a contiguous
// [B, T, Hkv, D] copy, repeats the KV heads and calls a generic attention per
// layer and per step (astrai/model/components/attention.py:83-103,
// astrai/inference/core/cache.py:254-274).  Two kernels replace that for a step
// with one new token per sequence:
//
//   rope_kv_write   rotates q and k of the new token (interleaved pairs, fp32,
//                   rope.py:26-33), stores q, and writes k and v into their page
//                   slot (cache.py:216-252);
//   paged_attn      softmax(q K^T / sqrt(D)) V over the pages of each sequence,
//                   all query heads of a KV head in one workgroup (grouped-query
//                   attention without materialising the repeated heads,
//                   attention.py:15-23).
//
// bf16 tensors, head dimension 128, fp32 arithmetic.  Unmapped pages (table
// entry < 0 or out of range) are skipped on write and read as zero keys and
// values, as the reference's gather does.
#include "aq_common.h"

namespace aq {

constexpr int AD = 128;          // head dimension

struct RopeArgs {
  const uint16_t* qkv;   // [B, (Hq + 2 Hkv) * D]
  const float* freqs;    // [B, D/2, 2] (cos, sin) of the new token's position; sequence stride freqs_stride floats
  int64_t freqs_stride;
  const int64_t* table;  // [B, P]
  uint16_t* kc;          // [n_pages, page, Hkv, D]
  uint16_t* vc;
  uint16_t* q_out;       // [B, Hq, D]
  int64_t P, pos, page, n_pages;
  int B, Hq, Hkv;
};

// one wavefront per head vector: lane l owns the pair (2l, 2l+1)
__global__ __launch_bounds__(64) void rope_kv_write_kernel(RopeArgs p) {
  const int lane = threadIdx.x;
  const int heads = p.Hq + 2 * p.Hkv;
  const int b = blockIdx.x / heads, h = blockIdx.x % heads;
  const uint32_t pair = reinterpret_cast<const uint32_t*>(p.qkv + ((int64_t)b * heads + h) * AD)[lane];
  uint32_t out = pair;
  if (h < p.Hq + p.Hkv) {  // q and k heads rotate, v heads do not
    const float x0 = bf16_bits_to_f32((uint16_t)(pair & 0xffffu)), x1 = bf16_bits_to_f32((uint16_t)(pair >> 16));
    const float2 cs = reinterpret_cast<const float2*>(p.freqs + (int64_t)b * p.freqs_stride)[lane];
    // (x0 + i x1)(c + i s): four rounded products, one rounded difference, one rounded sum
    const float r0 = __fsub_rn(__fmul_rn(x0, cs.x), __fmul_rn(x1, cs.y));
    const float r1 = __fadd_rn(__fmul_rn(x0, cs.y), __fmul_rn(x1, cs.x));
    out = pack_bf16x2(r0, r1);
  }
  if (h < p.Hq) {
    reinterpret_cast<uint32_t*>(p.q_out + ((int64_t)b * p.Hq + h) * AD)[lane] = out;
    return;
  }
  const int64_t lp = p.pos / p.page;
  const int64_t phys = lp < p.P ? p.table[(int64_t)b * p.P + lp] : -1;
  if (phys < 0 || phys >= p.n_pages) return;  // unmapped: the token is dropped, as in the reference
  const bool is_k = h < p.Hq + p.Hkv;
  const int kvh = is_k ? h - p.Hq : h - p.Hq - p.Hkv;
  uint16_t* dst = (is_k ? p.kc : p.vc) + ((phys * p.page + p.pos % p.page) * p.Hkv + kvh) * AD;
  reinterpret_cast<uint32_t*>(dst)[lane] = out;
}

struct AttnArgs {
  const uint16_t* q;     // [B, Hq, D]
  const uint16_t* kc;    // [n_pages, page, Hkv, D]
  const uint16_t* vc;
  const int64_t* table;  // [B, P]
  uint16_t* out;         // [B, Hq, D]
  int64_t P, T, page, n_pages;
  float scale_log2e;     // softmax scale times log2(e): scores live in the exp2 domain
  int B, Hq, Hkv;
};

// Workgroup = one (sequence, KV head): its G query heads share every K and V
// byte.  The T cached positions are cut into batches of 64; wavefront w takes
// batches w, w + ATT_WAVES, ...  In a batch lane l owns key position t0 + l for
// the scores (its 256-byte K row against the G queries held in LDS) and the
// dimension pair (2l, 2l+1) for the weighted sum of V rows.  All of a batch's
// loads -- 16 per lane for K, 64 for V -- are requested before anything is
// computed: with a few dozen workgroups on the device the kernel lives on memory
// latency, not bandwidth.  Each wavefront keeps a running maximum, denominator
// and numerator per head (online softmax); the partial results are merged
// through LDS at the end.
template <int G, int ATT_WAVES>
__global__ __launch_bounds__(ATT_WAVES * 64) void paged_attn_decode_kernel(AttnArgs p) {
  constexpr int ATT_THREADS = ATT_WAVES * 64;
  __shared__ float q_s[G][AD];                       // queries, pre-scaled
  __shared__ float p_s[ATT_WAVES][64][G];            // a batch's probabilities, per wavefront
  __shared__ float m_s[ATT_WAVES][G], l_s[ATT_WAVES][G];
  __shared__ float acc_s[ATT_WAVES][G][AD];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = blockIdx.x / p.Hkv, kvh = blockIdx.x % p.Hkv;

  for (int i = tid; i < G * AD; i += ATT_THREADS) {
    const int g = i / AD, d = i % AD;
    q_s[g][d] = __fmul_rn(bf16_bits_to_f32(p.q[((int64_t)b * p.Hq + kvh * G + g) * AD + d]), p.scale_log2e);
  }
  __syncthreads();

  float m[G], l[G], acc0[G], acc1[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.0f;
    acc0[g] = 0.0f;
    acc1[g] = 0.0f;
  }
  const int64_t T = p.T;
  for (int64_t t0 = (int64_t)wave * 64; t0 < T; t0 += ATT_WAVES * 64) {
    // ---- scores of key t0 + lane
    const int64_t t = t0 + lane;
    int64_t row = -1;  // element offset of this key's row, or -1
    if (t < T) {
      const int64_t lp = t / p.page;
      const int64_t phys = lp < p.P ? p.table[(int64_t)b * p.P + lp] : -1;
      if (phys >= 0 && phys < p.n_pages) row = ((phys * p.page + t % p.page) * p.Hkv + kvh) * AD;
    }
    uint4 kv[AD / 8];
    if (row >= 0) {
      const uint4* src = reinterpret_cast<const uint4*>(p.kc + row);
#pragma unroll
      for (int c = 0; c < AD / 8; ++c) kv[c] = src[c];
    } else {
#pragma unroll
      for (int c = 0; c < AD / 8; ++c) kv[c] = make_uint4(0, 0, 0, 0);
    }
    // the V rows of the whole batch: the row offset of key j sits in lane j
    const int nkeys = (T - t0) < 64 ? (int)(T - t0) : 64;
    uint32_t vv[64];
#pragma unroll
    for (int j = 0; j < 64; ++j) {
      const int lo = __builtin_amdgcn_readlane((int)(uint32_t)row, j), hi = __builtin_amdgcn_readlane((int)(row >> 32), j);
      const int64_t r = ((int64_t)hi << 32) | (uint32_t)lo;  // wavefront-uniform
      vv[j] = (j < nkeys && r >= 0) ? reinterpret_cast<const uint32_t*>(p.vc + r)[lane] : 0u;
    }
    float s[G];
#pragma unroll
    for (int g = 0; g < G; ++g) s[g] = 0.0f;
#pragma unroll
    for (int c = 0; c < AD / 8; ++c) {
      float k8[8];
      k8[0] = __uint_as_float(kv[c].x << 16);
      k8[1] = __uint_as_float(kv[c].x & 0xffff0000u);
      k8[2] = __uint_as_float(kv[c].y << 16);
      k8[3] = __uint_as_float(kv[c].y & 0xffff0000u);
      k8[4] = __uint_as_float(kv[c].z << 16);
      k8[5] = __uint_as_float(kv[c].z & 0xffff0000u);
      k8[6] = __uint_as_float(kv[c].w << 16);
      k8[7] = __uint_as_float(kv[c].w & 0xffff0000u);
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float4 qa = *reinterpret_cast<const float4*>(&q_s[g][c * 8]);
        const float4 qb = *reinterpret_cast<const float4*>(&q_s[g][c * 8 + 4]);
        s[g] = __builtin_fmaf(k8[0], qa.x, s[g]);
        s[g] = __builtin_fmaf(k8[1], qa.y, s[g]);
        s[g] = __builtin_fmaf(k8[2], qa.z, s[g]);
        s[g] = __builtin_fmaf(k8[3], qa.w, s[g]);
        s[g] = __builtin_fmaf(k8[4], qb.x, s[g]);
        s[g] = __builtin_fmaf(k8[5], qb.y, s[g]);
        s[g] = __builtin_fmaf(k8[6], qb.z, s[g]);
        s[g] = __builtin_fmaf(k8[7], qb.w, s[g]);
      }
    }
    // ---- online softmax update, per head
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const float sv = t < T ? s[g] : -INFINITY;
      float bm = sv;
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) bm = fmaxf(bm, __shfl_xor(bm, off, 64));
      const float mn = fmaxf(m[g], bm);  // finite: lane 0 of every batch is a valid position
      const float alpha = exp2f(m[g] - mn);
      const float pv = t < T ? exp2f(sv - mn) : 0.0f;
      float ps = pv;
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) ps += __shfl_xor(ps, off, 64);
      l[g] = l[g] * alpha + ps;
      acc0[g] *= alpha;
      acc1[g] *= alpha;
      m[g] = mn;
      p_s[wave][lane][g] = pv;
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // this wavefront's LDS writes are done (wavefront-private region)
    asm volatile("" ::: "memory");
    // ---- numerator: lane owns dimensions 2l, 2l+1 of every V row of the batch (zero rows and
    // positions past T carry probability-weighted zeros)
#pragma unroll
    for (int j = 0; j < 64; ++j) {
      const float v0 = __uint_as_float(vv[j] << 16), v1 = __uint_as_float(vv[j] & 0xffff0000u);
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float pj = p_s[wave][j][g];
        acc0[g] = __builtin_fmaf(pj, v0, acc0[g]);
        acc1[g] = __builtin_fmaf(pj, v1, acc1[g]);
      }
    }
    asm volatile("" ::: "memory");
  }
  // ---- merge the wavefronts' partial results
#pragma unroll
  for (int g = 0; g < G; ++g) {
    if (lane == 0) {
      m_s[wave][g] = m[g];
      l_s[wave][g] = l[g];
    }
    acc_s[wave][g][2 * lane] = acc0[g];
    acc_s[wave][g][2 * lane + 1] = acc1[g];
  }
  __syncthreads();
  for (int i = tid; i < G * AD; i += ATT_THREADS) {
    const int g = i / AD, d = i % AD;
    float mm = -INFINITY;
#pragma unroll
    for (int w = 0; w < ATT_WAVES; ++w) mm = fmaxf(mm, m_s[w][g]);
    float num = 0.0f, den = 0.0f;
#pragma unroll
    for (int w = 0; w < ATT_WAVES; ++w) {
      const float a = m_s[w][g] == -INFINITY ? 0.0f : exp2f(m_s[w][g] - mm);  // wavefronts without a batch
      num = __builtin_fmaf(acc_s[w][g][d], a, num);
      den = __builtin_fmaf(l_s[w][g], a, den);
    }
    p.out[((int64_t)b * p.Hq + kvh * G + g) * AD + d] = (uint16_t)f32_to_bf16_bits(num / den);
  }
}

}  // namespace aq

extern "C" int aq_rope_kv_write(const void* qkv, const float* freqs, int64_t freqs_stride, const int64_t* page_table, int64_t P,
                                int64_t pos, int64_t page_size, void* k_cache, void* v_cache, int64_t n_pages,
                                void* q_out, int64_t B, int64_t Hq, int64_t Hkv, int64_t D, void* stream) {
  if (D != aq::AD) return AQ_E_SHAPE;
  if (B < 0 || Hq <= 0 || Hkv <= 0 || P <= 0 || pos < 0 || page_size <= 0 || n_pages <= 0) return AQ_E_SHAPE;
  if (freqs_stride != 0 && freqs_stride < D) return AQ_E_SHAPE;
  if (B == 0) return AQ_OK;
  if (!qkv || !freqs || !page_table || !k_cache || !v_cache || !q_out) return AQ_E_NULL;
  if (aq::check_ptr16(qkv) || aq::check_ptr16(k_cache) || aq::check_ptr16(v_cache) || aq::check_ptr16(q_out) ||
      (reinterpret_cast<uintptr_t>(freqs) & 7u) || (freqs_stride & 1))
    return AQ_E_ALIGN;
  if (B * (Hq + 2 * Hkv) > (int64_t)0x7fffffff) return AQ_E_RANGE;
  aq::RopeArgs a{};
  a.qkv = static_cast<const uint16_t*>(qkv);
  a.freqs = freqs;
  a.freqs_stride = freqs_stride;
  a.table = page_table;
  a.kc = static_cast<uint16_t*>(k_cache);
  a.vc = static_cast<uint16_t*>(v_cache);
  a.q_out = static_cast<uint16_t*>(q_out);
  a.P = P;
  a.pos = pos;
  a.page = page_size;
  a.n_pages = n_pages;
  a.B = (int)B;
  a.Hq = (int)Hq;
  a.Hkv = (int)Hkv;
  hipLaunchKernelGGL(aq::rope_kv_write_kernel, dim3((unsigned)(B * (Hq + 2 * Hkv))), dim3(64), 0,
                     static_cast<hipStream_t>(stream), a);
  return (int)hipGetLastError();
}

extern "C" int aq_paged_attn_decode(const void* q, const void* k_cache, const void* v_cache,
                                    const int64_t* page_table, int64_t P, int64_t total_len, int64_t page_size,
                                    int64_t n_pages, float scale, void* out, int64_t B, int64_t Hq, int64_t Hkv,
                                    int64_t D, void* stream) {
  if (D != aq::AD) return AQ_E_SHAPE;
  if (B < 0 || Hq <= 0 || Hkv <= 0 || (Hq % Hkv) != 0 || P <= 0 || total_len <= 0 || page_size <= 0 ||
      n_pages <= 0 || !(scale > 0.0f))
    return AQ_E_SHAPE;
  if (B == 0) return AQ_OK;
  if (!q || !k_cache || !v_cache || !page_table || !out) return AQ_E_NULL;
  if (aq::check_ptr16(q) || aq::check_ptr16(k_cache) || aq::check_ptr16(v_cache) || aq::check_ptr16(out))
    return AQ_E_ALIGN;
  if (B * Hkv > (int64_t)0x7fffffff) return AQ_E_RANGE;
  aq::AttnArgs a{};
  a.q = static_cast<const uint16_t*>(q);
  a.kc = static_cast<const uint16_t*>(k_cache);
  a.vc = static_cast<const uint16_t*>(v_cache);
  a.table = page_table;
  a.out = static_cast<uint16_t*>(out);
  a.P = P;
  a.T = total_len;
  a.page = page_size;
  a.n_pages = n_pages;
  a.scale_log2e = scale * 1.44269504088896341f;
  a.B = (int)B;
  a.Hq = (int)Hq;
  a.Hkv = (int)Hkv;
  // 8 wavefronts per (sequence, KV head): 256 registers each, enough to hold a batch's K and V
  // loads in flight together
  const dim3 grid((unsigned)(B * Hkv)), block(512);
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (Hq / Hkv) {
    case 1: hipLaunchKernelGGL((aq::paged_attn_decode_kernel<1, 8>), grid, block, 0, st, a); break;
    case 2: hipLaunchKernelGGL((aq::paged_attn_decode_kernel<2, 8>), grid, block, 0, st, a); break;
    case 4: hipLaunchKernelGGL((aq::paged_attn_decode_kernel<4, 8>), grid, block, 0, st, a); break;
    case 8: hipLaunchKernelGGL((aq::paged_attn_decode_kernel<8, 8>), grid, block, 0, st, a); break;
    default: return AQ_E_SHAPE;  // query heads per KV head: 1, 2, 4 or 8
  }
  return (int)hipGetLastError();
}
