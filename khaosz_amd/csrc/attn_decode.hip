// Attention around the quantized projections, on the paged KV cache in place:
// the reference rotates q and k with complex multiplies, writes k/v page by
// page, gathers every page into a contiguous [B, T, Hkv, D] copy, repeats the
// KV heads and calls a generic attention, per layer and per step
// (astrai/model/components/attention.py:83-103,
// astrai/inference/core/cache.py:216-274).  Kernels here:
//
//   rope_kv_write   rotates q and k of the new tokens (interleaved pairs, fp32,
//                   rope.py:26-33), stores q, and writes k and v into their page
//                   slots (cache.py:216-252) -- one token per sequence at decode,
//                   the whole prompt at prefill;
//   paged_attn      softmax(q K^T / sqrt(D)) V for one query token per sequence
//                   over the pages of that sequence, all query heads of a KV
//                   head in one workgroup (grouped-query attention without
//                   materialising the repeated heads, attention.py:15-23);
//                   optionally doing rope_kv_write's work for that token itself.
//
// bf16 tensors, head dimension 64 or 128, fp32 arithmetic.  Unmapped pages
// (table entry < 0 or out of range) are skipped on write and read as zero keys
// and values, as the reference's gather does.
#include "aq_common.h"
#include "aq_rows.h"

namespace aq {

// Rotates 8 consecutive elements (4 interleaved pairs): (x0 + i x1)(c + i s) with four rounded
// products, one rounded difference and one rounded sum per pair.
__device__ __forceinline__ uint4 rope8(uint4 x, const float* cs /* 4 (cos, sin) pairs */) {
  const float4 a = *reinterpret_cast<const float4*>(cs), b = *reinterpret_cast<const float4*>(cs + 4);
  const float c[4] = {a.x, a.z, b.x, b.z}, sn[4] = {a.y, a.w, b.y, b.w};
  const uint32_t in[4] = {x.x, x.y, x.z, x.w};
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float x0 = __uint_as_float(in[i] << 16), x1 = __uint_as_float(in[i] & 0xffff0000u);
    const float r0 = __fsub_rn(__fmul_rn(x0, c[i]), __fmul_rn(x1, sn[i]));
    const float r1 = __fadd_rn(__fmul_rn(x0, sn[i]), __fmul_rn(x1, c[i]));
    o[i] = pack_bf16x2(r0, r1);
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

// the same on table values already in registers
__device__ __forceinline__ uint4 rope8(uint4 x, float4 a, float4 b) {
  const float c[4] = {a.x, a.z, b.x, b.z}, sn[4] = {a.y, a.w, b.y, b.w};
  const uint32_t in[4] = {x.x, x.y, x.z, x.w};
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float x0 = __uint_as_float(in[i] << 16), x1 = __uint_as_float(in[i] & 0xffff0000u);
    const float r0 = __fsub_rn(__fmul_rn(x0, c[i]), __fmul_rn(x1, sn[i]));
    const float r1 = __fadd_rn(__fmul_rn(x0, sn[i]), __fmul_rn(x1, c[i]));
    o[i] = pack_bf16x2(r0, r1);
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

// RMSNorm over the head dimension of a rotated query or key (attention.py:62-64, 86-89: after the rotation, before
// the key goes into the cache).  The rotated values are taken as they are stored, rounded to bf16.  Sum of squares
// in a fixed order that does not depend on which kernel holds the vector how: per 8-element chunk the rounded
// squares are added in memory order, then the D / 8 chunk sums are combined by a butterfly over the chunk index
// (chunk c with c ^ 1, then ^ 2, ^ 4, ^ 8; fl(a + b) is the same whichever partner computes it).  Then
// r = 1 / sqrt(ss / D + eps) (every operation correctly rounded) and y = bf16((x * r) * gain).
__device__ __forceinline__ float chunk_sumsq(uint4 x) {
  const uint32_t in[4] = {x.x, x.y, x.z, x.w};
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float x0 = __uint_as_float(in[i] << 16), x1 = __uint_as_float(in[i] & 0xffff0000u);
    s = __fadd_rn(s, __fmul_rn(x0, x0));
    s = __fadd_rn(s, __fmul_rn(x1, x1));
  }
  return s;
}
__device__ __forceinline__ uint4 chunk_normed(uint4 x, float r, uint4 gain) {
  const uint32_t in[4] = {x.x, x.y, x.z, x.w}, gn[4] = {gain.x, gain.y, gain.z, gain.w};
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float x0 = __uint_as_float(in[i] << 16), x1 = __uint_as_float(in[i] & 0xffff0000u);
    const float g0 = __uint_as_float(gn[i] << 16), g1 = __uint_as_float(gn[i] & 0xffff0000u);
    o[i] = pack_bf16x2(__fmul_rn(__fmul_rn(x0, r), g0), __fmul_rn(__fmul_rn(x1, r), g1));
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

struct RopeArgs {
  const uint16_t* qkv;   // [B, S, (Hq + 2 Hkv) * D]
  const float* freqs;    // [S, D/2, 2] (cos, sin) per sequence; sequences freqs_stride floats apart (0: shared)
  int64_t freqs_stride;
  const int64_t* table;  // [B, P]
  uint16_t* kc;          // [n_pages, page, Hkv, D]
  uint16_t* vc;
  uint16_t* q_out;       // [B, S, Hq, D]
  uint16_t* k_out;       // [B, S, Hkv, D] rotated keys, or null
  int64_t P, pos, page, n_pages, S;
  int B, Hq, Hkv, D;
  const uint16_t* q_gain;  // [D] RMSNorm gains of the rotated q / k heads, or null: no qk-norm
  const uint16_t* k_gain;
  float eps;
};

// one thread per 16-byte chunk (8 elements) of a head vector of a token
__global__ __launch_bounds__(256) void rope_kv_write_kernel(RopeArgs p) {
  const int64_t heads = p.Hq + 2 * p.Hkv;
  const int cph = p.D / 8;  // chunks per head vector
  const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (c >= (int64_t)p.B * p.S * heads * cph) return;
  const int ch = (int)(c % cph);
  const int64_t hv = c / cph, tokn = hv / heads;
  const int h = (int)(hv % heads);
  const int64_t b = tokn / p.S, s = tokn % p.S;
  uint4 x = *reinterpret_cast<const uint4*>(p.qkv + hv * p.D + ch * 8);
  if (h < p.Hq + p.Hkv) x = rope8(x, p.freqs + b * p.freqs_stride + s * p.D + ch * 8);  // v heads do not rotate
  if (p.q_gain) {  // uniform: qk-norm.  A head vector's D / 8 chunks sit in neighbouring lanes of one DPP row.
    float ss = chunk_sumsq(x);
    ss = __fadd_rn(ss, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(ss), 0xB1, 0xf, 0xf, false)));   // c ^ 1
    ss = __fadd_rn(ss, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(ss), 0x4E, 0xf, 0xf, false)));   // c ^ 2
    ss = __fadd_rn(ss, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(ss), 0x141, 0xf, 0xf, false)));  // the other quad of the half row: c ^ 4
    if (p.D == 128)
      ss = __fadd_rn(ss, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(ss), 0x140, 0xf, 0xf, false)));  // the other half row: c ^ 8
    if (h < p.Hq + p.Hkv) {
      const uint16_t* gain = h < p.Hq ? p.q_gain : p.k_gain;
      x = chunk_normed(x, rms_scale(ss, (float)p.D, p.eps), *reinterpret_cast<const uint4*>(gain + ch * 8));
    }
  }
  if (h < p.Hq) {
    *reinterpret_cast<uint4*>(p.q_out + (tokn * p.Hq + h) * p.D + ch * 8) = x;
    return;
  }
  const bool is_k = h < p.Hq + p.Hkv;
  const int kvh = is_k ? h - p.Hq : h - p.Hq - p.Hkv;
  if (is_k && p.k_out) *reinterpret_cast<uint4*>(p.k_out + (tokn * p.Hkv + kvh) * p.D + ch * 8) = x;
  const int64_t pos = p.pos + s, lp = pos / p.page;
  const int64_t phys = lp < p.P ? p.table[b * p.P + lp] : -1;
  if (phys < 0 || phys >= p.n_pages) return;  // unmapped: the token is dropped, as in the reference
  uint16_t* dst = (is_k ? p.kc : p.vc) + ((phys * p.page + pos % p.page) * p.Hkv + kvh) * p.D + ch * 8;
  *reinterpret_cast<uint4*>(dst) = x;
}

struct AttnArgs {
  const uint16_t* q;     // [B, Hq, D]
  const uint16_t* kc;    // [n_pages, page, Hkv, D]
  const uint16_t* vc;
  const int64_t* table;  // [B, P]
  const int64_t* lens;   // [B] positions each sequence may attend to (its own length), or null: all T
  uint16_t* out;         // [B, Hq, D]
  float* ws;             // partial results [B, Hq, NS, D + 4] when NS > 1
  const uint16_t* qkv;   // ROPE kernels: [B, (Hq + 2 Hkv) * D] projections of the new token (position T - 1)
  const float* freqs;    // ROPE kernels: its rotary table, as in RopeArgs
  uint16_t* kc_w;        // ROPE kernels: the caches again, writable
  uint16_t* vc_w;
  int64_t freqs_stride;
  int64_t P, T, page, n_pages;
  float scale_log2e;     // softmax scale times log2(e): scores live in the exp2 domain
  int B, Hq, Hkv, NS;
  const uint16_t* q_gain;  // QKN kernels: [D] RMSNorm gains of the rotated q / k heads
  const uint16_t* k_gain;
  float eps;
};

constexpr int ATT_WAVES = 4;
constexpr int ATT_KPW = 64;                  // positions per wavefront
constexpr int ATT_KPG = ATT_WAVES * ATT_KPW; // positions per workgroup
constexpr int ATT_MAX_D = 128;
constexpr float ATT_MASKED = -1.0e30f;  // score (exp2 domain) of a cached position the sequence may not attend to

// maximum / sum over each row of 16 consecutive lanes, result in all of them
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, false)));   // quad_perm [1,0,3,2]
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, false)));   // quad_perm [2,3,0,1]
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, false)));  // row_half_mirror
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, false)));  // row_mirror
  return v;
}
__device__ __forceinline__ float row16_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, false));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, false));
  return v;
}

typedef __bf16 attn_bf16x8 __attribute__((ext_vector_type(8)));
typedef float attn_f32x4 __attribute__((ext_vector_type(4)));

// Workgroup = one (sequence, KV head, slice of the cached positions): the G
// query heads of the KV head share every K and V byte.  A wavefront owns 64
// consecutive positions, a workgroup 256; the NS slices of a sequence run as
// separate workgroups so that a decode batch of a few sequences still spreads
// over the device.  Every K and V load of a wavefront, 16 bytes per lane, is
// requested before anything is computed.
//   scores   on the matrix core: S[head, key] = Q K^T as v_mfma_f32_16x16x32_bf16
//            tiles, the G <= 8 query heads padded to 16 rows, four tiles of 16
//            keys, D / 32 steps each.  K rows are loaded straight in operand
//            order (lane l: key l % 16 of the tile, dimensions 8 (l / 16) .. + 8
//            of the step), queries likewise; a lane ends up with the scores of
//            one key per tile for 4 heads;
//   softmax  maximum and denominator over a row of 16 lanes by DPP and over the
//            four tiles in registers; probabilities to LDS;
//   values   V rows are loaded CPR = D / 8 lanes to a row (a load covers 4 or 8
//            whole rows); a lane accumulates p * V over the keys it loaded (8
//            dimensions x G heads, fma), the key groups are summed with xor
//            shuffles.
// The wavefronts' (maximum, denominator, numerator) are merged through LDS and
// either normalised into the output (NS == 1) or left in the workspace for
// attn_merge_kernel.
// ROPE: the kernel also does rope_kv_write_kernel's work for the new token at
// position T - 1 -- every workgroup rotates its own queries from the raw
// projection, and the one wavefront whose positions include T - 1 rotates the
// new key, stores it and the new value into their page slot and uses them from
// registers instead of what it read from the cache.  Same roundings, so caches
// and outputs are the bits the two separate launches give.
// QKN (with ROPE): the rotated queries and the rotated new key are RMS-normalised over the head dimension (see
// chunk_sumsq) before they are used and stored: what rope_kv_write_kernel does with gains, same bits.  A head
// vector's chunk c = 4 ks + kq sits in register ks of the lane with that kq.
template <int G, int D, bool ROPE, bool QKN = false>
__global__ __launch_bounds__(ATT_WAVES * 64) void paged_attn_decode_kernel(AttnArgs p) {
  static_assert(!QKN || ROPE, "qk-norm belongs to the kernels that rotate");
  constexpr int CPR = D / 8;     // 16-byte chunks per row: 16 or 8
  constexpr int RPL = 64 / CPR;  // rows per load instruction: 4 or 8
  constexpr int NL = 64 / RPL;   // loads per wavefront (= CPR)
  constexpr int KPW = ATT_KPW, KPG = ATT_KPG;
  constexpr int ATT_THREADS = ATT_WAVES * 64;
  constexpr int PART = D + 4;    // numerator[D], maximum, denominator, 2 floats of padding
  static_assert(D == 64 || D == 128, "head dimension");
  __shared__ __align__(16) float p_s[ATT_WAVES][KPW][G];
  __shared__ float m_s[ATT_WAVES][G], l_s[ATT_WAVES][G];
  __shared__ __align__(16) float acc_s[ATT_WAVES][G][D];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int sub = lane / CPR, ch = lane % CPR;  // key within a load, 16-byte chunk of the row
  // the KV heads of one slice are neighbours in the launch order: together they read whole
  // [position][Hkv][D] stretches of the pages at about the same time
  const int kvh = blockIdx.x % p.Hkv, bs = blockIdx.x / p.Hkv;
  const int split = bs % p.NS, b = bs / p.NS;
  const int64_t T = p.T;
  const int64_t t0 = (int64_t)split * KPG + wave * KPW;  // first position of this wavefront
  // A sequence shorter than T (a decode batch of sequences at different positions): positions from its own
  // length on are masked, as the additive mask of the reference's forward does.  The mask value is finite, so
  // a wavefront or slice whose positions are all masked leaves a partial result that later merges weigh with 0.
  int64_t vis = T;
  if (p.lens) {
    const int64_t l = p.lens[b];
    vis = l < T ? (l > 0 ? l : 0) : T;
  }

  constexpr int KS = D / 32;                  // matrix-core steps over the head dimension
  const int col = lane & 15, kq = lane >> 4;  // operand row / column, group of 8 dimensions inside a step
  float acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[g][e] = 0.0f;
  }
  // The queries (and their rotary table values) do not depend on the page table: requested first, used after
  // the K and V loads have been issued, so that the wavefront waits for one memory round trip less.
  uint4 qraw[KS];
  float4 fa[KS], fb[KS];
  if (t0 < T) {
    const int hq = col < G ? col : 0;  // heads past G: zero rows of the operand (their loads read head 0)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = ks * 32 + kq * 8;
      if constexpr (ROPE) {
        qraw[ks] = *reinterpret_cast<const uint4*>(p.qkv + ((int64_t)b * (p.Hq + 2 * p.Hkv) + kvh * G + hq) * D + d0);
        const float* cs = p.freqs + (int64_t)b * p.freqs_stride + d0;
        fa[ks] = *reinterpret_cast<const float4*>(cs);
        fb[ks] = *reinterpret_cast<const float4*>(cs + 4);
      } else {
        qraw[ks] = *reinterpret_cast<const uint4*>(p.q + ((int64_t)b * p.Hq + kvh * G + hq) * D + d0);
      }
    }
  }
  // RMSNorm of a rotated head vector held as KS chunks per lane (chunk 4 ks + kq), gains requested by the caller
  auto head_norm = [&](uint4 (&v)[KS], const uint4 (&gain)[KS]) {
    float ss[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      ss[ks] = chunk_sumsq(v[ks]);
      ss[ks] = __fadd_rn(ss[ks], __shfl_xor(ss[ks], 16, 64));  // c ^ 1
      ss[ks] = __fadd_rn(ss[ks], __shfl_xor(ss[ks], 32, 64));  // c ^ 2
    }
    float tot = __fadd_rn(ss[0], ss[1]);                            // c ^ 4
    if constexpr (KS == 4) tot = __fadd_rn(tot, __fadd_rn(ss[2], ss[3]));  // c ^ 8
    const float r = rms_scale(tot, (float)D, p.eps);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) v[ks] = chunk_normed(v[ks], r, gain[ks]);
  };
  uint4 qgain[KS], kgain[KS];
  if constexpr (QKN) {
    if (t0 < T) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        qgain[ks] = *reinterpret_cast<const uint4*>(p.q_gain + ks * 32 + kq * 8);
        kgain[ks] = *reinterpret_cast<const uint4*>(p.k_gain + ks * 32 + kq * 8);
      }
    }
  }
  if (t0 < T) {  // wavefront-uniform
    // lane L looks up the row of position t0 + L (element offset, -1: unmapped or past T)
    int64_t row = -1;
    {
      const int64_t t = t0 + lane;
      if (t < T) {
        const int64_t lp = t / p.page;
        const int64_t phys = lp < p.P ? p.table[(int64_t)b * p.P + lp] : -1;
        if (phys >= 0 && phys < p.n_pages) row = ((phys * p.page + t % p.page) * p.Hkv + kvh) * D;
      }
    }
    auto row_of = [&](int src) -> int64_t {
      const int lo = __shfl((int)(uint32_t)row, src, 64), hi = __shfl((int)(row >> 32), src, 64);
      return ((int64_t)hi << 32) | (uint32_t)lo;
    };
    const bool has_new = ROPE && T - 1 >= t0 && T - 1 < t0 + KPW;  // wavefront-uniform
    // ---- operands of the scores
    // keys: tile t holds positions t0 + 16 t .. + 16; lane = (key col, dimensions ks * 32 + kq * 8 .. + 8).
    // values: lane = (key sub of a load, 16-byte chunk ch of the row).  Rows that are unmapped or past T read
    // row 0 of the cache and are zeroed afterwards.  Every load is issued before any loaded value is touched
    // (the fix-ups below are selects on data, kept out of the issue loops: with them inside, the compiler
    // waited for each load before issuing the next).
    uint4 kb[4][KS], vv[NL];
    uint32_t kneg = 0, vneg = 0;  // bit t / i: that row is not there
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int64_t r = row_of(t * 16 + col);
      kneg |= (r < 0 ? 1u : 0u) << t;
      const uint16_t* src = p.kc + (r >= 0 ? r : 0) + kq * 8;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) kb[t][ks] = *reinterpret_cast<const uint4*>(src + ks * 32);
    }
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int64_t r = row_of(i * RPL + sub);
      vneg |= (r < 0 ? 1u : 0u) << i;
      vv[i] = *reinterpret_cast<const uint4*>(p.vc + (r >= 0 ? r : 0) + ch * 8);
    }
    __builtin_amdgcn_sched_barrier(0);  // nothing that waits for a load may move above the last load's issue
    if (__builtin_amdgcn_ballot_w64(row < 0) != 0) {  // wavefront-uniform; rare: a hole, or the wavefront that holds T - 1
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          if (kneg & (1u << t)) kb[t][ks] = make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int i = 0; i < NL; ++i)
        if (vneg & (1u << i)) vv[i] = make_uint4(0, 0, 0, 0);
    }
    if (ROPE && has_new) {  // wavefront-uniform: this wavefront owns position T - 1
      // the new key and value: rotated here, stored into their page slot, and used from registers in place
      // of what was just read from that slot
      const uint16_t* tok = p.qkv + (int64_t)b * (p.Hq + 2 * p.Hkv) * D;
      const int64_t rn = row_of((int)(T - 1 - t0));  // the same in every lane; -1: its page is unmapped
      if (rn >= 0) {
        const int tn = (int)(T - 1 - t0) >> 4, cn = (int)(T - 1 - t0) & 15;  // tile and column of the new key
        uint4 kn[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          kn[ks] = rope8(*reinterpret_cast<const uint4*>(tok + (int64_t)(p.Hq + kvh) * D + ks * 32 + kq * 8), fa[ks], fb[ks]);
        if constexpr (QKN) head_norm(kn, kgain);  // (every column holds the same new key: all lanes take part)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const int d0 = ks * 32 + kq * 8;
          if (col == cn) *reinterpret_cast<uint4*>(p.kc_w + rn + d0) = kn[ks];
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (t == tn && col == cn) kb[t][ks] = kn[ks];
        }
        const uint4 vn = *reinterpret_cast<const uint4*>(tok + (int64_t)(p.Hq + p.Hkv + kvh) * D + ch * 8);
        const int in = (int)(T - 1 - t0) / RPL, sn = (int)(T - 1 - t0) % RPL;  // load and key group of the new value
        if (sub == sn) *reinterpret_cast<uint4*>(p.vc_w + rn + ch * 8) = vn;
#pragma unroll
        for (int i = 0; i < NL; ++i)
          if (i == in && sub == sn) vv[i] = vn;
      }
    }
    // queries: lane = (head col, dimensions ks * 32 + kq * 8 .. + 8)
    uint4 qa[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if constexpr (ROPE)
        qa[ks] = rope8(qraw[ks], fa[ks], fb[ks]);
      else
        qa[ks] = qraw[ks];
    }
    if constexpr (QKN) head_norm(qa, qgain);  // (columns past G normalise a copy of head 0 and are zeroed below)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (col >= G) qa[ks] = make_uint4(0, 0, 0, 0);
    }
    // ---- scores: S[head][key] per tile; this lane gets key col of the tile, heads 4 kq .. + 4
    attn_f32x4 sc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      attn_f32x4 c = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(attn_bf16x8, qa[ks]),
                                                   __builtin_bit_cast(attn_bf16x8, kb[t][ks]), c, 0, 0, 0);
      sc[t] = c;
    }
    // ---- softmax over the wavefront's 64 positions, per head
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int head = 4 * kq + r;
      float sv[4], mx = -INFINITY;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int64_t pos = t0 + t * 16 + col;
        sv[t] = pos < T ? (pos < vis ? sc[t][r] * p.scale_log2e : ATT_MASKED) : -INFINITY;
        mx = fmaxf(mx, sv[t]);
      }
      mx = row16_max(mx);  // finite: position t0 is valid
      float sum = 0.0f;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const float pv = __builtin_amdgcn_exp2f(sv[t] - mx);  // 0 for positions past T
        sum += pv;
        if (head < G) p_s[wave][t * 16 + col][head] = pv;
      }
      sum = row16_sum(sum);
      if (col == 0 && head < G) {
        m_s[wave][head] = mx;
        l_s[wave][head] = sum;
      }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // this wavefront's LDS writes are done (wavefront-private region)
    asm volatile("" ::: "memory");
    // ---- numerator (unmapped rows and positions past T contribute zeros)
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      float v8[8];
      v8[0] = __uint_as_float(vv[i].x << 16);
      v8[1] = __uint_as_float(vv[i].x & 0xffff0000u);
      v8[2] = __uint_as_float(vv[i].y << 16);
      v8[3] = __uint_as_float(vv[i].y & 0xffff0000u);
      v8[4] = __uint_as_float(vv[i].z << 16);
      v8[5] = __uint_as_float(vv[i].z & 0xffff0000u);
      v8[6] = __uint_as_float(vv[i].w << 16);
      v8[7] = __uint_as_float(vv[i].w & 0xffff0000u);
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float pj = p_s[wave][i * RPL + sub][g];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = __builtin_fmaf(pj, v8[e], acc[g][e]);
      }
    }
    // Sum over the RPL key groups (lanes CPR apart) with a transposed butterfly: at each stage a lane keeps
    // one half of its values and trades the other half with its partner, so the 8 G values per lane cost
    // 8 G (1 - 1 / RPL) exchanges instead of 8 G log2(RPL), and a lane ends up with 8 G / RPL finished sums.
    {
      constexpr int NV = 8 * G;
      float a[NV];
#pragma unroll
      for (int j = 0; j < NV; ++j) a[j] = acc[j / 8][j % 8];
      int base = 0;  // first original index of the values this lane still holds
#pragma unroll
      for (int st = 0; (CPR << st) < 64; ++st) {
        const int off = CPR << st, h = NV >> (st + 1);
        const bool up = (lane & off) != 0;
#pragma unroll
        for (int i = 0; i < h; ++i) {
          if (off == 32 || off == 16) {
            // half / row swaps: lanes without the bit receive the partner's a[i], lanes with it the partner's
            // a[i + h], next to their own; one add finishes the exchange
            typedef unsigned att_u2 __attribute__((ext_vector_type(2)));
            const att_u2 r = off == 32 ? __builtin_amdgcn_permlane32_swap(__float_as_uint(a[i]), __float_as_uint(a[i + h]), false, false)
                                       : __builtin_amdgcn_permlane16_swap(__float_as_uint(a[i]), __float_as_uint(a[i + h]), false, false);
            a[i] = __uint_as_float(r.x) + __uint_as_float(r.y);
          } else {
            // select by mask rather than by ?: -- the compiler turned the latter into per-exchange branches
            const uint32_t lo = __float_as_uint(a[i]), hi = __float_as_uint(a[i + h]);
            const uint32_t t = (lo ^ hi) & (up ? 0xffffffffu : 0u);
            a[i] = __uint_as_float(t ^ lo) + __shfl_xor(__uint_as_float(t ^ hi), off, 64);  // keep + partner's send
          }
        }
        base += up ? h : 0;
      }
      asm volatile("" : "+v"(base));  // one address computation below, not a code path per value of base
      float* dst = &acc_s[wave][0][ch * 8];
#pragma unroll
      for (int i = 0; i < NV / RPL; ++i) {
        const int j = base + i;
        dst[(j >> 3) * D + (j & 7)] = a[i];
      }
    }
  } else {  // a wavefront past T: nothing to add
    if (lane < G) {
      m_s[wave][lane] = -INFINITY;
      l_s[wave][lane] = 0.0f;
    }
    for (int i = lane; i < G * D; i += 64) acc_s[wave][i / D][i % D] = 0.0f;
  }
  // ---- merge the wavefronts' partial results
  __syncthreads();
  for (int i = tid; i < G * D / 2; i += ATT_THREADS) {
    const int g = i / (D / 2), d = (i % (D / 2)) * 2;  // dimensions d, d + 1
    float mm = -INFINITY;
#pragma unroll
    for (int w = 0; w < ATT_WAVES; ++w) mm = fmaxf(mm, m_s[w][g]);
    float n0 = 0.0f, n1 = 0.0f, den = 0.0f;
#pragma unroll
    for (int w = 0; w < ATT_WAVES; ++w) {
      const float a = m_s[w][g] == -INFINITY ? 0.0f : exp2f(m_s[w][g] - mm);  // wavefronts past T
      n0 = __builtin_fmaf(acc_s[w][g][d], a, n0);
      n1 = __builtin_fmaf(acc_s[w][g][d + 1], a, n1);
      den = __builtin_fmaf(l_s[w][g], a, den);
    }
    const int64_t head = (int64_t)b * p.Hq + kvh * G + g;
    if (p.NS == 1 && p.out != nullptr) {  // out == nullptr: the caller wants the partial results whatever NS is
      const float r = attn_inv_denominator(den);
      store_wt(reinterpret_cast<uint32_t*>(p.out + head * D + d), pack_bf16x2(__fmul_rn(n0, r), __fmul_rn(n1, r)));
    } else {
      float* part = p.ws + (head * p.NS + split) * PART;
      store_wt(reinterpret_cast<uint2*>(part + d), make_uint2(__float_as_uint(n0), __float_as_uint(n1)));
      if (d == 0) store_wt(reinterpret_cast<uint2*>(part + D), make_uint2(__float_as_uint(mm), __float_as_uint(den)));
    }
  }
}

// Combines the NS slices of one (sequence, query head): thread = dimension pair (D / 2 threads).
__global__ __launch_bounds__(ATT_MAX_D / 2) void attn_merge_kernel(const float* ws, uint16_t* out, int NS, int D) {
  const int d = threadIdx.x * 2, part_sz = D + 4;
  const float* part = ws + (int64_t)blockIdx.x * NS * part_sz;
  // Slices are taken eight at a time, all loads of a group requested before any is used: with one slice per
  // loop turn every load waited for the one before it (32 slices: two passes of 32 round trips).  The sums
  // still run in slice order.
  constexpr int GRP = 8;
  float mm = -INFINITY;
  float n0 = 0.0f, n1 = 0.0f, den = 0.0f;
  if (NS <= GRP) {
    // The usual case (up to 2048 positions): (maximum, denominator) and the numerators of every slice are
    // requested together, so the launch is one memory round trip instead of two (maxima first, then values).
    float2 md[GRP], v[GRP];
#pragma unroll
    for (int i = 0; i < GRP; ++i) {
      const bool ok = i < NS;  // uniform
      md[i] = ok ? *reinterpret_cast<const float2*>(part + i * part_sz + D) : make_float2(-INFINITY, 0.0f);
      v[i] = ok ? *reinterpret_cast<const float2*>(part + i * part_sz + d) : make_float2(0.0f, 0.0f);
    }
#pragma unroll
    for (int i = 0; i < GRP; ++i) mm = fmaxf(mm, md[i].x);
#pragma unroll
    for (int i = 0; i < GRP; ++i) {
      if (i < NS) {
        const float a = attn_slice_weight(md[i].x, mm);
        n0 = __builtin_fmaf(v[i].x, a, n0);
        n1 = __builtin_fmaf(v[i].y, a, n1);
        den = __builtin_fmaf(md[i].y, a, den);
      }
    }
  } else {
    for (int s0 = 0; s0 < NS; s0 += GRP) {  // slice 0 always holds a position
      float mv[GRP];
#pragma unroll
      for (int i = 0; i < GRP; ++i) mv[i] = s0 + i < NS ? part[(s0 + i) * part_sz + D] : -INFINITY;
#pragma unroll
      for (int i = 0; i < GRP; ++i) mm = fmaxf(mm, mv[i]);
    }
    for (int s0 = 0; s0 < NS; s0 += GRP) {
      float2 md[GRP], v[GRP];
#pragma unroll
      for (int i = 0; i < GRP; ++i) {
        const bool ok = s0 + i < NS;  // uniform
        md[i] = ok ? *reinterpret_cast<const float2*>(part + (s0 + i) * part_sz + D) : make_float2(0.0f, 0.0f);
        v[i] = ok ? *reinterpret_cast<const float2*>(part + (s0 + i) * part_sz + d) : make_float2(0.0f, 0.0f);
      }
#pragma unroll
      for (int i = 0; i < GRP; ++i) {
        if (s0 + i < NS) {
          const float a = attn_slice_weight(md[i].x, mm);
          n0 = __builtin_fmaf(v[i].x, a, n0);
          n1 = __builtin_fmaf(v[i].y, a, n1);
          den = __builtin_fmaf(md[i].y, a, den);
        }
      }
    }
  }
  const float r = attn_inv_denominator(den);
  store_wt(reinterpret_cast<uint32_t*>(out + (int64_t)blockIdx.x * D + d), pack_bf16x2(__fmul_rn(n0, r), __fmul_rn(n1, r)));
}

inline int64_t attn_slices(int64_t T) { return (T + ATT_KPG - 1) / ATT_KPG; }
// sized for the larger head dimension, so that the size does not depend on D
inline int64_t attn_workspace_bytes(int64_t B, int64_t Hq, int64_t ns) {
  return B * Hq * ns * (ATT_MAX_D + 4) * (int64_t)sizeof(float);
}

}  // namespace aq

// q_gain == nullptr: no qk-norm (then k_gain and eps are not looked at)
static int rope_kv_write(const void* qkv, const float* freqs, int64_t freqs_stride, const int64_t* page_table,
                         int64_t P, int64_t pos, int64_t S, int64_t page_size, void* k_cache, void* v_cache,
                         int64_t n_pages, void* q_out, void* k_out, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                         const void* q_gain, const void* k_gain, float eps, void* stream) {
  if (D != 64 && D != 128) return AQ_E_SHAPE;
  if (q_gain && (!k_gain || !(eps >= 0.0f))) return k_gain ? AQ_E_SHAPE : AQ_E_NULL;
  if (aq::check_ptr16(q_gain) || (q_gain && aq::check_ptr16(k_gain))) return AQ_E_ALIGN;
  if (B < 0 || S < 0 || Hq <= 0 || Hkv <= 0 || P <= 0 || pos < 0 || page_size <= 0 || n_pages <= 0) return AQ_E_SHAPE;
  if (freqs_stride != 0 && freqs_stride < S * D) return AQ_E_SHAPE;
  if (B == 0 || S == 0) return AQ_OK;
  if (!qkv || !freqs || !page_table || !k_cache || !v_cache || !q_out) return AQ_E_NULL;
  if (aq::check_ptr16(qkv) || aq::check_ptr16(k_cache) || aq::check_ptr16(v_cache) || aq::check_ptr16(q_out) ||
      aq::check_ptr16(freqs) || (freqs_stride & 3) || (k_out && aq::check_ptr16(k_out)))
    return AQ_E_ALIGN;
  const int64_t chunks = B * S * (Hq + 2 * Hkv) * (D / 8);
  if (chunks > (int64_t)0x7fffffff * 256) return AQ_E_RANGE;
  aq::RopeArgs a{};
  a.qkv = static_cast<const uint16_t*>(qkv);
  a.freqs = freqs;
  a.freqs_stride = freqs_stride;
  a.table = page_table;
  a.kc = static_cast<uint16_t*>(k_cache);
  a.vc = static_cast<uint16_t*>(v_cache);
  a.q_out = static_cast<uint16_t*>(q_out);
  a.k_out = static_cast<uint16_t*>(k_out);
  a.P = P;
  a.pos = pos;
  a.page = page_size;
  a.n_pages = n_pages;
  a.S = S;
  a.B = (int)B;
  a.Hq = (int)Hq;
  a.Hkv = (int)Hkv;
  a.D = (int)D;
  a.q_gain = static_cast<const uint16_t*>(q_gain);
  a.k_gain = static_cast<const uint16_t*>(k_gain);
  a.eps = eps;
  hipLaunchKernelGGL(aq::rope_kv_write_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), a);
  return (int)hipGetLastError();
}

extern "C" int aq_rope_kv_write(const void* qkv, const float* freqs, int64_t freqs_stride, const int64_t* page_table,
                                int64_t P, int64_t pos, int64_t S, int64_t page_size, void* k_cache, void* v_cache,
                                int64_t n_pages, void* q_out, void* k_out, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                                void* stream) {
  return rope_kv_write(qkv, freqs, freqs_stride, page_table, P, pos, S, page_size, k_cache, v_cache, n_pages, q_out, k_out,
                       B, Hq, Hkv, D, nullptr, nullptr, 0.0f, stream);
}

extern "C" int aq_rope_kv_write_qknorm(const void* qkv, const float* freqs, int64_t freqs_stride,
                                       const int64_t* page_table, int64_t P, int64_t pos, int64_t S, int64_t page_size,
                                       void* k_cache, void* v_cache, int64_t n_pages, void* q_out, void* k_out, int64_t B,
                                       int64_t Hq, int64_t Hkv, int64_t D, const void* q_gain, const void* k_gain,
                                       float eps, void* stream) {
  if (!q_gain || !k_gain) return AQ_E_NULL;
  return rope_kv_write(qkv, freqs, freqs_stride, page_table, P, pos, S, page_size, k_cache, v_cache, n_pages, q_out, k_out,
                       B, Hq, Hkv, D, q_gain, k_gain, eps, stream);
}

extern "C" int64_t aq_paged_attn_decode_workspace_bytes(int64_t B, int64_t Hq, int64_t Hkv, int64_t total_len) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || total_len <= 0) return 0;
  const int64_t ns = aq::attn_slices(total_len);
  return ns == 1 ? 0 : aq::attn_workspace_bytes(B, Hq, ns);
}

template <int G, int D>
static void attn_launch(bool rope, dim3 grid, dim3 block, hipStream_t st, const aq::AttnArgs& a) {
  if (rope && a.q_gain)
    hipLaunchKernelGGL((aq::paged_attn_decode_kernel<G, D, true, true>), grid, block, 0, st, a);
  else if (rope)
    hipLaunchKernelGGL((aq::paged_attn_decode_kernel<G, D, true>), grid, block, 0, st, a);
  else
    hipLaunchKernelGGL((aq::paged_attn_decode_kernel<G, D, false>), grid, block, 0, st, a);
}

// q == nullptr: the fused form, queries and the new token come from qkv / freqs.
// partials: stop after the slices' partial results (no merge launch, `out` unused).
static int attn_decode(const void* q, const void* qkv, const float* freqs, int64_t freqs_stride, void* k_cache,
                       void* v_cache, const int64_t* page_table, int64_t P, int64_t total_len,
                       const int64_t* seq_lens, int64_t page_size,
                       int64_t n_pages, float scale, void* out, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                       void* workspace, int64_t workspace_bytes, void* stream, bool partials = false,
                       const void* q_gain = nullptr, const void* k_gain = nullptr, float eps = 0.0f) {
  const bool rope = q == nullptr;
  if (D != 64 && D != 128) return AQ_E_SHAPE;
  if (q_gain && (!rope || !k_gain)) return AQ_E_NULL;  // qk-norm belongs to the forms that rotate
  if (q_gain && !(eps >= 0.0f)) return AQ_E_SHAPE;
  if (aq::check_ptr16(q_gain) || (q_gain && aq::check_ptr16(k_gain))) return AQ_E_ALIGN;
  if (B < 0 || Hq <= 0 || Hkv <= 0 || (Hq % Hkv) != 0 || P <= 0 || total_len <= 0 || page_size <= 0 ||
      n_pages <= 0 || !(scale > 0.0f))
    return AQ_E_SHAPE;
  const int64_t G = Hq / Hkv;
  if (G != 1 && G != 2 && G != 3 && G != 4 && G != 6 && G != 8) return AQ_E_SHAPE;  // query heads per KV head
  if (rope && freqs_stride != 0 && freqs_stride < D) return AQ_E_SHAPE;
  if (B == 0) return AQ_OK;
  if (!(rope ? (qkv != nullptr && freqs != nullptr) : (q != nullptr)) || !k_cache || !v_cache || !page_table ||
      (!out && !partials))
    return AQ_E_NULL;
  if (aq::check_ptr16(rope ? qkv : q) || aq::check_ptr16(k_cache) || aq::check_ptr16(v_cache) ||
      (!partials && aq::check_ptr16(out)))
    return AQ_E_ALIGN;
  if (rope && (aq::check_ptr16(freqs) || (freqs_stride & 3))) return AQ_E_ALIGN;
  const int64_t ns = aq::attn_slices(total_len);
  if (B * Hkv * ns > (int64_t)0x7fffffff || B * Hq > (int64_t)0x7fffffff) return AQ_E_RANGE;
  if (ns > 1 || partials) {
    if (!workspace) return AQ_E_NULL;
    if (aq::check_ptr16(workspace)) return AQ_E_ALIGN;
    if (workspace_bytes < aq::attn_workspace_bytes(B, Hq, ns)) return AQ_E_WORKSPACE;
  }
  aq::AttnArgs a{};
  a.q = static_cast<const uint16_t*>(q);
  a.qkv = static_cast<const uint16_t*>(qkv);
  a.freqs = freqs;
  a.freqs_stride = freqs_stride;
  a.kc = static_cast<const uint16_t*>(k_cache);
  a.vc = static_cast<const uint16_t*>(v_cache);
  a.kc_w = static_cast<uint16_t*>(k_cache);
  a.vc_w = static_cast<uint16_t*>(v_cache);
  a.table = page_table;
  a.lens = seq_lens;
  a.out = partials ? nullptr : static_cast<uint16_t*>(out);
  a.ws = static_cast<float*>(workspace);
  a.P = P;
  a.T = total_len;
  a.page = page_size;
  a.n_pages = n_pages;
  a.scale_log2e = scale * 1.44269504088896341f;
  a.B = (int)B;
  a.Hq = (int)Hq;
  a.Hkv = (int)Hkv;
  a.NS = (int)ns;
  a.q_gain = static_cast<const uint16_t*>(q_gain);
  a.k_gain = static_cast<const uint16_t*>(k_gain);
  a.eps = eps;
  const dim3 grid((unsigned)(B * Hkv * ns)), block(aq::ATT_WAVES * 64);
  hipStream_t st = static_cast<hipStream_t>(stream);
#define AQ_ATTN_CASE(G_)                                            \
  case G_:                                                          \
    if (D == 128) attn_launch<G_, 128>(rope, grid, block, st, a);   \
    else attn_launch<G_, 64>(rope, grid, block, st, a);             \
    break;
  switch (G) {
    AQ_ATTN_CASE(1)
    AQ_ATTN_CASE(2)
    AQ_ATTN_CASE(3)
    AQ_ATTN_CASE(4)
    AQ_ATTN_CASE(6)
    AQ_ATTN_CASE(8)
  }
#undef AQ_ATTN_CASE
  int rc = (int)hipGetLastError();
  if (rc != 0 || ns == 1 || partials) return rc;
  hipLaunchKernelGGL(aq::attn_merge_kernel, dim3((unsigned)(B * Hq)), dim3((unsigned)(D / 2)), 0, st, a.ws, a.out, a.NS,
                     (int)D);
  return (int)hipGetLastError();
}

extern "C" int aq_paged_attn_decode(const void* q, const void* k_cache, const void* v_cache,
                                    const int64_t* page_table, int64_t P, int64_t total_len,
                                    const int64_t* seq_lens, int64_t page_size,
                                    int64_t n_pages, float scale, void* out, int64_t B, int64_t Hq, int64_t Hkv,
                                    int64_t D, void* workspace, int64_t workspace_bytes, void* stream) {
  if (!q && B > 0) return AQ_E_NULL;
  return attn_decode(q, nullptr, nullptr, 0, const_cast<void*>(k_cache), const_cast<void*>(v_cache), page_table, P,
                     total_len, seq_lens, page_size, n_pages, scale, out, B, Hq, Hkv, D, workspace, workspace_bytes, stream);
}

extern "C" int aq_rope_paged_attn_decode(const void* qkv, const float* freqs, int64_t freqs_stride,
                                         const int64_t* page_table, int64_t P, int64_t total_len,
                                         const int64_t* seq_lens, int64_t page_size,
                                         void* k_cache, void* v_cache, int64_t n_pages, float scale, void* out,
                                         int64_t B, int64_t Hq, int64_t Hkv, int64_t D, void* workspace,
                                         int64_t workspace_bytes, void* stream) {
  if ((!qkv || !freqs) && B > 0) return AQ_E_NULL;
  return attn_decode(nullptr, qkv, freqs, freqs_stride, k_cache, v_cache, page_table, P, total_len, seq_lens, page_size, n_pages,
                     scale, out, B, Hq, Hkv, D, workspace, workspace_bytes, stream);
}

extern "C" int64_t aq_paged_attn_decode_slices(int64_t total_len) { return total_len <= 0 ? 0 : aq::attn_slices(total_len); }

extern "C" int64_t aq_paged_attn_decode_partials_bytes(int64_t B, int64_t Hq, int64_t total_len) {
  if (B <= 0 || Hq <= 0 || total_len <= 0) return 0;
  return aq::attn_workspace_bytes(B, Hq, aq::attn_slices(total_len));
}

extern "C" int aq_paged_attn_decode_partials(const void* q, const void* k_cache, const void* v_cache,
                                             const int64_t* page_table, int64_t P, int64_t total_len,
                                             const int64_t* seq_lens,
                                             int64_t page_size, int64_t n_pages, float scale, int64_t B, int64_t Hq,
                                             int64_t Hkv, int64_t D, void* partials, int64_t partials_bytes,
                                             void* stream) {
  if (!q && B > 0) return AQ_E_NULL;
  return attn_decode(q, nullptr, nullptr, 0, const_cast<void*>(k_cache), const_cast<void*>(v_cache), page_table, P,
                     total_len, seq_lens, page_size, n_pages, scale, nullptr, B, Hq, Hkv, D, partials, partials_bytes, stream,
                     true);
}

extern "C" int aq_rope_paged_attn_decode_partials(const void* qkv, const float* freqs, int64_t freqs_stride,
                                                  const int64_t* page_table, int64_t P, int64_t total_len,
                                                  const int64_t* seq_lens,
                                                  int64_t page_size, void* k_cache, void* v_cache, int64_t n_pages,
                                                  float scale, int64_t B, int64_t Hq, int64_t Hkv, int64_t D,
                                                  void* partials, int64_t partials_bytes, void* stream) {
  if ((!qkv || !freqs) && B > 0) return AQ_E_NULL;
  return attn_decode(nullptr, qkv, freqs, freqs_stride, k_cache, v_cache, page_table, P, total_len, seq_lens, page_size, n_pages,
                     scale, nullptr, B, Hq, Hkv, D, partials, partials_bytes, stream, true);
}

extern "C" int aq_rope_paged_attn_decode_qknorm(const void* qkv, const float* freqs, int64_t freqs_stride,
                                                const int64_t* page_table, int64_t P, int64_t total_len,
                                                const int64_t* seq_lens, int64_t page_size, void* k_cache, void* v_cache,
                                                int64_t n_pages, float scale, void* out, int64_t B, int64_t Hq,
                                                int64_t Hkv, int64_t D, const void* q_gain, const void* k_gain, float eps,
                                                void* workspace, int64_t workspace_bytes, void* stream) {
  if ((!qkv || !freqs) && B > 0) return AQ_E_NULL;
  if (!q_gain || !k_gain) return AQ_E_NULL;
  return attn_decode(nullptr, qkv, freqs, freqs_stride, k_cache, v_cache, page_table, P, total_len, seq_lens, page_size, n_pages,
                     scale, out, B, Hq, Hkv, D, workspace, workspace_bytes, stream, false, q_gain, k_gain, eps);
}

extern "C" int aq_rope_paged_attn_decode_partials_qknorm(const void* qkv, const float* freqs, int64_t freqs_stride,
                                                         const int64_t* page_table, int64_t P, int64_t total_len,
                                                         const int64_t* seq_lens, int64_t page_size, void* k_cache,
                                                         void* v_cache, int64_t n_pages, float scale, int64_t B,
                                                         int64_t Hq, int64_t Hkv, int64_t D, const void* q_gain,
                                                         const void* k_gain, float eps, void* partials,
                                                         int64_t partials_bytes, void* stream) {
  if ((!qkv || !freqs) && B > 0) return AQ_E_NULL;
  if (!q_gain || !k_gain) return AQ_E_NULL;
  return attn_decode(nullptr, qkv, freqs, freqs_stride, k_cache, v_cache, page_table, P, total_len, seq_lens, page_size, n_pages,
                     scale, nullptr, B, Hq, Hkv, D, partials, partials_bytes, stream, true, q_gain, k_gain, eps);
}
