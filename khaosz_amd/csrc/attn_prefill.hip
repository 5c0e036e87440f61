// Causal self-attention over a prompt (prefill from an empty cache): what the
// reference computes with repeat_kv + scaled_dot_product_attention
// (astrai/model/components/attention.py:15-23, 93-100) when the query and key
// positions coincide.  Grouped-query attention without repeating heads, bf16
// tensors, fp32 softmax statistics and accumulation, head dimension 64 or 128.
//
// Workgroup = (128 query positions, one query head, one sequence), 4 wavefronts
// of 32 query rows; K/V are walked in blocks of 64 positions up to the causal
// limit.  Everything is computed transposed so that no register ever has to
// change lanes:
//
//   S^T[key, q] = K Q^T    v_mfma_f32_32x32x16_bf16 with A = K (rows of the LDS
//                          tile, 16-byte reads), B = Q^T (the wavefront's query
//                          rows, held in registers for the whole kernel).  A
//                          lane ends up with the scores of ONE query (column
//                          l % 32) against 16 keys per 32-key tile.
//   softmax                per query = per lane: running maximum and denominator
//                          need one exchange with lane l ^ 32 per block, the
//                          rescale of the output accumulator is lane-wise.
//   O^T[d, q] += V^T P^T   B = P^T: the probabilities a lane already holds are,
//                          packed to bf16 in register order, exactly its operand
//                          (the matrix core does not care which key sits in which
//                          k slot as long as A agrees); A = V^T read from an LDS
//                          tile that was written transposed ([d][key]) when the
//                          block was staged, two 8-byte reads per operand.
//
// The next block's K and V are fetched into registers while the current one is
// being multiplied.
#include "aq_common.h"

namespace aq {

struct PrefillAttnArgs {
  const uint16_t* q;   // element (b, s, h, d) at q + (b*S + s)*q_stride + h*D + d
  const uint16_t* k;   // likewise with KV heads
  const uint16_t* v;
  uint16_t* out;       // [B, S, Hq, D]
  int64_t q_stride, k_stride, v_stride;  // elements between consecutive tokens
  float scale_log2e;
  int S, Hq, Hkv, B;
  // PAGED kernels: keys and values of positions 0 .. start + S - 1 are read through the page table from
  // caches [n_pages, page, Hkv, D]; query s sits at position start + s
  const uint16_t* kc;
  const uint16_t* vc;
  const int64_t* table;  // [B, P] physical page ids, < 0: unmapped (zero keys and values)
  int64_t P, page, n_pages;
  int start, page_shift;
  int paired;  // != 0: the second half of the workgroups takes the query blocks lightest first
};

typedef __bf16 pa_bf16x8 __attribute__((ext_vector_type(8)));
typedef float pa_f32x16 __attribute__((ext_vector_type(16)));

constexpr int PA_QB = 128;  // query rows per workgroup
constexpr int PA_KB = 64;   // keys per block

// Two workgroups per compute unit (2 wavefronts per SIMD, at most 256 registers each): the other workgroup's
// matrix work is what overlaps this one's softmax and staging.
// PAGED: a chunk of S new tokens on top of `start` cached ones -- K and V of all start + S positions come from the
// paged cache (the new tokens' rows have been written there already), causality is by position.
template <int D, bool PAGED = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void prefill_attn_kernel(PrefillAttnArgs p) {
  constexpr int KP = D + 8;       // K tile row pitch (elements): 16-byte reads of 32 rows hit distinct banks
  constexpr int VP = PA_KB + 4;   // V^T tile row pitch
  constexpr int DSTEPS = D / 16;  // matrix-core steps over the head dimension
  constexpr int DT = D / 32;      // 32-row tiles of the transposed output
  constexpr int CPT = PA_KB * (D / 8) / 256;  // 16-byte chunks of a K (or V) block per thread: 2 or 4
  constexpr int KS_ELEMS = PA_KB * KP, VT_ELEMS = D * VP;
  extern __shared__ __align__(16) uint16_t pa_lds[];  // [K tile | V^T tile]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 31, g = lane >> 5;
  const int S = p.S;
  // Workgroups are numbered heaviest first: a query block attends to every key block up to its own, so the
  // last block of a sequence has the most work.  All (head, sequence) pairs of the last query block come
  // first, then the block before it, ... -- the long workgroups start at once and the short ones fill in
  // behind them (in launch order the light blocks of head 0 would start first and the heavy ones of the last
  // heads would run alone at the end: 34 -> 28 us at 8 x 512, 339 -> 219 us at 4 x 2048 x 32 heads).
  // When the whole launch is resident at once (two workgroups per compute unit), the second half of the
  // numbering runs lightest first instead: the workgroup that joins a heavy one on its compute unit is then a
  // light one, and every compute unit gets the same sum (8 x 512 x 16 heads: 22.4 -> 21.6 us; with more
  // workgroups than slots the descending order is the better one, 4 x 2048 x 32 heads 186 against 194 us).
  const int nqb = (S + PA_QB - 1) / PA_QB, per = p.Hq * p.B;
  const int rank = (int)blockIdx.x / per, hrank = (nqb + 1) / 2;
  const int qblk = (p.paired && rank >= hrank) ? rank - hrank : nqb - 1 - rank;
  const int q0 = qblk * PA_QB, h = ((int)blockIdx.x % per) % p.Hq,
            b = ((int)blockIdx.x % per) / p.Hq;
  const int kvh = h / (p.Hq / p.Hkv);
  const int qw0 = q0 + wave * 32;          // first query row of this wavefront
  const int qpos = qw0 + col;              // this lane's query
  const int64_t tok0 = (int64_t)b * S;
  const int off = PAGED ? p.start : 0;     // position of query 0
  const int T = off + S;                   // key positions
  const int qw0p = qw0 + off, qposp = qpos + off;  // positions of the wavefront's first / this lane's query

  // Q^T operand: lane = (query col, dimensions 16 step + 8 g .. + 8); rows past S read row S - 1
  uint4 qf[DSTEPS];
  {
    const int qr = qpos < S ? qpos : S - 1;
    const uint16_t* src = p.q + (tok0 + qr) * p.q_stride + (int64_t)h * D + g * 8;
#pragma unroll
    for (int st = 0; st < DSTEPS; ++st) qf[st] = *reinterpret_cast<const uint4*>(src + st * 16);
  }
  // staging, fetched one block ahead: 16-byte chunks (key, 8 dimensions).  K chunks go to threads in memory
  // order (coalesced loads, row-major LDS tile).  V is written transposed; there a wavefront's lanes take
  // consecutive KEYS of one chunk column, so that the stores of an instruction fall into consecutive LDS
  // words instead of 4 banks.
  // (scalars, not arrays: the compiler kept a 4-element array of these in scratch memory)
  uint4 kreg0, kreg1, kreg2, kreg3, vreg0, vreg1, vreg2, vreg3;
  kreg2 = kreg3 = vreg2 = vreg3 = make_uint4(0, 0, 0, 0);
  // element offset of position t's row for this KV head in the paged caches, -1 when its page is unmapped
  uint32_t kneg = 0, vneg = 0;  // bit c: the row of staging chunk c is not there
  const int pshift = PAGED ? p.page_shift : 0;  // log2 of the page size, or -1 when it is not a power of two
  auto paged_row = [&](int t) -> int64_t {
    const int lp = pshift >= 0 ? t >> pshift : t / (int)p.page;
    const int in_page = pshift >= 0 ? t & ((1 << pshift) - 1) : t - lp * (int)p.page;
    const int64_t phys = p.table[(int64_t)b * p.P + lp];
    return (phys >= 0 && phys < p.n_pages) ? ((phys * p.page + in_page) * p.Hkv + kvh) * D : -1;
  };
  int64_t kro0 = -1, kro1 = -1, kro2 = -1, kro3 = -1, vro = -1;  // row offsets of the block fetched next
  auto lookup = [&](int j) __attribute__((always_inline)) {
    if constexpr (PAGED) {
      auto krow_of = [&](int c) -> int64_t {
        int kr = j * PA_KB + (c * 256 + tid) / (D / 8);
        return paged_row(kr < T ? kr : T - 1);
      };
      kro0 = krow_of(0);
      kro1 = krow_of(1);
      if constexpr (CPT > 2) {
        kro2 = krow_of(2);
        kro3 = krow_of(3);
      }
      const int vr = j * PA_KB + lane;
      vro = paged_row(vr < T ? vr : T - 1);
    }
  };
  // Direct kernel: K and V of this sequence and KV head behind buffer descriptors; a staging chunk's byte offset is
  // a lane constant (computed once) plus the block's row distance -- one add per load where a 64-bit row product
  // stood -- and rows past the sequence fall outside the descriptor and read as zero (they are masked anyway).
  __amdgpu_buffer_rsrc_t Kd = make_rsrc(nullptr, 0), Vd = make_rsrc(nullptr, 0);
  uint32_t koff[4] = {0, 0, 0, 0}, voff[4] = {0, 0, 0, 0};
  uint32_t kblk = 0, vblk = 0;  // bytes between consecutive key blocks
  if constexpr (!PAGED) {
    Kd = make_rsrc(p.k + tok0 * p.k_stride + (int64_t)kvh * D, (uint32_t)(((int64_t)(S - 1) * p.k_stride + D) * 2));
    Vd = make_rsrc(p.v + tok0 * p.v_stride + (int64_t)kvh * D, (uint32_t)(((int64_t)(S - 1) * p.v_stride + D) * 2));
    kblk = (uint32_t)(PA_KB * p.k_stride * 2);
    vblk = (uint32_t)(PA_KB * p.v_stride * 2);
#pragma unroll
    for (int c = 0; c < CPT; ++c) {
      const int idx = c * 256 + tid, key = idx / (D / 8), ch = idx % (D / 8);
      koff[c] = (uint32_t)(key * (int)p.k_stride + ch * 8) * 2u;
      voff[c] = (uint32_t)(lane * (int)p.v_stride + (wave + 4 * c) * 8) * 2u;
    }
  }
  auto fetch1 = [&](int j, int c, uint4& kr_out, uint4& vr_out) __attribute__((always_inline)) {
    const int idx = c * 256 + tid, key = idx / (D / 8), ch = idx % (D / 8);
    if constexpr (!PAGED) {
      kr_out = buffer_load_16(Kd, koff[c] + (uint32_t)j * kblk);
      vr_out = buffer_load_16(Vd, voff[c] + (uint32_t)j * vblk);
      return;
    }
    int kr = j * PA_KB + key;
    kr = kr < T ? kr : T - 1;  // past the last position: any valid row, masked by causality
    int vr = j * PA_KB + lane;
    vr = vr < T ? vr : T - 1;
    if constexpr (PAGED) {
      // the rows' offsets were looked up one block earlier (lookup below): the page-table round trip is off
      // the prefetch's path.  Rows of unmapped pages read row 0 and are zeroed when they are staged: a
      // select on the loaded value here would make every load of the prefetch wait for the one before it.
      const int64_t krow = c == 0 ? kro0 : c == 1 ? kro1 : c == 2 ? kro2 : kro3, vrow = vro;
      kr_out = *reinterpret_cast<const uint4*>(p.kc + (krow >= 0 ? krow : 0) + ch * 8);
      vr_out = *reinterpret_cast<const uint4*>(p.vc + (vrow >= 0 ? vrow : 0) + (wave + 4 * c) * 8);
      kneg = (kneg & ~(1u << c)) | ((krow < 0 ? 1u : 0u) << c);
      vneg = (vneg & ~(1u << c)) | ((vrow < 0 ? 1u : 0u) << c);
    } else {
      kr_out = *reinterpret_cast<const uint4*>(p.k + (tok0 + kr) * p.k_stride + (int64_t)kvh * D + ch * 8);
      vr_out = *reinterpret_cast<const uint4*>(p.v + (tok0 + vr) * p.v_stride + (int64_t)kvh * D + (wave + 4 * c) * 8);
    }
  };
  auto stage1 = [&](uint16_t* ks, uint16_t* vt, int c, const uint4& kr_in, const uint4& vr_in) __attribute__((always_inline)) {
    const int idx = c * 256 + tid, key = idx / (D / 8), ch = idx % (D / 8);
    uint4 kr_z = kr_in, vr_z = vr_in;
    if constexpr (PAGED) {
      if (kneg & (1u << c)) kr_z = make_uint4(0, 0, 0, 0);
      if (vneg & (1u << c)) vr_z = make_uint4(0, 0, 0, 0);
    }
    *reinterpret_cast<uint4*>(&ks[key * KP + ch * 8]) = kr_z;
    // V chunk (key = lane, dimensions 8 (wave + 4 c) .. + 8) into the transposed tile, two keys per 4-byte
    // store: neighbouring lanes swap dwords (DPP) and byte-permute them into "one dimension, both keys" --
    // even lanes then hold the even dimensions of the key pair, odd lanes the odd ones.
    const bool odd = lane & 1;
    const uint32_t sel = odd ? 0x03020706u : 0x05040100u;
    uint32_t* vdst = reinterpret_cast<uint32_t*>(&vt[((wave + 4 * c) * 8 + (odd ? 1 : 0)) * VP + (lane & ~1)]);
    const uint32_t w[4] = {vr_z.x, vr_z.y, vr_z.z, vr_z.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t other = (uint32_t)__builtin_amdgcn_mov_dpp((int)w[e], 0xB1 /* quad_perm [1,0,3,2] */, 0xf, 0xf, true);
      // even lane: {mine.lo, other.lo} = dimension 2e of keys (lane, lane + 1); odd: {other.hi, mine.hi} = 2e + 1
      vdst[e * VP] = __builtin_amdgcn_perm(other, w[e], sel);  // e * VP words = 2e rows of VP halfwords
    }
  };
#define PA_FETCH(J)                        \
  fetch1((J), 0, kreg0, vreg0);            \
  fetch1((J), 1, kreg1, vreg1);            \
  if constexpr (CPT > 2) {                 \
    fetch1((J), 2, kreg2, vreg2);          \
    fetch1((J), 3, kreg3, vreg3);          \
  }
#define PA_STAGE(BUF)                                                        \
  {                                                                          \
    uint16_t* ks_w = pa_lds + (BUF) * (KS_ELEMS + VT_ELEMS);                  \
    uint16_t* vt_w = ks_w + KS_ELEMS;                                        \
    stage1(ks_w, vt_w, 0, kreg0, vreg0);                                     \
    stage1(ks_w, vt_w, 1, kreg1, vreg1);                                     \
    if constexpr (CPT > 2) {                                                 \
      stage1(ks_w, vt_w, 2, kreg2, vreg2);                                   \
      stage1(ks_w, vt_w, 3, kreg3, vreg3);                                   \
    }                                                                        \
  }

  pa_f32x16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[dt][r] = 0.0f;
  float m = -INFINITY, l = 0.0f;  // running maximum of this lane's query; this lane's half of its denominator

  const int last_q = (q0 + PA_QB < S ? q0 + PA_QB : S) - 1 + off;  // position of the workgroup's last query
  const int nblk = last_q / PA_KB + 1;  // blocks that hold a key some query of the workgroup may see
  // One LDS buffer, two barriers per block; the next block's global loads are in flight while this one is
  // multiplied.  (Two buffers with one barrier per block measured 15 % slower.)
  const uint16_t* ks = pa_lds;
  const uint16_t* vt = pa_lds + KS_ELEMS;
  lookup(0);
  PA_FETCH(0)
  if (nblk > 1) lookup(1);
  for (int j = 0; j < nblk; ++j) {
    __syncthreads();  // everyone is done reading the previous block's tiles
    PA_STAGE(0)
    __syncthreads();
    if (j + 1 < nblk) {
      PA_FETCH(j + 1)
      if (j + 2 < nblk) lookup(j + 2);
    }
    const int kb0 = j * PA_KB;
    if (kb0 > qw0p + 31) continue;  // wavefront-uniform: every key of the block is ahead of every query here
    // ---- scores, transposed: two tiles of 32 keys
    // The K fragments are read two dimension steps ahead of the products that take them, and the two tiles'
    // accumulation chains alternate: left to itself the compiler put every LDS read right in front of its MFMA
    // (one LDS round trip per product, sixteen in a row) and ran the second tile's chain after the first's.
    // Each chain still adds its steps in ascending order: same bits.
    pa_f32x16 s[2];
    {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[0][r] = s[1][r] = 0.0f;
      const uint16_t* k0 = &ks[col * KP + g * 8];
      const uint16_t* k1 = k0 + 32 * KP;
      constexpr int GRP = 2, NG = DSTEPS / GRP;
      static_assert(DSTEPS % GRP == 0, "whole groups of dimension steps");
      uint4 fa[2][GRP][2];
      auto ldk = [&](int buf, int st0) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < GRP; ++i) {
          fa[buf][i][0] = *reinterpret_cast<const uint4*>(k0 + (st0 + i) * 16);
          fa[buf][i][1] = *reinterpret_cast<const uint4*>(k1 + (st0 + i) * 16);
        }
      };
      ldk(0, 0);
      if (NG > 1) ldk(1, GRP);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int gi = 0; gi < NG; ++gi) {
#pragma unroll
        for (int i = 0; i < GRP; ++i) {
          const pa_bf16x8 qv = __builtin_bit_cast(pa_bf16x8, qf[gi * GRP + i]);
          s[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pa_bf16x8, fa[gi & 1][i][0]), qv, s[0], 0, 0, 0);
          s[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pa_bf16x8, fa[gi & 1][i][1]), qv, s[1], 0, 0, 0);
        }
        if (gi + 2 < NG) ldk(gi & 1, (gi + 2) * GRP);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // ---- online softmax for this lane's query; register r of tile kt is key kb0 + 32 kt + 8 (r / 4) + 4 g + r % 4.
    // Scores stay unscaled; the scale (> 0) is applied to the maximum and inside the exponent's fma.
    const bool diag = kb0 + PA_KB - 1 > qw0p;  // wavefront-uniform: some key of the block is ahead of some query
    float bm = -INFINITY;
    if (diag) {  // a branch, not 32 compares and selects in every block: most blocks lie wholly behind the queries
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (kb0 + kt * 32 + 8 * (r / 4) + 4 * g + (r % 4) > qposp) s[kt][r] = -INFINITY;
    }
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int r = 0; r < 16; ++r) bm = fmaxf(bm, s[kt][r]);
    bm = fmaxf(bm, __shfl_xor(bm, 32, 64)) * p.scale_log2e;
    // The running maximum only has to bound the exponents, not equal the true maximum: it is raised (and the
    // accumulators rescaled) only when some query of the wavefront would otherwise see an exponent above 2^8;
    // with probabilities up to 256 nothing overflows and bf16 keeps its relative precision.  After the first
    // blocks this is rare, and the 64-register rescale is skipped.
    const bool raise = __builtin_amdgcn_ballot_w64(bm > m + 8.0f) != 0;  // m = -inf in block 0: raised there
    float alpha = 1.0f;
    if (raise) {
      const float mn = fmaxf(m, bm);  // finite from block 0 on: key 0 is visible to every query
      alpha = __builtin_amdgcn_exp2f(m - mn);
      m = mn;
      l *= alpha;
    }
    float ps = 0.0f;
    uint4 pf[2][2];  // P^T operands: tile kt, keys 16 s2 .. + 16
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      float pv[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        pv[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][r], p.scale_log2e, -m));
        ps += pv[r];
      }
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
        pf[kt][s2] = make_uint4(pack_bf16x2(pv[8 * s2 + 0], pv[8 * s2 + 1]), pack_bf16x2(pv[8 * s2 + 2], pv[8 * s2 + 3]),
                                pack_bf16x2(pv[8 * s2 + 4], pv[8 * s2 + 5]), pack_bf16x2(pv[8 * s2 + 6], pv[8 * s2 + 7]));
    }
    l += ps;
    // ---- output, transposed: O^T[d, q] = alpha O^T + V^T P^T
    if (raise) {  // one branch for all tiles (a branch per tile kept the tiles' products apart)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
    }
    // V^T fragments of two dimension tiles at a time, all read before the pair's products, whose two chains
    // alternate; each chain adds its four key groups in ascending order: same bits.
    {
      uint4 fv[DT][4];
      auto ldv = [&](int dt) __attribute__((always_inline)) {
        const uint16_t* vrow = &vt[(dt * 32 + col) * VP + 4 * g];
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          // k slots of this lane group: keys 32 kt + 16 s2 + {4 g .. + 4, 8 + 4 g .. + 4}, kk = 2 kt + s2
          const uint2 lo = *reinterpret_cast<const uint2*>(vrow + kk * 16);
          const uint2 hi = *reinterpret_cast<const uint2*>(vrow + kk * 16 + 8);
          fv[dt][kk] = make_uint4(lo.x, lo.y, hi.x, hi.y);
        }
      };
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) ldv(dt);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int d0 = 0; d0 < DT; d0 += 2) {
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          const pa_bf16x8 pv8 = __builtin_bit_cast(pa_bf16x8, pf[kk >> 1][kk & 1]);
          o[d0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pa_bf16x8, fv[d0][kk]), pv8, o[d0], 0, 0, 0);
          o[d0 + 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pa_bf16x8, fv[d0 + 1][kk]), pv8, o[d0 + 1], 0, 0, 0);
        }
      }
    }
  }
  // ---- normalise and store: register r of tile dt is dimension 32 dt + 8 (r / 4) + 4 g + r % 4 of query col
  l += __shfl_xor(l, 32, 64);
  if (qpos < S) {
    const float inv = 1.0f / l;
    uint16_t* dst = p.out + ((tok0 + qpos) * p.Hq + h) * D + 4 * g;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        uint2 w;
        w.x = pack_bf16x2(o[dt][4 * a + 0] * inv, o[dt][4 * a + 1] * inv);
        w.y = pack_bf16x2(o[dt][4 * a + 2] * inv, o[dt][4 * a + 3] * inv);
        *reinterpret_cast<uint2*>(dst + dt * 32 + 8 * a) = w;
      }
  }
}

#undef PA_FETCH
#undef PA_STAGE

}  // namespace aq

extern "C" int aq_prefill_attn_causal(const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                                      int64_t v_stride, void* out, float scale, int64_t B, int64_t S, int64_t Hq,
                                      int64_t Hkv, int64_t D, void* stream) {
  if (D != 64 && D != 128) return AQ_E_SHAPE;
  if (B < 0 || S < 0 || Hq <= 0 || Hkv <= 0 || (Hq % Hkv) != 0 || !(scale > 0.0f)) return AQ_E_SHAPE;
  if (q_stride < Hq * D || k_stride < Hkv * D || v_stride < Hkv * D) return AQ_E_SHAPE;
  if (B == 0 || S == 0) return AQ_OK;
  if (!q || !k || !v || !out) return AQ_E_NULL;
  if (aq::check_ptr16(q) || aq::check_ptr16(k) || aq::check_ptr16(v) || aq::check_ptr16(out) || (q_stride & 7) ||
      (k_stride & 7) || (v_stride & 7))
    return AQ_E_ALIGN;
  if (S > (1 << 30) || Hq > 65535 || B > 65535 || ((S + aq::PA_QB - 1) / aq::PA_QB) * Hq * B > (int64_t)0x7fffffff)
    return AQ_E_RANGE;
  // 32-bit byte offsets inside one sequence's K and V (a key block past the end included)
  if ((S + aq::PA_KB) * k_stride * 2 > (int64_t)0x7fffffff || (S + aq::PA_KB) * v_stride * 2 > (int64_t)0x7fffffff)
    return AQ_E_RANGE;
  aq::PrefillAttnArgs a{};
  a.q = static_cast<const uint16_t*>(q);
  a.k = static_cast<const uint16_t*>(k);
  a.v = static_cast<const uint16_t*>(v);
  a.out = static_cast<uint16_t*>(out);
  a.q_stride = q_stride;
  a.k_stride = k_stride;
  a.v_stride = v_stride;
  a.scale_log2e = scale * 1.44269504088896341f;
  a.S = (int)S;
  a.Hq = (int)Hq;
  a.Hkv = (int)Hkv;
  a.B = (int)B;
  const dim3 grid((unsigned)(((S + aq::PA_QB - 1) / aq::PA_QB) * Hq * B));
  a.paired = grid.x <= 2u * (unsigned)aq::device_cus();
  hipStream_t st = static_cast<hipStream_t>(stream);
  const size_t lds = (size_t)(aq::PA_KB * (D + 8) + D * (aq::PA_KB + 4)) * sizeof(uint16_t);  // 34 KiB at most
  if (D == 128)
    hipLaunchKernelGGL((aq::prefill_attn_kernel<128, false>), grid, dim3(256), lds, st, a);
  else
    hipLaunchKernelGGL((aq::prefill_attn_kernel<64, false>), grid, dim3(256), lds, st, a);
  return (int)hipGetLastError();
}

extern "C" int aq_prefill_attn_paged(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                                     const int64_t* page_table, int64_t P, int64_t start, int64_t page_size,
                                     int64_t n_pages, void* out, float scale, int64_t B, int64_t S, int64_t Hq,
                                     int64_t Hkv, int64_t D, void* stream) {
  if (D != 64 && D != 128) return AQ_E_SHAPE;
  if (B < 0 || S < 0 || start < 0 || Hq <= 0 || Hkv <= 0 || (Hq % Hkv) != 0 || P <= 0 || page_size <= 0 ||
      n_pages <= 0 || !(scale > 0.0f) || q_stride < Hq * D)
    return AQ_E_SHAPE;
  if (start + S > P * page_size) return AQ_E_SHAPE;  // positions the page table does not cover
  if (B == 0 || S == 0) return AQ_OK;
  if (!q || !k_cache || !v_cache || !page_table || !out) return AQ_E_NULL;
  if (aq::check_ptr16(q) || aq::check_ptr16(k_cache) || aq::check_ptr16(v_cache) || aq::check_ptr16(out) ||
      (q_stride & 7))
    return AQ_E_ALIGN;
  if (start + S > (1 << 30) || Hq > 65535 || B > 65535 ||
      ((S + aq::PA_QB - 1) / aq::PA_QB) * Hq * B > (int64_t)0x7fffffff)
    return AQ_E_RANGE;
  aq::PrefillAttnArgs a{};
  a.q = static_cast<const uint16_t*>(q);
  a.out = static_cast<uint16_t*>(out);
  a.q_stride = q_stride;
  a.kc = static_cast<const uint16_t*>(k_cache);
  a.vc = static_cast<const uint16_t*>(v_cache);
  a.table = page_table;
  a.P = P;
  a.page = page_size;
  a.n_pages = n_pages;
  a.start = (int)start;
  a.page_shift = -1;
  for (int sh = 0; sh < 31; ++sh)
    if (page_size == ((int64_t)1 << sh)) a.page_shift = sh;
  a.scale_log2e = scale * 1.44269504088896341f;
  a.S = (int)S;
  a.Hq = (int)Hq;
  a.Hkv = (int)Hkv;
  a.B = (int)B;
  const dim3 grid((unsigned)(((S + aq::PA_QB - 1) / aq::PA_QB) * Hq * B));
  a.paired = grid.x <= 2u * (unsigned)aq::device_cus();
  hipStream_t st = static_cast<hipStream_t>(stream);
  const size_t lds = (size_t)(aq::PA_KB * (D + 8) + D * (aq::PA_KB + 4)) * sizeof(uint16_t);
  if (D == 128)
    hipLaunchKernelGGL((aq::prefill_attn_kernel<128, true>), grid, dim3(256), lds, st, a);
  else
    hipLaunchKernelGGL((aq::prefill_attn_kernel<64, true>), grid, dim3(256), lds, st, a);
  return (int)hipGetLastError();
}
