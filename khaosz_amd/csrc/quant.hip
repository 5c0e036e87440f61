// Activation / weight quantisation kernels for gfx950: symmetric absmax int8
// per row and per-tensor FP8 (OCP e4m3fn).  Both are HBM-bound streaming
// kernels: 16-byte loads per lane, one wavefront per row, wavefront-wide
// absmax through cross-lane shuffles, no LDS.
#include <type_traits>

#include "aq_common.h"
#include "aq_rows.h"

namespace aq {

// ---------------------------------------------------------------- int8 rows

template <bool BF16>
__device__ __forceinline__ void quant_store(const uint4& v, float s, float rs, bool fast_ok, int8_t* dst) {
  constexpr int EPV = RowIn<BF16>::EPV;
  float f[EPV];
  uint32_t c[EPV / 4];
  RowIn<BF16>::unpack(v, f);
  quant_codes_packed<EPV, quant_steps<BF16, false>()>(f, s, rs, fast_ok, c);
  if constexpr (BF16) {
    store_wt(reinterpret_cast<uint2*>(dst), make_uint2(c[0], c[1]));
  } else {
    store_wt(reinterpret_cast<uint32_t*>(dst), c[0]);
  }
}

// One wavefront per row at a time.  The first NC vectors of the lane stay in
// registers between the absmax pass and the rounding pass; longer rows are
// re-read (from L2) for the part that does not fit.  A wavefront walks rows
// row0, row0 + stride, ... and, when PREFETCH, requests the next row's vectors
// before it reduces, rounds and stores the current one, so that the reads of
// one row overlap the arithmetic and the writes of another (all wavefronts of a
// one-row-per-wavefront launch start together and would otherwise read, then
// compute, then write in lockstep).
template <bool BF16, int NC, bool PREFETCH, bool FULL>
__global__ __launch_bounds__(256) void quant_rowwise_i8_kernel(const void* __restrict__ x, int64_t M,
                                                                 int K, int64_t ldx,
                                                                 int8_t* __restrict__ q,
                                                                 float* __restrict__ scale) {
  constexpr int EPV = RowIn<BF16>::EPV;
  const int lane = threadIdx.x & 63;
  const int64_t stride = (int64_t)gridDim.x * 4;
  int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const int nvec = K / EPV;  // 16-byte vectors per row
  auto row_src = [&](int64_t r) {
    return reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(x) + r * ldx * (BF16 ? 2 : 4));
  };
  auto load_cache = [&](int64_t r, uint4 (&c)[NC]) {
    const uint4* src = row_src(r);
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const int v = i * 64 + lane;
      if (FULL || v < nvec) c[i] = src[v];
    }
  };
  auto process = [&](int64_t r, const uint4 (&c)[NC]) {
    const uint4* src = row_src(r);
    int8_t* dst = q + r * (int64_t)K;
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      if (FULL || i * 64 + lane < nvec) {
        float f[EPV];
        RowIn<BF16>::unpack(c[i], f);
        amax = fmaxf(amax, vec_amax<EPV>(f));
      }
    }
    if constexpr (!FULL) {
      for (int v = NC * 64 + lane; v < nvec; v += 64) {
        float f[EPV];
        RowIn<BF16>::unpack(src[v], f);
        amax = fmaxf(amax, vec_amax<EPV>(f));
      }
    }
    amax = wave_max(amax);
    const RowScale rsc = row_scale<quant_steps<BF16, false>()>(amax);
    const float s = rsc.s, rs = rsc.rs;
    const bool fast_ok = rsc.fast_ok;
    if (lane == 0) scale[r] = s;
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const int v = i * 64 + lane;
      if (FULL || v < nvec) quant_store<BF16>(c[i], s, rs, fast_ok, dst + (int64_t)v * EPV);
    }
    if constexpr (!FULL) {
      for (int v = NC * 64 + lane; v < nvec; v += 64)
        quant_store<BF16>(src[v], s, rs, fast_ok, dst + (int64_t)v * EPV);
    }
  };

  if constexpr (PREFETCH) {
    uint4 cur[NC], nxt[NC];
    load_cache(row, cur);
    while (true) {
      const int64_t r1 = row + stride;
      if (r1 < M) load_cache(r1, nxt);  // uniform per wavefront
      process(row, cur);
      if (r1 >= M) break;
#pragma unroll
      for (int i = 0; i < NC; ++i) cur[i] = nxt[i];
      row = r1;
    }
  } else {
    for (; row < M; row += stride) {
      uint4 c[NC];
      load_cache(row, c);
      process(row, c);
    }
  }
}

// One workgroup (4 wavefronts) per row, for rows long enough to feed 256 lanes.
// A lane holds NV 16-byte vectors; the row maximum is combined across the four
// wavefronts through LDS.  Compared with one wavefront per row this quarters
// the work that remains after a row's last byte has arrived, which is what
// bounds a launch whose rows are all requested at once.
template <bool BF16, int NV>
__global__ __launch_bounds__(256) void quant_row_wg_kernel(const void* __restrict__ x, int K, int64_t ldx,
                                                            int8_t* __restrict__ q, float* __restrict__ scale) {
  constexpr int EPV = RowIn<BF16>::EPV;
  __shared__ float wmax[4];
  const int tid = threadIdx.x;
  const int64_t row = blockIdx.x;
  const int nvec = K / EPV;
  const uint4* src =
      reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(x) + row * ldx * (BF16 ? 2 : 4));
  int8_t* dst = q + row * (int64_t)K;
  uint4 c[NV];
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = i * 256 + tid;
    if (v < nvec) c[i] = src[v];
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if (i * 256 + tid < nvec) {
      float f[EPV];
      RowIn<BF16>::unpack(c[i], f);
      amax = fmaxf(amax, vec_amax<EPV>(f));
    }
  }
  amax = wave_max(amax);
  if ((tid & 63) == 0) wmax[tid >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
  const RowScale rsc = row_scale<quant_steps<BF16, false>()>(amax);
  const float s = rsc.s, rs = rsc.rs;
  const bool fast_ok = rsc.fast_ok;
  if (tid == 0) scale[row] = s;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = i * 256 + tid;
    if (v < nvec) quant_store<BF16>(c[i], s, rs, fast_ok, dst + (int64_t)v * EPV);
  }
}

// -------------------------------------------------- RMSNorm -> row quantise
//
// y = x * (1 / sqrt(mean(x^2) + eps)) * gamma, quantised per row exactly like
// quant_rowwise_i8 would quantise y held in fp32 (no bf16 rounding in between).
// The sum of squares has a fixed order so that the result does not depend on
// the launch: lane l of the row's wavefront adds x*x (a rounded product, then a
// rounded add) over its 16-byte vectors l, l + 64, ... in ascending order,
// elements in memory order, and the 64 partial sums are combined by the
// butterfly p[l] += p[l ^ 1], ^2, ^4, ^8, ^16, ^32.  mean = ss / K,
// r = 1 / sqrt(mean + eps) with correctly rounded divide and square root,
// y = (x * r) * gamma as two rounded products.
// One wavefront per row; a lane keeps its NC vectors of the row in registers
// across the three passes (sum of squares, absmax of y, rounding).  GREG: the
// lane's gamma vectors are loaded once and kept too (short rows); otherwise
// they are re-read, from L2, in both passes over y.
template <bool BF16, int NC, bool GREG>
__global__ __launch_bounds__(256) void rmsnorm_quant_kernel(const void* __restrict__ x, const void* __restrict__ gamma,
                                                            float eps, int64_t M, int K, int64_t ldx,
                                                            int8_t* __restrict__ q, float* __restrict__ scale) {
  constexpr int EPV = RowIn<BF16>::EPV;
  const int lane = threadIdx.x & 63;
  const int64_t stride = (int64_t)gridDim.x * 4;
  const int nvec = K / EPV;
  const uint4* gsrc = reinterpret_cast<const uint4*>(gamma);
  uint4 gv[GREG ? NC : 1];
  if constexpr (GREG) {
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const int v = i * 64 + lane;
      gv[i] = v < nvec ? gsrc[v] : make_uint4(0, 0, 0, 0);
    }
  }
  const float kf = (float)K;
  for (int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); row < M; row += stride) {
    const uint4* src = reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(x) + row * ldx * (BF16 ? 2 : 4));
    uint4 c[NC];
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const int v = i * 64 + lane;
      c[i] = v < nvec ? src[v] : make_uint4(0, 0, 0, 0);  // zeros add nothing to any of the passes
    }
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      float f[EPV];
      RowIn<BF16>::unpack(c[i], f);
#pragma unroll
      for (int e = 0; e < EPV; ++e) ss = __fadd_rn(ss, __fmul_rn(f[e], f[e]));
    }
    ss = wave_sum_butterfly(ss);
    const float r = rms_scale(ss, kf, eps);
    auto normed = [&](int i, float* y) {
      float f[EPV], g[EPV];
      RowIn<BF16>::unpack(c[i], f);
      const int v = i * 64 + lane;
      RowIn<BF16>::unpack(GREG ? gv[GREG ? i : 0] : (v < nvec ? gsrc[v] : make_uint4(0, 0, 0, 0)), g);
#pragma unroll
      for (int e = 0; e < EPV; ++e) y[e] = __fmul_rn(__fmul_rn(f[e], r), g[e]);
    };
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      float y[EPV];
      normed(i, y);
      amax = fmaxf(amax, vec_amax<EPV>(y));
    }
    const RowScale rsc = row_scale(wave_max(amax));
    if (lane == 0) scale[row] = rsc.s;
    int8_t* dst = q + row * (int64_t)K;
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const int v = i * 64 + lane;
      if (v < nvec) {
        float y[EPV];
        uint32_t code[EPV / 4];
        normed(i, y);
        quant_codes_packed<EPV>(y, rsc.s, rsc.rs, rsc.fast_ok, code);
        if constexpr (BF16) {
          uint2 o;
          o.x = code[0];
          o.y = code[1];
          store_wt(reinterpret_cast<uint2*>(dst + (int64_t)v * EPV), o);
        } else {
          store_wt(reinterpret_cast<uint32_t*>(dst + (int64_t)v * EPV), code[0]);
        }
      }
    }
  }
}

// ------------------------------------------------ SwiGLU -> row quantise
//
// h = up * silu(gate) for one row of the fused up/gate projection's output
// ([up | gate], 2 F columns), quantised per row like any fp32 row: the codes and
// scales the down projection consumes.  Replaces the activation, the product and
// the quantiser launches (three passes over [M, F]) by one.  A lane first turns
// its NC vector pairs into h (fp32, kept in registers; the inputs die as it goes),
// then reduces the absmax and rounds.
//
// The kernel is bound by its vector arithmetic (about 34 operations per element at first: the exponential's
// polynomial, a correctly rounded divide, the two-correction rounding; 4096 x 5632 was 20 us of it at 2.4 GHz),
// so the work went into keeping the vector ALUs fed and into the operation count:
//  * every load of a row is requested up front, pair by pair (up vector, gate vector), and the arithmetic walks
//    the pairs in that order, waiting for one pair at a time (loads return in request order).  A row's first pair
//    arrives within a microsecond and the rest streams in behind the arithmetic.  (Left to itself the compiler
//    waited for the whole row before the first operation; with only a few pairs requested ahead, a wavefront's
//    time was the memory latency times its pairs.)
//  * the divide is div_midrange (11 instead of 14 operation slots; 9 for bf16 gates, div_bf16_gate) whenever the
//    row's gates allow it, which is tested on the raw bf16 pairs with packed 16-bit operations; a row with a gate
//    outside is done again with the general divide, out of line; the exponential goes without its argument clamp
//    for such rows, and the rounding add packs its own byte (quant_codes_packed).
//  * NC is the row's own number of vector pairs per lane (a pair past the row would cost its full arithmetic).
// Four wavefronts fit a SIMD (128 registers: a row's h is 88 of them at F = 5632); the SIMD serves the oldest
// first, so a compute unit's 16 rows finish one after the other, 4096 x 5632 bf16 in 26.2 us (at first: 31.5).
template <bool BF16, int NC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4))) void swiglu_quant_kernel(
    const void* __restrict__ ug, int64_t M, int F, int64_t ld, int8_t* __restrict__ q, float* __restrict__ scale) {
  constexpr int EPV = RowIn<BF16>::EPV;
  const int lane = threadIdx.x & 63;
  const int64_t stride = (int64_t)gridDim.x * 4;
  const int nvec = F / EPV;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar: the row's descriptors live in SGPRs
  for (int64_t row = (int64_t)blockIdx.x * 4 + wave; row < M; row += stride) {
    // descriptors over the row's two halves: vectors past the row read as zeros.  (Buffer loads also stay where
    // they are written, between the scheduling barriers below: plain loads of read-only memory moved freely.)
    const char* up = reinterpret_cast<const char*>(ug) + row * ld * (BF16 ? 2 : 4);
    const uint32_t half_bytes = (uint32_t)F * (BF16 ? 2u : 4u);
    const __amdgpu_buffer_rsrc_t Ur = make_rsrc(up, half_bytes), Gr = make_rsrc(up + half_bytes, half_bytes);
    uint4 cu[NC], cg[NC];
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const uint32_t off = (uint32_t)(i * 64 + lane) * 16u;
      cu[i] = buffer_load_16(Ur, off);
      cg[i] = buffer_load_16(Gr, off);
      __builtin_amdgcn_sched_barrier(0);  // pair by pair (the scheduler would put all up halves in front of all gate halves)
    }
    asm volatile("" ::: "memory");
    float h[NC][EPV];
    float amax = 0.0f;
    bool ok = true;
    GateRangeBf16 range;
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      float u[EPV], g[EPV];
      RowIn<BF16>::unpack(cu[i], u);
      RowIn<BF16>::unpack(cg[i], g);
      // (a last pair that lies partly past the row's end reads zeros there: h = 0 * silu(0) = 0)
      if constexpr (BF16)
        range.add(cg[i]);
      else
        ok &= gates_midrange<EPV>(g);
      swiglu_group_midrange<EPV, false, BF16>(u, g, h[i]);
      amax = fmaxf(amax, vec_amax<EPV>(h[i]));
      // h is wanted HERE: left to itself the compiler takes the range checks of all pairs (which need the gates only)
      // and the branch on them first, and requests each pair's up half inside the branch, one by one
      if constexpr (BF16)
        asm volatile("" ::"v"(h[i][0]), "v"(h[i][1]), "v"(h[i][2]), "v"(h[i][3]), "v"(h[i][4]), "v"(h[i][5]), "v"(h[i][6]), "v"(h[i][7]));
      else
        asm volatile("" ::"v"(h[i][0]), "v"(h[i][1]), "v"(h[i][2]), "v"(h[i][3]));
      __builtin_amdgcn_sched_barrier(0);  // pairs in the order they were requested, which is the order they arrive in
    }
    int8_t* dst = q + row * (int64_t)F;
    if constexpr (BF16) ok = range.ok();
    if (__builtin_amdgcn_ballot_w64(!ok) != 0) {
      // Some gate of the row lies outside the range of the short divide (an outlier beyond +-80, a denormal):
      // rare, so the row is simply done again with the general divide, in two rolled loops that keep nothing in
      // registers (maximum, then codes) and leave the main path's register budget alone.
      float am = 0.0f;
      for (int i = 0; i < NC; ++i) {
        const uint32_t off = (uint32_t)(i * 64 + lane) * 16u;
        float u[EPV], g[EPV];
        RowIn<BF16>::unpack(buffer_load_16(Ur, off), u);
        RowIn<BF16>::unpack(buffer_load_16(Gr, off), g);
#pragma unroll
        for (int e = 0; e < EPV; ++e) am = fmaxf(am, fabsf(swiglu_repro(u[e], g[e])));
      }
      const RowScale rsc = row_scale(wave_max(am));
      if (lane == 0) scale[row] = rsc.s;
      for (int i = 0; i < NC; ++i) {
        const int v = i * 64 + lane;
        const uint32_t off = (uint32_t)v * 16u;
        float u[EPV], g[EPV], hh[EPV];
        uint32_t code[EPV / 4];
        RowIn<BF16>::unpack(buffer_load_16(Ur, off), u);
        RowIn<BF16>::unpack(buffer_load_16(Gr, off), g);
#pragma unroll
        for (int e = 0; e < EPV; ++e) hh[e] = swiglu_repro(u[e], g[e]);
        quant_codes_packed<EPV>(hh, rsc.s, rsc.rs, rsc.fast_ok, code);
        if (v < nvec) {
          if constexpr (BF16) {
            uint2 o;
            o.x = code[0];
            o.y = code[1];
            store_wt(reinterpret_cast<uint2*>(dst + (int64_t)v * EPV), o);
          } else {
            store_wt(reinterpret_cast<uint32_t*>(dst + (int64_t)v * EPV), code[0]);
          }
        }
      }
      continue;
    }
    const RowScale rsc = row_scale(wave_max(amax));
    if (lane == 0) scale[row] = rsc.s;
    // codes through a descriptor over the row (written through, like store_wt): one lane offset for the whole
    // row and the vector's position as a constant, instead of a 64-bit address per store; what lies past the
    // row falls outside the descriptor and is dropped
    const __amdgpu_buffer_rsrc_t Qr = make_rsrc(dst, (uint32_t)F);
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      uint32_t code[EPV / 4];
      quant_codes_packed<EPV>(h[i], rsc.s, rsc.rs, rsc.fast_ok, code);
      if constexpr (BF16) {
        typedef int v2i_t __attribute__((ext_vector_type(2)));
        const v2i_t o = {(int)code[0],
                         (int)code[1]};
        __builtin_amdgcn_raw_buffer_store_b64(o, Qr, lane * 8, i * 512, STORE_WT);
      } else {
        __builtin_amdgcn_raw_buffer_store_b32((int)code[0], Qr, lane * 4,
                                              i * 256, STORE_WT);
      }
    }
  }
}

// The same with a workgroup per row, one vector pair per thread: with few rows a
// wavefront per row leaves the device empty while each lane works through a
// dozen vector pairs of exponentials.  The row maximum crosses the wavefronts
// through LDS; a maximum does not depend on the order, so codes and scales are
// the same bits as the kernel above gives.
template <bool BF16>
__global__ __launch_bounds__(1024) void swiglu_quant_wg_kernel(const void* __restrict__ ug, int F, int64_t ld,
                                                               int8_t* __restrict__ q, float* __restrict__ scale) {
  constexpr int EPV = RowIn<BF16>::EPV;
  __shared__ float wmax[16];
  const int v = threadIdx.x, lane = v & 63, wave = v >> 6, nwaves = blockDim.x >> 6;
  const int nvec = F / EPV;
  const int64_t row = blockIdx.x;
  const uint4* up = reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(ug) + row * ld * (BF16 ? 2 : 4));
  const uint4* gate = up + nvec;
  const uint4 cu = v < nvec ? up[v] : make_uint4(0, 0, 0, 0);
  const uint4 cg = v < nvec ? gate[v] : make_uint4(0, 0, 0, 0);
  float u[EPV], g[EPV], h[EPV];
  RowIn<BF16>::unpack(cu, u);
  RowIn<BF16>::unpack(cg, g);
  swiglu_group_midrange<EPV>(u, g, h);
  if (__builtin_amdgcn_ballot_w64(!gates_midrange<EPV>(g)) != 0) {  // a gate outside the short divide's range: again
#pragma unroll
    for (int e = 0; e < EPV; ++e) h[e] = swiglu_repro(u[e], g[e]);
  }
  const float wm = wave_max(vec_amax<EPV>(h));
  if (lane == 0) wmax[wave] = wm;
  __syncthreads();
  // one LDS read per lane and a wavefront maximum, not a loop of dependent reads (at most 16 wavefronts)
  const float amax = wave_max(lane < nwaves ? wmax[lane] : 0.0f);
  const RowScale rsc = row_scale(amax);
  if (v == 0) scale[row] = rsc.s;
  if (v < nvec) {
    int8_t* dst = q + row * (int64_t)F;
    uint32_t code[EPV / 4];
    quant_codes_packed<EPV>(h, rsc.s, rsc.rs, rsc.fast_ok, code);
    if constexpr (BF16) {
      uint2 o;
      o.x = code[0];
      o.y = code[1];
      store_wt(reinterpret_cast<uint2*>(dst + (int64_t)v * EPV), o);
    } else {
      store_wt(reinterpret_cast<uint32_t*>(dst + (int64_t)v * EPV), code[0]);
    }
  }
}

// ---------------------------------------------------------------- FP8 tensor

constexpr int FP8_BATCH = 4;  // 16-byte loads a thread keeps in flight in the per-tensor passes
constexpr int AMAX_THREADS = 1024;  // few, large workgroups: the pass ends with one partial maximum per workgroup
constexpr int AMAX_SLOTS = AQ_FP8_AMAX_WS_BYTES / 4;  // partial maxima in the workspace

// Pass 1: every workgroup leaves the maximum of its share in its own workspace slot (the launcher fills
// all AMAX_SLOTS slots: workgroups past the data write 0).  No atomics and nothing to reset: the
// workspace needs no initial value and a call leaves no state behind, so the whole quantisation is two
// launches.  (A single slot updated with atomicMax needed a third launch to clear it, and same-address
// atomics from 8 XCDs serialise at about 15 ns each.)
template <bool BF16>
__global__ __launch_bounds__(AMAX_THREADS) void amax_kernel(const void* __restrict__ x, int64_t nvec,
                                                    uint32_t* __restrict__ amax_slots) {
  constexpr int EPV = RowIn<BF16>::EPV;
  const uint4* src = reinterpret_cast<const uint4*>(x);
  float amax = 0.0f;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  // FP8_BATCH independent 16-byte loads in flight per thread; indices past the end re-read the
  // last vector, which cannot change a maximum
  for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < nvec; v += FP8_BATCH * stride) {
    uint4 t[FP8_BATCH];
#pragma unroll
    for (int u = 0; u < FP8_BATCH; ++u) {
      const int64_t i = v + u * stride;
      t[u] = src[i < nvec ? i : nvec - 1];
    }
#pragma unroll
    for (int u = 0; u < FP8_BATCH; ++u) {
      float f[EPV];
      RowIn<BF16>::unpack(t[u], f);
      amax = fmaxf(amax, vec_amax<EPV>(f));
    }
  }
  amax = wave_max(amax);
  // one atomic per workgroup: same-address atomics serialise at the L2
  __shared__ float wmax[AMAX_THREADS / 64];
  if ((threadIdx.x & 63) == 0) wmax[threadIdx.x >> 6] = amax;
  __syncthreads();
  if (threadIdx.x == 0) {
    float m = 0.0f;
#pragma unroll
    for (int w = 0; w < AMAX_THREADS / 64; ++w) m = fmaxf(m, wmax[w]);
    amax_slots[blockIdx.x] = __float_as_uint(m);
  }
}

// x / s clamped to the e4m3 range.  For scales in [2^-64, 2^64] the short sequences of quant_codes
// (aq_common.h) stand in for the correctly rounded divide, whose vector operations had made this kernel
// ALU-bound: with STEPS = 2, rs = the once-refined hardware reciprocal and the result is fl(x / s); with
// STEPS = 1 (x a bf16 number), rs = fl(1 / s) and one correction gives fl(x / s) whenever the quotient is
// above 2^-11 in magnitude, and something that still rounds to the code 0 below (every pair of bf16
// maximum and value evaluated on the CPU, as for the int8 rows).  Other scales take the full divide.
template <int STEPS>
__device__ __forceinline__ float fp8_reciprocal(float s) {
  if constexpr (STEPS == 1) return __fdiv_rn(1.0f, s);
  const float y0 = __builtin_amdgcn_rcpf(s);
  return __builtin_fmaf(__builtin_fmaf(-s, y0, 1.0f), y0, y0);
}
template <int STEPS, int N>
__device__ __forceinline__ void fp8_prescale(float* f, float s, float rs, bool lean_ok) {
  if (__builtin_expect(lean_ok, 1)) {  // one uniform branch around the whole vector
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const float a = f[i];
      float v = a * rs;
      v = __builtin_fmaf(__builtin_fmaf(-s, v, a), rs, v);
      if constexpr (STEPS == 2) v = __builtin_fmaf(__builtin_fmaf(-s, v, a), rs, v);
      // a zero residual added to a quotient of -0 gives +0: the quotient takes the sign of a (s > 0), as the
      // divide's does, so that -0.0 still becomes the code 0x80
      v = __uint_as_float((__float_as_uint(v) & 0x7fffffffu) | (__float_as_uint(a) & 0x80000000u));
      f[i] = fminf(fmaxf(v, -448.0f), 448.0f);
    }
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) f[i] = fminf(fmaxf(__fdiv_rn(f[i], s), -448.0f), 448.0f);
  }
}

template <bool BF16>
__global__ __launch_bounds__(256) void cast_fp8_kernel(const void* __restrict__ x, int64_t nvec,
                                                        const uint32_t* __restrict__ amax_slots,
                                                        uint8_t* __restrict__ q,
                                                        float* __restrict__ scale) {
  constexpr int EPV = RowIn<BF16>::EPV;
  // Pass 2 starts by combining the partial maxima: one slot per thread (1 KiB, served by the L2), a
  // wavefront maximum, and the four wavefront results through LDS.  A maximum has no order: same bits
  // whatever the grouping.
  static_assert(AMAX_SLOTS == 256, "one slot per thread of the 256-thread workgroup");
  __shared__ float part[4];
  {
    const float m = wave_max(__uint_as_float(amax_slots[threadIdx.x]));
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = m;
  }
  __syncthreads();
  const float amax = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
  float s = __fdiv_rn(amax, 448.0f);
  if (amax == 0.0f) s = 1.0f;
  if (blockIdx.x == 0 && threadIdx.x == 0) *scale = s;
  constexpr int STEPS = BF16 ? 1 : 2;
  const float rs = fp8_reciprocal<STEPS>(s);
  const bool lean_ok = s >= 5.421010862427522e-20f && s <= 1.8446744073709552e19f;  // [2^-64, 2^64]
  const uint4* src = reinterpret_cast<const uint4*>(x);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t v0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v0 < nvec; v0 += FP8_BATCH * stride) {
    uint4 t[FP8_BATCH];
#pragma unroll
    for (int u = 0; u < FP8_BATCH; ++u) {
      const int64_t i = v0 + u * stride;
      t[u] = src[i < nvec ? i : nvec - 1];
    }
#pragma unroll
    for (int u = 0; u < FP8_BATCH; ++u) {
      const int64_t v = v0 + u * stride;
      if (v >= nvec) break;
      float f[EPV];
      RowIn<BF16>::unpack(t[u], f);
      fp8_prescale<STEPS, EPV>(f, s, rs, lean_ok);
      // v_cvt_pk_fp8_f32: two fp32 -> two OCP e4m3fn codes, round to nearest even.
      int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false);
      w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w0, true);
      if constexpr (BF16) {
        int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], 0, false);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], w1, true);
        uint2 o;
        o.x = (uint32_t)w0;
        o.y = (uint32_t)w1;
        store_wt(reinterpret_cast<uint2*>(q + v * EPV), o);
      } else {
        store_wt(reinterpret_cast<uint32_t*>(q + v * EPV), (uint32_t)w0);
      }
    }
  }
}

// Both passes in ONE launch for tensors that fit the register files: a workgroup per compute unit keeps its share
// of x in registers (ONEPASS_R 16-byte vectors per thread: 32 MiB over 256 workgroups of 1024 threads), takes the
// maximum of it, exchanges the partial maxima with the other workgroups through `slots`, and casts from the
// registers -- x is read from HBM once instead of twice.  What does not fit the registers is read again in the
// second phase, as the two-launch form does.
//
// The exchange.  slots[b] = (tag << 32) | bits of workgroup b's maximum, one 8-byte device-scope store.  Every
// launch leaves all G slots carrying the same tag, and that is the only state: a workgroup reads the tag T its own
// slot holds, publishes T + 1 with its maximum, and polls until all G slots carry T + 1 (thread t watches slot t).
// The slots must start out equal (zero-filled) and a workspace must always be used with the same G; overlapping
// launches must not share one.  The wait is bounded: workgroups that cannot all be resident at once (another
// kernel holding compute units, a device with fewer than G of them) would otherwise wait for each other forever.
// After spin_limit polls a workgroup stops waiting and takes the maximum of the WHOLE tensor itself -- slow, the
// same bits (a maximum has no order) -- and still publishes its slot, so the state stays consistent.
constexpr int ONEPASS_THREADS = 1024;
constexpr int ONEPASS_R = 8;

template <bool BF16>
__global__ __launch_bounds__(ONEPASS_THREADS) void quant_fp8_onepass_kernel(const void* __restrict__ x, int64_t nvec,
                                                                            unsigned long long* __restrict__ slots,
                                                                            uint8_t* __restrict__ q,
                                                                            float* __restrict__ scale, int spin_limit) {
  constexpr int EPV = RowIn<BF16>::EPV;
  constexpr int NW = ONEPASS_THREADS / 64;
  __shared__ float wmax[NW];
  __shared__ uint32_t tag_lds;
  const int tid = threadIdx.x, G = gridDim.x;
  const uint4* src = reinterpret_cast<const uint4*>(x);
  // vector index of (sweep k, this thread): workgroups interleaved per sweep, 16 KiB contiguous per workgroup
  const int64_t sweep = (int64_t)G * ONEPASS_THREADS;
  const int64_t v0 = (int64_t)blockIdx.x * ONEPASS_THREADS + tid;
  uint4 c[ONEPASS_R];
#pragma unroll
  for (int k = 0; k < ONEPASS_R; ++k) {
    const int64_t i = v0 + k * sweep;
    c[k] = make_uint4(0, 0, 0, 0);
    if (i < nvec) c[k] = src[i];
  }
  // the tag this launch publishes: one more than the one this workgroup's slot carries.  Requested behind the
  // data (loads return in request order; the tag is not needed before the maximum is known)
  asm volatile("" ::: "memory");
  unsigned long long old_slot = 0;
  if (tid == 0) old_slot = __hip_atomic_load(slots + blockIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  asm volatile("" ::: "memory");
  float amax = 0.0f;
#pragma unroll
  for (int k = 0; k < ONEPASS_R; ++k) {
    float f[EPV];
    RowIn<BF16>::unpack(c[k], f);
    amax = fmaxf(amax, vec_amax<EPV>(f));
  }
  for (int64_t i = v0 + ONEPASS_R * sweep; i < nvec; i += sweep) {  // the part that does not fit the registers
    float f[EPV];
    RowIn<BF16>::unpack(src[i], f);
    amax = fmaxf(amax, vec_amax<EPV>(f));
  }
  amax = wave_max(amax);
  if ((tid & 63) == 0) wmax[tid >> 6] = amax;
  if (tid == 0) tag_lds = (uint32_t)(old_slot >> 32) + 1u;
  __syncthreads();
  const uint32_t tag = tag_lds;
  if (tid == 0) {
    float m = 0.0f;
#pragma unroll
    for (int w = 0; w < NW; ++w) m = fmaxf(m, wmax[w]);
    __hip_atomic_store(slots + blockIdx.x, ((unsigned long long)tag << 32) | __float_as_uint(m), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
  }
  // wait for the other workgroups' slots (bounded)
  float seen = 0.0f;
  bool mine = tid >= G;
  int all = 0;
  for (int spin = 0; spin < spin_limit; ++spin) {
    if (!mine) {
      const unsigned long long u = __hip_atomic_load(slots + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if ((uint32_t)(u >> 32) == tag) {
        mine = true;
        seen = __uint_as_float((uint32_t)u);
      }
    }
    all = __syncthreads_and(mine ? 1 : 0);
    if (all) break;
    __builtin_amdgcn_s_sleep(4);
  }
  if (!all) {  // uniform: the others did not show up in time; the whole tensor's maximum, taken here
    seen = 0.0f;
    for (int64_t i = tid; i < nvec; i += ONEPASS_THREADS) {
      float f[EPV];
      RowIn<BF16>::unpack(src[i], f);
      seen = fmaxf(seen, vec_amax<EPV>(f));
    }
  }
  seen = wave_max(seen);
  __syncthreads();  // wmax is reused
  if ((tid & 63) == 0) wmax[tid >> 6] = seen;
  __syncthreads();
  float tmax = 0.0f;
#pragma unroll
  for (int w = 0; w < NW; ++w) tmax = fmaxf(tmax, wmax[w]);
  float s = __fdiv_rn(tmax, 448.0f);
  if (tmax == 0.0f) s = 1.0f;
  if (blockIdx.x == 0 && tid == 0) *scale = s;
  constexpr int STEPS = BF16 ? 1 : 2;
  const float rs = fp8_reciprocal<STEPS>(s);
  const bool lean_ok = s >= 5.421010862427522e-20f && s <= 1.8446744073709552e19f;  // [2^-64, 2^64]
  auto cast_store = [&](const uint4& t, int64_t i) {
    float f[EPV];
    RowIn<BF16>::unpack(t, f);
    fp8_prescale<STEPS, EPV>(f, s, rs, lean_ok);
    int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false);
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w0, true);
    if constexpr (BF16) {
      int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], 0, false);
      w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], w1, true);
      uint2 o;
      o.x = (uint32_t)w0;
      o.y = (uint32_t)w1;
      store_wt(reinterpret_cast<uint2*>(q + i * EPV), o);
    } else {
      store_wt(reinterpret_cast<uint32_t*>(q + i * EPV), (uint32_t)w0);
    }
  };
#pragma unroll
  for (int k = 0; k < ONEPASS_R; ++k) {
    const int64_t i = v0 + k * sweep;
    if (i < nvec) cast_store(c[k], i);
  }
  for (int64_t i = v0 + ONEPASS_R * sweep; i < nvec; i += sweep) cast_store(src[i], i);
}

}  // namespace aq

// ------------------------------------------------------------------- C ABI

extern "C" int aq_quant_rowwise_i8(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                   int8_t* q, float* scale, void* stream) {
  if (x_dtype != AQ_F32 && x_dtype != AQ_BF16) return AQ_E_DTYPE;
  if (M < 0 || K < 0 || (K % 16) != 0 || ldx < K) return AQ_E_SHAPE;
  if (M == 0 || K == 0) {
    // K == 0: amax of an empty row is 0, so every scale is 1; nothing to do for codes.
    if (K == 0 && M > 0) return AQ_E_SHAPE;
    return AQ_OK;
  }
  if (!x || !q || !scale) return AQ_E_NULL;
  if (K > (int64_t)1 << 30 || M > (int64_t)1 << 31) return AQ_E_RANGE;
  const int esz = x_dtype == AQ_BF16 ? 2 : 4;
  if (aq::check_ptr16(x) || aq::check_ptr16(q) || ((ldx * esz) & 15)) return AQ_E_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // Rows that fit 4 cached vectors per lane (2048 bf16 / 1024 fp32) take the
  // double-buffered kernel; with enough rows each wavefront gets two of them so
  // that reads, arithmetic and writes of different rows overlap.
  const int epv = x_dtype == AQ_BF16 ? 8 : 4;
  const int64_t nvec = K / epv;
  // bf16 rows of <= 2048 do as well one wavefront per row once there are enough rows to fill the
  // device; a handful of rows (decode) always gains from the shorter per-lane chain of a workgroup per row
  const int64_t wg_min_vec = (x_dtype == AQ_BF16 && M >= 64) ? 257 : 128;
  if (nvec >= wg_min_vec && nvec <= 1024) {
    // enough rows to fill the device and rows of 128..1024 vectors: one workgroup per row
    const unsigned g = (unsigned)M;
    if (x_dtype == AQ_BF16) {
      if (nvec <= 256)
        hipLaunchKernelGGL((aq::quant_row_wg_kernel<true, 1>), dim3(g), dim3(256), 0, st, x, (int)K, ldx, q, scale);
      else if (nvec <= 512)
        hipLaunchKernelGGL((aq::quant_row_wg_kernel<true, 2>), dim3(g), dim3(256), 0, st, x, (int)K, ldx, q, scale);
      else
        hipLaunchKernelGGL((aq::quant_row_wg_kernel<true, 4>), dim3(g), dim3(256), 0, st, x, (int)K, ldx, q, scale);
    } else {
      if (nvec <= 256)
        hipLaunchKernelGGL((aq::quant_row_wg_kernel<false, 1>), dim3(g), dim3(256), 0, st, x, (int)K, ldx, q, scale);
      else if (nvec <= 512)
        hipLaunchKernelGGL((aq::quant_row_wg_kernel<false, 2>), dim3(g), dim3(256), 0, st, x, (int)K, ldx, q, scale);
      else
        hipLaunchKernelGGL((aq::quant_row_wg_kernel<false, 4>), dim3(g), dim3(256), 0, st, x, (int)K, ldx, q, scale);
    }
    return (int)hipGetLastError();
  }
  const bool small_row = K <= 4 * 64 * epv;
  const bool full_row = K == 4 * 64 * epv;  // every lane holds exactly 4 vectors: no bounds checks
  int64_t wgs = (M + 3) / 4;
  if (small_row && M >= 2048) wgs = (wgs + 1) / 2;
  const unsigned grid = (unsigned)wgs;
  if (x_dtype == AQ_BF16) {
    if (full_row)
      hipLaunchKernelGGL((aq::quant_rowwise_i8_kernel<true, 4, true, true>), dim3(grid), dim3(256), 0, st, x, M,
                         (int)K, ldx, q, scale);
    else if (small_row)
      hipLaunchKernelGGL((aq::quant_rowwise_i8_kernel<true, 4, true, false>), dim3(grid), dim3(256), 0, st, x, M,
                         (int)K, ldx, q, scale);
    else
      hipLaunchKernelGGL((aq::quant_rowwise_i8_kernel<true, 16, false, false>), dim3(grid), dim3(256), 0, st, x,
                         M, (int)K, ldx, q, scale);
  } else {
    if (full_row)
      hipLaunchKernelGGL((aq::quant_rowwise_i8_kernel<false, 4, true, true>), dim3(grid), dim3(256), 0, st, x, M,
                         (int)K, ldx, q, scale);
    else if (small_row)
      hipLaunchKernelGGL((aq::quant_rowwise_i8_kernel<false, 4, true, false>), dim3(grid), dim3(256), 0, st, x, M,
                         (int)K, ldx, q, scale);
    else
      hipLaunchKernelGGL((aq::quant_rowwise_i8_kernel<false, 16, false, false>), dim3(grid), dim3(256), 0, st, x,
                         M, (int)K, ldx, q, scale);
  }
  return (int)hipGetLastError();
}

template <bool BF16>
static int launch_rmsnorm_quant(const void* x, const void* gamma, float eps, int64_t M, int64_t K, int64_t ldx,
                                int8_t* q, float* scale, hipStream_t st) {
  const int64_t vpl = (K / (BF16 ? 8 : 4) + 63) / 64;  // vectors per lane
  int64_t wgs = (M + 3) / 4;
  if (wgs > 1024) wgs = 1024;  // four workgroups per CU; wavefronts walk the remaining rows
  const dim3 g((unsigned)wgs), b(256);
  if (vpl <= 4)
    hipLaunchKernelGGL((aq::rmsnorm_quant_kernel<BF16, 4, true>), g, b, 0, st, x, gamma, eps, M, (int)K, ldx, q, scale);
  else if (vpl <= 12)
    hipLaunchKernelGGL((aq::rmsnorm_quant_kernel<BF16, 12, false>), g, b, 0, st, x, gamma, eps, M, (int)K, ldx, q, scale);
  else if (vpl <= 24)  // 24 vectors per lane is what fits the register file without spilling for bf16 rows
    hipLaunchKernelGGL((aq::rmsnorm_quant_kernel<BF16, 24, false>), g, b, 0, st, x, gamma, eps, M, (int)K, ldx, q, scale);
  else
    return AQ_E_RANGE;
  return (int)hipGetLastError();
}

extern "C" int aq_rmsnorm_quant_rowwise_i8(const void* x, int x_dtype, const void* gamma, int gamma_dtype, float eps,
                                           int64_t M, int64_t K, int64_t ldx, int8_t* q, float* scale,
                                           void* stream) {
  if (x_dtype != AQ_F32 && x_dtype != AQ_BF16) return AQ_E_DTYPE;
  if (gamma_dtype != x_dtype) return AQ_E_DTYPE;  // the norm's gain lives in the activations' dtype
  if (M < 0 || K <= 0 || (K % 16) != 0 || ldx < K || !(eps >= 0.0f)) return AQ_E_SHAPE;
  if (M == 0) return AQ_OK;
  if (!x || !gamma || !q || !scale) return AQ_E_NULL;
  const int esz = x_dtype == AQ_BF16 ? 2 : 4;
  if (aq::check_ptr16(x) || aq::check_ptr16(gamma) || aq::check_ptr16(q) || ((ldx * esz) & 15)) return AQ_E_ALIGN;
  if (M > (int64_t)1 << 31) return AQ_E_RANGE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  return x_dtype == AQ_BF16 ? launch_rmsnorm_quant<true>(x, gamma, eps, M, K, ldx, q, scale, st)
                            : launch_rmsnorm_quant<false>(x, gamma, eps, M, K, ldx, q, scale, st);
}

#ifndef AQ_SWIGLU_WG_MAX_M
#define AQ_SWIGLU_WG_MAX_M 1024
#endif
template <bool BF16>
static int launch_swiglu_quant(const void* ug, int64_t M, int64_t F, int64_t ld, int8_t* q, float* scale,
                               hipStream_t st) {
  const int64_t vpl = (F / (BF16 ? 8 : 4) + 63) / 64;  // vector pairs per lane
  if (vpl > 16) return AQ_E_RANGE;
  // few rows, or rows too long for one wavefront's registers: a workgroup of vpl wavefronts per row
  if (vpl > 1 && (M <= AQ_SWIGLU_WG_MAX_M || vpl > 12)) {
    hipLaunchKernelGGL((aq::swiglu_quant_wg_kernel<BF16>), dim3((unsigned)M), dim3((unsigned)vpl * 64), 0, st, ug, (int)F,
                       ld, q, scale);
    return (int)hipGetLastError();
  }
  // four wavefronts of this kernel fit a SIMD (128 registers each): 16 rows at a time per compute unit, and
  // wavefronts walk the rows beyond that
  int64_t wgs = (M + 3) / 4;
  const int64_t cap = (int64_t)aq::device_cus() * 4;
  if (wgs > cap) wgs = cap;
  const dim3 g((unsigned)wgs), b(256);
  // as many vector pairs per lane as the row has (a slot past the row costs its full arithmetic: a 5632-wide row
  // is 11 pairs per lane, and a 12th would be 8 % more work)
  switch (vpl) {
#define AQ_SWIGLU_CASE(nc)                                                                                   \
  case nc: hipLaunchKernelGGL((aq::swiglu_quant_kernel<BF16, nc>), g, b, 0, st, ug, M, (int)F, ld, q, scale); break;
    AQ_SWIGLU_CASE(1) AQ_SWIGLU_CASE(2) AQ_SWIGLU_CASE(3) AQ_SWIGLU_CASE(4) AQ_SWIGLU_CASE(5) AQ_SWIGLU_CASE(6)
    AQ_SWIGLU_CASE(7) AQ_SWIGLU_CASE(8) AQ_SWIGLU_CASE(9) AQ_SWIGLU_CASE(10) AQ_SWIGLU_CASE(11) AQ_SWIGLU_CASE(12)
#undef AQ_SWIGLU_CASE
    default: return AQ_E_RANGE;
  }
  return (int)hipGetLastError();
}

extern "C" int aq_swiglu_quant_rowwise_i8(const void* ug, int dtype, int64_t M, int64_t F, int64_t ld, int8_t* q,
                                          float* scale, void* stream) {
  if (dtype != AQ_F32 && dtype != AQ_BF16) return AQ_E_DTYPE;
  if (M < 0 || F <= 0 || (F % 16) != 0 || ld < 2 * F) return AQ_E_SHAPE;
  if (M == 0) return AQ_OK;
  if (!ug || !q || !scale) return AQ_E_NULL;
  const int esz = dtype == AQ_BF16 ? 2 : 4;
  if (aq::check_ptr16(ug) || aq::check_ptr16(q) || ((ld * esz) & 15)) return AQ_E_ALIGN;
  if (M > (int64_t)1 << 31) return AQ_E_RANGE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  return dtype == AQ_BF16 ? launch_swiglu_quant<true>(ug, M, F, ld, q, scale, st)
                          : launch_swiglu_quant<false>(ug, M, F, ld, q, scale, st);
}

// (not static: the lab library's hook in lab.hip calls it with its own bound on the wait)
namespace aq {
int quant_tensor_fp8_onepass(const void* x, int x_dtype, int64_t numel, uint8_t* q, float* scale, void* ws,
                             size_t ws_bytes, int spin_limit, hipStream_t st) {
  if (x_dtype != AQ_F32 && x_dtype != AQ_BF16) return AQ_E_DTYPE;
  if (numel < 0 || (numel % 16) != 0) return AQ_E_SHAPE;
  if (!scale || !ws) return AQ_E_NULL;
  if (numel > 0 && (!x || !q)) return AQ_E_NULL;
  if (ws_bytes < AQ_FP8_ONEPASS_WS_BYTES) return AQ_E_WORKSPACE;
  if (aq::check_ptr16(x) || aq::check_ptr16(q) || aq::check_ptr(ws, 8) || aq::check_ptr(scale, 4)) return AQ_E_ALIGN;
  const int epv = x_dtype == AQ_BF16 ? 8 : 4;
  const int64_t nvec = numel / epv;
  // one workgroup per compute unit, at most one per slot; always the same count on a device, whatever the size
  int g = aq::device_cus();
  if (g > AQ_FP8_ONEPASS_WS_BYTES / 8) g = AQ_FP8_ONEPASS_WS_BYTES / 8;
  if (x_dtype == AQ_BF16)
    hipLaunchKernelGGL((aq::quant_fp8_onepass_kernel<true>), dim3((unsigned)g), dim3(aq::ONEPASS_THREADS), 0, st, x, nvec,
                       static_cast<unsigned long long*>(ws), q, scale, spin_limit);
  else
    hipLaunchKernelGGL((aq::quant_fp8_onepass_kernel<false>), dim3((unsigned)g), dim3(aq::ONEPASS_THREADS), 0, st, x, nvec,
                       static_cast<unsigned long long*>(ws), q, scale, spin_limit);
  return (int)hipGetLastError();
}
}  // namespace aq

extern "C" int aq_quant_tensor_fp8_onepass(const void* x, int x_dtype, int64_t numel, uint8_t* q, float* scale,
                                           void* ws, size_t ws_bytes, void* stream) {
  // 4096 polls of a few hundred nanoseconds each: a millisecond or two before a workgroup stops waiting
  return aq::quant_tensor_fp8_onepass(x, x_dtype, numel, q, scale, ws, ws_bytes, 4096, static_cast<hipStream_t>(stream));
}

extern "C" int aq_quant_tensor_fp8(const void* x, int x_dtype, int64_t numel, uint8_t* q,
                                   float* scale, uint32_t* amax_ws, size_t ws_bytes, void* stream) {
  if (x_dtype != AQ_F32 && x_dtype != AQ_BF16) return AQ_E_DTYPE;
  if (numel < 0 || (numel % 16) != 0) return AQ_E_SHAPE;
  if (!scale || !amax_ws) return AQ_E_NULL;
  if (ws_bytes < AQ_FP8_AMAX_WS_BYTES) return AQ_E_WORKSPACE;  // every call writes all of its partial-maximum slots
  if (numel > 0 && (!x || !q)) return AQ_E_NULL;
  if (aq::check_ptr16(x) || aq::check_ptr16(q) || aq::check_ptr(amax_ws, 4) || aq::check_ptr(scale, 4)) return AQ_E_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int epv = x_dtype == AQ_BF16 ? 8 : 4;
  const int64_t nvec = numel / epv;
  int64_t blocks = (nvec + 255) / 256;
  if (blocks > 2048) blocks = 2048;  // 8 workgroups per CU, grid-stride beyond
  if (blocks < 1) blocks = 1;
  int64_t ablocks = (nvec + aq::AMAX_THREADS * aq::FP8_BATCH - 1) / (aq::AMAX_THREADS * aq::FP8_BATCH);
  // every slot is written each call: the grid is always AMAX_SLOTS workgroups (about one per compute unit;
  // those past the data leave 0, which cannot change a maximum of magnitudes)
  (void)ablocks;
  ablocks = aq::AMAX_SLOTS;
  if (x_dtype == AQ_BF16) {
    hipLaunchKernelGGL((aq::amax_kernel<true>), dim3((unsigned)ablocks), dim3(aq::AMAX_THREADS), 0, st, x, nvec, amax_ws);
    hipLaunchKernelGGL((aq::cast_fp8_kernel<true>), dim3((unsigned)blocks), dim3(256), 0, st, x, nvec,
                       amax_ws, q, scale);
  } else {
    hipLaunchKernelGGL((aq::amax_kernel<false>), dim3((unsigned)ablocks), dim3(aq::AMAX_THREADS), 0, st, x, nvec, amax_ws);
    hipLaunchKernelGGL((aq::cast_fp8_kernel<false>), dim3((unsigned)blocks), dim3(256), 0, st, x, nvec,
                       amax_ws, q, scale);
  }
  return (int)hipGetLastError();
}

