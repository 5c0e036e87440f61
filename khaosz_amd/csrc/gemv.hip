// Decode path (M <= 16 tokens): a weight-streaming int8 GEMV.  The weight
// matrix is read exactly once with 16-byte loads, one wavefront reading 1 KiB
// contiguous of a row per instruction; the few activation rows are quantised
// by the row-wise kernel into the caller's workspace, pulled into LDS once per
// workgroup by direct global->LDS loads and reused by every row of W.
// Products are v_dot4_i32_i8 (no MFMA tiles, no LDS staging of W); a wavefront
// reduces its 4 x MT partial sums with a transposed butterfly so that each
// lane ends up owning one output, then applies the same dequantising epilogue
// as the MFMA GEMM.  The int32 sums are exact, so the result is bit-identical
// to quantise + GEMM.
//
// Every byte the kernel will need is requested before anything is waited for:
// a wavefront first issues its share of the activation copy, then the weight
// loads of its first two K chunks, and only then waits for the activations.
#include <type_traits>

#include "aq_common.h"
#include "aq_rows.h"

namespace aq {

#ifndef AQ_GV_ROWS
#define AQ_GV_ROWS 4
#endif
#ifndef AQ_GV_WAVES
#define AQ_GV_WAVES 8
#endif
constexpr int GV_ROWS = AQ_GV_ROWS;    // weight rows per wavefront pass
constexpr int GV_WAVES = AQ_GV_WAVES;  // wavefronts per workgroup
constexpr int GV_THREADS = GV_WAVES * 64;
constexpr int GV_CHUNK = 64 * 16;  // K bytes one wavefront covers per load
constexpr int GV_DEPTH = 2;        // weight chunks in flight per wavefront

typedef __attribute__((address_space(3))) void gv_lds_void;
typedef unsigned gv_u2 __attribute__((ext_vector_type(2)));

// Reduce V values per lane across the 64 lanes so that afterwards v[0] of lane
// l holds the full sum of value index l >> (6 - log2 V) (for V <= 64).
// Lane-bit 5 and 4 stages use the gfx950 half/row swaps: one swap exchanges the
// two halves a pair of values needs, one add finishes it.  The remaining
// stages (at most 15 live values for V = 64) use cross-lane shuffles.
template <int CUR, int OFF>
struct Butterfly {
  template <int V>
  __device__ static __forceinline__ void run(int (&v)[V], int lane) {
    if constexpr (CUR > 1) {
      constexpr int H = CUR / 2;
      if constexpr (OFF == 32 || OFF == 16) {
#pragma unroll
        for (int i = 0; i < H; ++i) {
          const gv_u2 r = OFF == 32 ? __builtin_amdgcn_permlane32_swap((unsigned)v[i], (unsigned)v[i + H], false, false)
                                    : __builtin_amdgcn_permlane16_swap((unsigned)v[i], (unsigned)v[i + H], false, false);
          v[i] = (int)(r.x + r.y);
        }
      } else {
        const bool up = (lane & OFF) != 0;
#pragma unroll
        for (int i = 0; i < H; ++i) {
          const int lo = v[i], hi = v[i + H];
          const int send = up ? lo : hi;
          const int keep = up ? hi : lo;
          v[i] = keep + __shfl_xor(send, OFF, AQ_WAVE);
        }
      }
      if constexpr (OFF > 1) Butterfly<H, OFF / 2>::run(v, lane);
    } else {
      v[0] += __shfl_xor(v[0], OFF, AQ_WAVE);
      if constexpr (OFF > 1) Butterfly<1, OFF / 2>::run(v, lane);
    }
  }
};

constexpr int ilog2(int v) { return v <= 1 ? 0 : 1 + ilog2(v / 2); }

struct GemvArgs {
  const void* x;      // [M, K] bf16 activations (fused-quantise kernels), row stride K
  const int8_t* xq;   // [M, K] codes (kernels that take codes)
  const float* sx;    // [M]
  const int8_t* wq;   // [N, K]
  const float* sw;    // [N]
  const void* bias;   // [N] or null
  const void* res;    // [M, N] residual in y's dtype (row stride ldr), or null; may be y itself
  void* y;            // [M, N]
  int64_t ldr;
  int M, N, K;
  int bias_dtype, y_dtype;
  int ksplit, groups;  // matrix-core variant: wavefronts sharing a row group, row groups per workgroup
  const void* gamma;   // NORM kernels: RMSNorm gain [K] in x's dtype
  float eps;
  const float* parts;  // MERGE kernels: attention partial results in place of x
  int parts_ns, parts_d;
};

// y (+ residual): the projection is rounded to the output type first and the
// sum rounded again, the bits a separate elementwise add of the two tensors gives.
__device__ __forceinline__ float add_residual_bf16(float y, uint32_t res_bits) {
  return __fadd_rn(bf16_bits_to_f32((uint16_t)f32_to_bf16_bits(y)), bf16_bits_to_f32((uint16_t)res_bits));
}

// Epilogue operands (activation scale, weight scale, bias, residual) are requested at the very start of a
// kernel through buffer descriptors, without a branch: a descriptor of size 0 (no bias, no residual, a
// wavefront or lane that stores nothing) makes the load return 0 without touching memory.  Written as
// `if (bias) load`, the compiler waited for the loads at every join of those branches -- a full memory
// round trip in front of the weight stream whenever a bf16 bias was given.
struct EpiOperands {
  __amdgpu_buffer_rsrc_t sx, sw, bias_f32, bias_bf16, res_f32, res_bf16;
  __device__ __forceinline__ EpiOperands(const GemvArgs& p, bool live, bool want_sx, bool want_res) {
    const bool has_bias = p.bias != nullptr;
    const bool bias_is_bf16 = p.bias_dtype == AQ_BF16, res_is_bf16 = p.y_dtype == AQ_BF16;
    const uint32_t n = (uint32_t)p.N;
    sx = make_rsrc(want_sx ? (const void*)p.sx : (const void*)p.sw, live && want_sx ? (uint32_t)p.M * 4u : 0u);
    sw = make_rsrc(p.sw, live ? n * 4u : 0u);
    bias_f32 = make_rsrc(has_bias ? p.bias : (const void*)p.sw, live && has_bias && !bias_is_bf16 ? n * 4u : 0u);
    bias_bf16 = make_rsrc(has_bias ? p.bias : (const void*)p.sw, live && has_bias && bias_is_bf16 ? n * 2u : 0u);
    const bool has_res = want_res && p.res != nullptr;
    const uint32_t res_elems = (uint32_t)p.M * (uint32_t)p.ldr;
    res_f32 = make_rsrc(has_res ? p.res : (const void*)p.sw, live && has_res && !res_is_bf16 ? res_elems * 4u : 0u);
    res_bf16 = make_rsrc(has_res ? p.res : (const void*)p.sw, live && has_res && res_is_bf16 ? res_elems * 2u : 0u);
  }
  __device__ __forceinline__ float load_sx(int m, bool ok) const {
    return __uint_as_float((uint32_t)__builtin_amdgcn_raw_buffer_load_b32(sx, ok ? m * 4 : (int)OOB_OFFSET, 0, 0));
  }
  __device__ __forceinline__ float load_sw(int n, bool ok) const {
    return __uint_as_float((uint32_t)__builtin_amdgcn_raw_buffer_load_b32(sw, ok ? n * 4 : (int)OOB_OFFSET, 0, 0));
  }
  // Both element sizes are requested; only the descriptor of the operand's own type has a size, the other
  // load returns 0, and the two results are OR-ed: no select on the type (which the compiler turns back
  // into a branch around each load, with a wait at its join).
  __device__ __forceinline__ float load_bias(int n, bool ok) const {
    const uint32_t f = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(bias_f32, ok ? n * 4 : (int)OOB_OFFSET, 0, 0);
    const uint32_t h = (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(bias_bf16, ok ? n * 2 : (int)OOB_OFFSET, 0, 0);
    return __uint_as_float(f | (h << 16));
  }
  __device__ __forceinline__ uint32_t load_res(int m, int n, bool ok, int ldr) const {  // raw bits of one element
    const int e = m * ldr + n;
    const uint32_t f = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(res_f32, ok ? e * 4 : (int)OOB_OFFSET, 0, 0);
    const uint32_t h = (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(res_bf16, ok ? e * 2 : (int)OOB_OFFSET, 0, 0);
    return f | (h & 0xffffu);
  }
};

// Weight loads are marked as streaming (nt): every byte is read exactly once per launch.  Measured 0.05 - 0.35 us
// per launch against plain loads (M = 1: 5.50 -> 5.15 us; a one-shot 16 MiB read: 4.4 -> 4.0 us).
#define GV_WLOAD buffer_load_16_stream
#define GV_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0f70 | ((n) & 15) | (((n) >> 4) << 14))

// FUSED: the kernel quantises the bf16 activation rows itself (VPL 16-byte vectors
// per lane per row) instead of copying codes a separate launch produced.
// Wavefronts per workgroup: GV_WAVES for the fused kernels (they split the row
// quantisation among them: with fewer, each would round several rows one after
// the other before any product can start), taken from the launch otherwise.  A
// workgroup covers GV_ROWS * wavefronts weight rows; the launcher shrinks it
// when N is too small for 8-wavefront workgroups to reach every compute unit.
// NORM (with FUSED): the rows are RMS-normalised with the gain p.gamma before they are quantised.
// MERGE > 0 (with FUSED): the rows are a decode step's attention output, combined here from the attention
// kernel's partial results of up to MERGE slices (p.parts) -- the separate merge launch disappears.
// FW: wavefronts per workgroup of a FUSED kernel (8, or 4 for short matrices).
// FK: K parts of a FUSED kernel (1; 4 for a short matrix with long rows, an MLP's down projection: every wavefront
// still rounds a row, then FK wavefronts share a group of weight rows, so that the launch has a workgroup for
// every compute unit where whole rows per wavefront would leave most of them without loads in flight).
template <int MT, bool FUSED, int VPL, bool NORM = false, int MERGE = 0, int FW = GV_WAVES, int FK = 1>
__global__ __launch_bounds__(GV_THREADS) void gemv_w8a8_kernel(GemvArgs p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t xs[];  // [MT][K] activation codes, then [MT] scales
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int K = p.K, N = p.N, M = p.M;
  // wavefront-uniform first row, kept scalar so the buffer descriptor lives in SGPRs
  constexpr int WAVES = FUSED ? FW : GV_WAVES;
  const int nwaves = FUSED ? WAVES : (int)(blockDim.x >> 6);
  // K parts: ksplit wavefronts share a group of GV_ROWS rows, wavefront kpart taking chunks kpart,
  // kpart + ksplit, ...; their sums meet in LDS (exact int32).  For short N and long K, where whole rows per
  // wavefront would leave most of the device without loads in flight.
  const int ksplit = FUSED ? FK : p.ksplit;
  const int kpart = wave % ksplit;
  const int n0 = __builtin_amdgcn_readfirstlane((blockIdx.x * (nwaves / ksplit) + wave / ksplit) * GV_ROWS);

  // 0. After the reduction lane l owns output (row n0 + idx / MT, token idx % MT)
  // with idx = l >> (6 - log2(rows * MT)).  Its scales and bias are requested
  // ahead of the weight stream, so the epilogue never waits on memory, but behind
  // the activation rows (step 1): loads return in request order, and these lines,
  // which no other workgroup shares, come from HBM while the rows come from cache.
  constexpr int V = GV_ROWS * MT;
  constexpr int SH = 6 - ilog2(V);
  static_assert(V <= 64, "one output per lane at most");
  const int oidx = lane >> SH;
  const int om = oidx % MT, on = n0 + oidx / MT;
  const bool out_lane = (lane & ((1 << SH) - 1)) == 0 && om < M && on < N;
  float* sx_lds = reinterpret_cast<float*>(xs + MT * K);
  const EpiOperands epi(p, true, !FUSED, true);
  float sxv = 0.0f, swv, bv;
  uint32_t rv;  // residual element, raw bits
  auto load_epi = [&]() {
    sxv = epi.load_sx(om, out_lane);
    swv = epi.load_sw(on, out_lane);
    bv = epi.load_bias(on, out_lane);
    rv = epi.load_res(om, on, out_lane, (int)p.ldr);
  };
  // (the copy of ready-made codes goes straight to LDS and is waited for by counting the requests behind it:
  // there the operands stay in front)
  if constexpr (!FUSED) load_epi();

  // 1. activation codes -> LDS.  Either copied, 16 bytes per lane, straight from
  // global memory (rows m >= M lie outside the descriptor and arrive as zeros),
  // or produced here: each wavefront requests its rows of the bf16 activation now
  // and quantises them while the weight loads queued behind are in flight.
  constexpr int RPW = FUSED ? (MT + WAVES - 1) / WAVES : 1;
  RowsToLds<true, RPW, VPL> xrows;
  AttnRows<RPW, VPL, MERGE> arows;
  if constexpr (MERGE > 0) {
    arows.issue(p.parts, M, K, p.parts_d, p.parts_ns, wave, WAVES, lane);
  } else if constexpr (FUSED) {
    xrows.issue(p.x, M, K, K, wave, WAVES, lane);
    if constexpr (NORM) xrows.issue_gamma(p.gamma, K, lane);
  } else {
    const __amdgpu_buffer_rsrc_t Xr = make_rsrc(p.xq, (uint32_t)M * (uint32_t)K);
    const int xbytes = MT * K;
    const int xrounds = (xbytes + nwaves * 1024 - 1) / (nwaves * 1024);
    for (int r = 0; r < xrounds; ++r) {
      const int base = (r * nwaves + wave) * 1024;  // this wavefront's 1 KiB of the copy
      if (base < xbytes)  // uniform; xbytes is a multiple of 16 but not always of 1024:
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            Xr, (gv_lds_void*)(xs + base), 16,
            (base + lane * 16) < xbytes ? (uint32_t)(base + lane * 16) : OOB_OFFSET, 0, 0, 0);
    }
  }

  asm volatile("" ::: "memory");  // request order: activation rows, epilogue operands, the weight stream
  if constexpr (FUSED) load_epi();
  asm volatile("" ::: "memory");

  // 2. the first GV_DEPTH weight chunks of this wavefront's rows.  The
  // descriptor spans these rows only; rows past N and bytes past K fall
  // outside it and read as zero.
  const int nchunk_all = (K + GV_CHUNK - 1) / GV_CHUNK;
  const int nchunk = (nchunk_all - kpart + ksplit - 1) / ksplit;  // this wavefront's chunks (0 is possible)
  const int rows = n0 < N ? ((N - n0) < GV_ROWS ? (N - n0) : GV_ROWS) : 0;
  const __amdgpu_buffer_rsrc_t Wr =
      make_rsrc(p.wq + (int64_t)(n0 < N ? n0 : 0) * K, (uint32_t)rows * (uint32_t)K);
  auto wload = [&](int c, uint4 (&dst)[GV_ROWS]) {
    const int kb = (kpart + c * ksplit) * GV_CHUNK + lane * 16;
    const bool ok = kb < K;  // past K the offset would alias the next row
#pragma unroll
    for (int r = 0; r < GV_ROWS; ++r)
      dst[r] = GV_WLOAD(Wr, ok ? (uint32_t)r * (uint32_t)K + (uint32_t)kb : OOB_OFFSET);
  };
  uint4 w[GV_DEPTH][GV_ROWS];
#pragma unroll
  for (int d = 0; d < GV_DEPTH; ++d) wload(d, w[d]);  // chunks past the end read zeros

  // 3. the activation requests are older than the weight loads: wait until at
  // most those are outstanding (the fused path's own use of the rows makes the
  // compiler place that wait), then make every wavefront's part visible through
  // a barrier that does not drain the weight loads.
  if constexpr (FUSED) {
    if constexpr (MERGE > 0) arows.merge(xrows.c, M, K, p.parts_ns, wave, WAVES, lane);
    xrows.template finish<NORM>(M, MT, K, xs, K, sx_lds, wave, WAVES, lane, p.eps);
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wavefront's LDS writes are done
  } else {
    GV_WAIT_VMCNT(GV_DEPTH * GV_ROWS);
  }
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  if constexpr (FUSED) {
    if (out_lane) sxv = sx_lds[om];
  }

  int acc[GV_ROWS * MT];
#pragma unroll
  for (int i = 0; i < GV_ROWS * MT; ++i) acc[i] = 0;

  auto consume = [&](int c, const uint4 (&wc)[GV_ROWS]) {
    const int kb = (kpart + c * ksplit) * GV_CHUNK + lane * 16;
    const int kx = kb < K ? kb : 0;  // lanes past the end multiply zeros; keep the LDS read in range
    // activation rows in blocks of 4: four LDS reads in flight cover the 64 dot
    // products of the previous block without holding all MT rows in registers
    constexpr int MB = MT < 4 ? MT : 4;
#pragma unroll
    for (int m0 = 0; m0 < MT; m0 += MB) {
      uint4 x[MB];
#pragma unroll
      for (int i = 0; i < MB; ++i) x[i] = *reinterpret_cast<const uint4*>(xs + (m0 + i) * K + kx);
#pragma unroll
      for (int i = 0; i < MB; ++i) {
#pragma unroll
        for (int r = 0; r < GV_ROWS; ++r) {
          int a = acc[r * MT + m0 + i];
          a = __builtin_amdgcn_sdot4((int)wc[r].x, (int)x[i].x, a, false);
          a = __builtin_amdgcn_sdot4((int)wc[r].y, (int)x[i].y, a, false);
          a = __builtin_amdgcn_sdot4((int)wc[r].z, (int)x[i].z, a, false);
          a = __builtin_amdgcn_sdot4((int)wc[r].w, (int)x[i].w, a, false);
          acc[r * MT + m0 + i] = a;
        }
      }
      if constexpr (MT > 8) __builtin_amdgcn_sched_barrier(0);
    }
  };
  // K loop.  Rows of up to 2 KiB (the common decode shapes) are two chunks that
  // are already in flight: no loop.  Longer rows rotate two register buffers.
  static_assert(GV_DEPTH == 2, "the K loop below rotates exactly two buffers");
  consume(0, w[0]);
  if (nchunk > 2) wload(2, w[0]);
  __builtin_amdgcn_sched_barrier(0);
  if (nchunk > 1) consume(1, w[1]);
  for (int c = 2; c < nchunk; c += 2) {
    if (c + 1 < nchunk) wload(c + 1, w[1]);
    __builtin_amdgcn_sched_barrier(0);
    consume(c, w[0]);
    if (c + 2 < nchunk) wload(c + 2, w[0]);
    __builtin_amdgcn_sched_barrier(0);
    if (c + 1 < nchunk) consume(c + 1, w[1]);
  }

  Butterfly<V, 32>::run(acc, lane);
  if (ksplit > 1) {  // uniform over the workgroup
    int* part = reinterpret_cast<int*>(sx_lds + MT);  // [wavefront][lane]
    if (kpart != 0) part[wave * 64 + lane] = acc[0];
    __syncthreads();
    if (kpart != 0) return;
    for (int k = 1; k < ksplit; ++k) acc[0] += part[(wave + k) * 64 + lane];
  }
  if (!out_lane) return;
  float y = __fmul_rn(__fmul_rn((float)acc[0], sxv), swv);
  if (p.bias) y = __fadd_rn(y, bv);
  if (p.res) y = p.y_dtype == AQ_BF16 ? add_residual_bf16(y, rv) : __fadd_rn(y, __uint_as_float(rv));
  const int64_t o = (int64_t)om * N + on;
  if (p.y_dtype == AQ_BF16)
    reinterpret_cast<uint16_t*>(p.y)[o] = (uint16_t)f32_to_bf16_bits(y);
  else
    reinterpret_cast<float*>(p.y)[o] = y;
}

// Shape of a launch for N weight rows of K bytes.  Whole rows per wavefront, 8 wavefronts per workgroup,
// halved (down to 2) while the launch would have fewer workgroups than the device has compute units.  Rows
// of four or more chunks on a launch that still has fewer than 1024 wavefronts are cut into 2 or 4 K parts
// (more loads in flight; a wavefront keeps at least one chunk).
struct GemvShape {
  int waves, ksplit;
};

// A kernel whose dynamic LDS may exceed 64 KiB is opted in to the whole 160 KiB of a compute unit the first
// time a launch on a device needs it (one attribute call per kernel and device instead of one per launch).
// Two threads racing here both make the idempotent call.
struct LdsOptIn {
  bool done[64] = {};
  int ensure(const void* fn) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
    if (dev >= 0 && done[dev]) return 0;
    const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return (int)e;
    if (dev >= 0) done[dev] = true;
    return 0;
  }
};
static GemvShape gemv_shape(int N, int K, bool fused, int mt) {
  GemvShape sh{GV_WAVES, 1};
  if (fused) return sh;
  const int cus = device_cus();
  const int groups = (N + GV_ROWS - 1) / GV_ROWS, nchunk = (K + GV_CHUNK - 1) / GV_CHUNK;
  // K parts until the device holds 4 wavefronts per compute unit -- 8 for up to 4 tokens, where the extra loads in
  // flight pay (N = K = 4096, 1 token: 6.25 -> 5.5 us) and the token codes every workgroup copies are few; with 8
  // tokens the same change costs 0.4 us
  const int waves_per_cu = mt <= 4 ? 8 : 4;
  while (nchunk >= 4 && sh.ksplit < 4 && groups * sh.ksplit < waves_per_cu * cus && nchunk >= 2 * sh.ksplit) sh.ksplit *= 2;
  int per_wg = GV_WAVES / sh.ksplit;  // row groups per workgroup
  while (per_wg > 1 && (groups + per_wg - 1) / per_wg < cus) per_wg >>= 1;
  if (sh.ksplit == 1 && per_wg < 2) per_wg = 2;
  sh.waves = per_wg * sh.ksplit;
  return sh;
}

template <int MT, bool FUSED, int VPL, bool NORM, int MERGE, int FW, int FK = 1>
static int launch_gemv_fw(GemvArgs a, hipStream_t st) {
  GemvShape sh = gemv_shape(a.N, a.K, FUSED, MT);
  if (FUSED) {
    sh.waves = FW;
    sh.ksplit = FK;
  }
  a.ksplit = sh.ksplit;
  const int rows_per_wg = GV_ROWS * (sh.waves / sh.ksplit);
  const unsigned grid = (unsigned)((a.N + rows_per_wg - 1) / rows_per_wg);
  const size_t lds = (size_t)MT * a.K + MT * sizeof(float) + (sh.ksplit > 1 ? (size_t)sh.waves * 64 * sizeof(int) : 0);
  if (lds > 64 * 1024) {  // beyond the default dynamic-LDS limit: opt this kernel in, once per device
    static LdsOptIn opted;
    const int e = opted.ensure(reinterpret_cast<const void*>(&gemv_w8a8_kernel<MT, FUSED, VPL, NORM, MERGE, FW, FK>));
    if (e) return e;
  }
  hipLaunchKernelGGL((gemv_w8a8_kernel<MT, FUSED, VPL, NORM, MERGE, FW, FK>), dim3(grid), dim3(sh.waves * 64), lds, st, a);
  return (int)hipGetLastError();
}

// Fused kernels on a short matrix (N / 32 workgroups would leave most compute units without one) run with 4
// wavefronts per workgroup instead of 8: twice the workgroups, each quantising the rows again but reaching a
// compute unit of its own (q/k/v 3072 x 2048 at M = 8: 5.6 -> 5.2 us; 1536 x 1536 at M = 4: 3.8 -> 3.5 us).
// Only where a wavefront still holds at most one row of the in-kernel merge and the rows are short.
template <int MT, bool FUSED, int VPL, bool NORM = false, int MERGE = 0>
static int launch_gemv(GemvArgs a, hipStream_t st) {
  if constexpr (FUSED && VPL <= 4 && (MERGE == 0 || MT <= 4)) {
    if (a.N <= 4096) return launch_gemv_fw<MT, FUSED, VPL, NORM, MERGE, 4>(a, st);
  }
  return launch_gemv_fw<MT, FUSED, VPL, NORM, MERGE, GV_WAVES>(a, st);
}

constexpr int64_t GV_MAX_LDS = 160 * 1024;  // LDS of one gfx950 CU
#ifndef AQ_GV_MFMA_MIN_M
#define AQ_GV_MFMA_MIN_M 8
#endif
constexpr int GV_MFMA_MIN_M = AQ_GV_MFMA_MIN_M;  // more tokens than this take the matrix-core variant

// ---------------------------------------------------------------------------
// Streaming variant for 5..16 tokens.  With that many tokens the 16 dot
// products every weight dword needs make the vector ALU, not HBM, the limit
// of the kernel above.  This one keeps its structure -- every weight byte goes
// HBM -> registers exactly once, no LDS staging or macro-tiling of W -- but
// hands the products to the matrix core: a wavefront owns 16 weight rows, loads
// them 16 bytes per lane directly in the v_mfma_i32_16x16x64_i8 operand order
// (lane l: row l%16, K bytes 64j + 16*(l/16) .. +16 of step j, so the four
// lanes of a row cover 64 contiguous bytes and two consecutive steps consume
// whole 128-byte lines), and multiplies against the token codes held in LDS.
// The 16 x 16 result has rows = weight rows and columns = tokens, so a lane
// ends up with 4 consecutive outputs of one token: no cross-lane reduction.
// ksplit wavefronts share a row group, each taking a part of K; the parts are
// summed through LDS (exact int32).  A workgroup holds `groups` row groups:
// 2 x 2 wavefronts when N fills the device that way, fewer rows per workgroup
// and more K parts when it does not.
#ifdef AQ_LAB
// Lab build only (csrc/aq_lab.h, aq_lab_set_gemv_timeline): where the wavefronts of the matrix-core GEMV leave
// time stamps of the 100 MHz counter, 8 per wavefront.  Expands to nothing in the product library.
__device__ long long* gv_timeline = nullptr;
__device__ int gv_skip_weights = 0;  // != 0: the kernel that quantises its rows requests no weight bytes (products of zeros)
#define GV_STAMP(slot)                                                                                          \
  do {                                                                                                          \
    if (gv_timeline && lane == 0) gv_timeline[((size_t)blockIdx.x * 16 + wave) * 8 + (slot)] = wall_clock64(); \
  } while (0)
#else
#define GV_STAMP(slot) \
  do {                 \
  } while (0)
#endif

constexpr int GM_ROWS = 16;    // weight rows per wavefront
constexpr int GM_MAX_WAVES = 8;
constexpr int GM_BATCH = 8;    // MFMA steps (64 K bytes each) per register batch

// KS, GR: K parts and row groups per workgroup fixed at compile time (the common 2 x 2 shape), or 0: taken
// from the arguments.  RES: a residual is added (a compile-time switch: a conditional early load makes the
// compiler drain the weight loads at the join, 0.4 us of a 6.5 us launch).
// XR: rounds of token-code vectors (8 per thread each) requested ahead of the weight stream; rows too long for
// XR rounds copy the rest afterwards, which waits for the weight loads in flight.
// FQ > 0: the kernel quantises up to FQ (8 or 16) bf16 token rows of at most 2048 elements itself, one or two
// rows per wavefront of a KS x GR = 8 wavefront workgroup, while its weight loads are in flight (the row
// arithmetic of the stand-alone quantiser, shared through aq_rows.h: same codes and scales); NORM: after
// RMS-normalising them with the gain p.gamma.  One launch per decode step instead of two.
// FP8: weights and tokens are OCP e4m3fn codes with one scale per tensor (p.sx, p.sw point to scalars) and the
// products run on v_mfma_f32_16x16x128_f8f6f4 -- one instruction per 128-byte line instead of two -- with fp32
// accumulation; with FQ the kernel casts its bf16 rows itself, after the maximum over ALL rows (the per-tensor
// scale of aq_quant_tensor_fp8: s = amax / 448, codes = e4m3(clamp(x / s))) has gone round the workgroup.
// SWI: the weight is an MLP's up and gate projections stacked, rows [0, F) up and [F, 2F) gate with F = N / 2 (what
// QuantLinear.concat([up, gate]) builds), and the kernel writes h = up * silu(gate), [M, F], instead of the 2F
// projections: the first half of a workgroup's row groups takes 16-row blocks of up, the second half the same
// blocks of gate, the gate sums cross to the up wavefronts through LDS, and the up wavefronts apply the activation
// (the fixed-sequence exponential and correctly rounded divide of the stand-alone SwiGLU kernel) to the two
// projections as the separate launch would have stored them (rounded to the output type first).
template <int KS, int GR, bool RES, int XR, int FQ = 0, bool NORM = false, bool FP8 = false, bool SWI = false>
__global__ __launch_bounds__(GM_MAX_WAVES * 64) void gemv_mfma_kernel(GemvArgs p) {
  static_assert(FQ == 0 || (KS > 0 && GR > 0), "the in-kernel quantiser deals rows to a fixed number of wavefronts");
  static_assert(!(FP8 && NORM), "no fused norm in front of the FP8 cast");
  static_assert(!SWI || (FQ > 0 && !RES && !FP8 && GR % 2 == 0), "the SwiGLU epilogue exists for the int8 kernels that quantise their rows");
  extern __shared__ __attribute__((aligned(16))) uint8_t xs[];  // [16][K + 16] token codes, [16] scales, 16 spare bytes; later the partial sums
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ksplit = KS ? KS : p.ksplit, groups = GR ? GR : p.groups;
  const int nthreads = ksplit * groups * 64;
  const int grp = wave / ksplit, kh = wave % ksplit;
  const int K = p.K, N = p.N, M = p.M;
  // first weight row of this wavefront's group, and the end of the rows it may touch
  const int FH = N >> 1;  // SWI: rows per half
  const int hgroups = SWI ? groups >> 1 : groups;
  const int ghalf = SWI ? grp / hgroups : 0, gsub = SWI ? grp - ghalf * hgroups : grp;
  const int n0 = __builtin_amdgcn_readfirstlane((SWI ? ghalf * FH : 0) + (blockIdx.x * hgroups + gsub) * GM_ROWS);
  const int nlim = SWI ? (ghalf + 1) * FH : N;
  const int pitch = K + 16;  // 16 token rows then start 4 banks apart: conflict-free 16-byte reads
  const int khalf = K / ksplit;  // a multiple of 128 (checked by the launcher)
  const int nline = khalf / 128;  // 128-byte lines of a row's K part: two MFMA steps each

  // epilogue operands first: lane l -> token l%16, rows (l/16)*4 .. +3 of the group
  const int tok = lane & 15;
  const int rbase = n0 + (lane >> 4) * 4;
  float swv[4], bv[4];
  uint32_t rv[4];  // residual elements, raw bits
  // only the first K part's wavefront writes outputs: the others get empty descriptors.  Requested (load_epi)
  // between the token rows and the weight stream.  Loads return in request order: behind the weights the
  // epilogue would wait for the whole stream to drain (0.2 us), and in front of the tokens these few lines, which
  // no other workgroup shares and which therefore come from HBM, hold back the token rows that every workgroup
  // reads and the caches serve (M = 16, N = 8192: 7.45 -> 7.2 us with the rows quantised here, 5.85 -> 5.65 us on
  // codes).
  const EpiOperands epi(p, kh == 0, FQ == 0, RES);
  float sxv = 0.0f;
  auto load_epi = [&]() {
    sxv = epi.load_sx(FP8 ? 0 : tok, FP8 || tok < M);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int n = rbase + r;
      swv[r] = epi.load_sw(FP8 ? 0 : n, FP8 || n < nlim);
      bv[r] = epi.load_bias(n, n < nlim);
      rv[r] = RES ? epi.load_res(tok, n, tok < M && n < nlim, (int)p.ldr) : 0u;
    }
  };

  // weight stream: descriptor over this wavefront's 16 rows; rows past N read as zero
  const int rows = n0 < nlim ? ((nlim - n0) < GM_ROWS ? (nlim - n0) : GM_ROWS) : 0;
#ifdef AQ_LAB
  const __amdgpu_buffer_rsrc_t Wr = make_rsrc(p.wq + (int64_t)(n0 < nlim ? n0 : 0) * K,
                                              FQ > 0 && gv_skip_weights ? 0u : (uint32_t)rows * (uint32_t)K);
#else
  const __amdgpu_buffer_rsrc_t Wr =
      make_rsrc(p.wq + (int64_t)(n0 < nlim ? n0 : 0) * K, (uint32_t)rows * (uint32_t)K);
#endif
  // Whole 128-byte lines per load: an instruction covers one line of 8 rows (lane l: row l % 8, 16-byte piece
  // l / 8), two instructions (rows 0..7 and 8..15) per line index.  In the MFMA's own operand order (lane l: row
  // l % 16, piece l / 16 of a 64-byte step) an instruction would cover 16 half lines, and a one-shot read of
  // the weight in that pattern measures 0.35 us slower (4.65 against 4.30 us for 16 MiB).  The operands are put
  // together from a line's two registers by one row rotation per dword (see consume).
  const uint32_t woff = (uint32_t)(lane & 7) * (uint32_t)K + (uint32_t)(kh * khalf + (lane >> 3) * 16);
  const uint32_t woff8 = 8u * (uint32_t)K;
  constexpr int GM_LINES = GM_BATCH / 2;  // lines per register batch
  uint4 wa[GM_BATCH], wb[GM_BATCH];       // [2 t]: rows 0..7 of line t, [2 t + 1]: rows 8..15
  auto wload = [&](int line0, uint4 (&dst)[GM_BATCH]) {
#pragma unroll
    for (int t = 0; t < GM_LINES; ++t) {
      const bool ok = (line0 + t) < nline;
      const uint32_t o = woff + (uint32_t)(line0 + t) * 128u;
      dst[2 * t] = GV_WLOAD(Wr, ok ? o : OOB_OFFSET);
      dst[2 * t + 1] = GV_WLOAD(Wr, ok ? o + woff8 : OOB_OFFSET);
    }
  };

  // token codes -> LDS (padded rows; tokens >= M are zero).  Their loads are
  // issued before the weight loads, so they return first and the LDS fill
  // overlaps the weight stream's flight time.
  float* const sx_lds = reinterpret_cast<float*>(xs + 16 * pitch);
  if constexpr (FQ > 0) {
    // produced here: every wavefront requests its bf16 rows, then its weights, then rounds the rows while the
    // weights are in flight.  Rows >= M are not written: the lanes of those tokens read row 0 and their
    // products are never stored.
    constexpr int WAVES = KS * GR, RPW = (FQ + WAVES - 1) / WAVES;
    RowsToLds<true, RPW, 4> xrows;
    xrows.issue(p.x, M, K, K, wave, WAVES, lane);
    if constexpr (NORM) xrows.issue_gamma(p.gamma, K, lane);
    asm volatile("" ::: "memory");  // request order: token rows, epilogue operands, the weight stream
    load_epi();
    asm volatile("" ::: "memory");
    GV_STAMP(0);
    wload(0, wa);
    wload(GM_LINES, wb);
    asm volatile("" ::: "memory");
    if constexpr (!FP8) {
      xrows.template finish<NORM>(M, M, K, xs, pitch, sx_lds, wave, WAVES, lane, p.eps);
      GV_STAMP(3);
    } else {
      // the tensor's maximum: every wavefront's share through LDS (a maximum has no order), then the cast
      float amax = 0.0f;
#pragma unroll
      for (int j = 0; j < RPW; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float f[8];
          RowIn<true>::unpack(xrows.c[j][i], f);  // rows >= M and vectors past K were loaded as zeros
          amax = fmaxf(amax, vec_amax<8>(f));
        }
      amax = wave_max(amax);
      if (lane == 0) sx_lds[wave] = amax;
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();  // no memory fence: the weight loads stay in flight
      asm volatile("" ::: "memory");
      float all = 0.0f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) all = fmaxf(all, sx_lds[w]);
      float sc = __fdiv_rn(all, 448.0f);
      if (all == 0.0f) sc = 1.0f;
      sxv = sc;
      const float rsc = __fdiv_rn(1.0f, sc);  // correctly rounded: what the one-step sequence below needs
      const bool lean_ok = sc >= 5.421010862427522e-20f && sc <= 1.8446744073709552e19f;  // [2^-64, 2^64]
      const int nvec = K / 8;
#pragma unroll
      for (int j = 0; j < RPW; ++j) {
        const int m = wave + j * WAVES;
        if (m >= M) continue;  // uniform
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int v = i * 64 + lane;
          if (v < nvec) {
            float f[8];
            RowIn<true>::unpack(xrows.c[j][i], f);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              // x / s: the one-correction sequence that gives a bf16 number's e4m3 code exactly for in-range
              // scales (see quant_codes; a -0.0 comes out as +0.0, which no product can tell apart), the
              // divide itself otherwise; then the clamp to the e4m3 range
              float q;
              if (__builtin_expect(lean_ok, 1)) {
                q = f[e] * rsc;
                q = __builtin_fmaf(__builtin_fmaf(-sc, q, f[e]), rsc, q);
              } else {
                q = __fdiv_rn(f[e], sc);
              }
              f[e] = fminf(fmaxf(q, -448.0f), 448.0f);
            }
            int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false);
            w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w0, true);
            int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], 0, false);
            w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], w1, true);
            *reinterpret_cast<uint2*>(xs + m * pitch + v * 8) = make_uint2((uint32_t)w0, (uint32_t)w1);
          }
        }
      }
    }
  } else {
    const __amdgpu_buffer_rsrc_t Xr = make_rsrc(p.xq, (uint32_t)M * (uint32_t)K);
    const int nvec_row = K / 16;
    const int nvec = 16 * nvec_row;
    constexpr int XV = 8;  // vectors per thread per round: 16 x 2048 codes in one round of 256 threads
    uint4 xvr[XR][XV];
    auto xload = [&](int v0, uint4 (&xv)[XV]) {
#pragma unroll
      for (int i = 0; i < XV; ++i) {
        const int v = v0 + i * nthreads + tid;
        xv[i] = buffer_load_16(Xr, v < nvec ? (uint32_t)v * 16u : OOB_OFFSET);
      }
    };
    // Stores without a branch: vectors past the end go to the spare slot behind the scales.  (With the
    // store under `if (v < nvec)` the compiler sank a vector's load into that branch, behind the weight
    // loads, and then waited for every load of the wavefront before the first LDS store: the matrix
    // products started only after the whole weight stream had landed.)
    uint8_t* const spare = xs + 16 * pitch + 16 * sizeof(float);
    auto xstore = [&](int v0, const uint4 (&xv)[XV]) {
#pragma unroll
      for (int i = 0; i < XV; ++i) {
        const int v = v0 + i * nthreads + tid;
        const int m = v / nvec_row, c = v - m * nvec_row;
        *reinterpret_cast<uint4*>(v < nvec ? xs + m * pitch + c * 16 : spare) = xv[i];
      }
    };
#pragma unroll
    for (int r = 0; r < XR; ++r) xload(r * XV * nthreads, xvr[r]);
    asm volatile("" ::: "memory");  // request order: token codes, epilogue operands, the weight stream
    load_epi();
    asm volatile("" ::: "memory");
    wload(0, wa);
    wload(GM_LINES, wb);
    asm volatile("" ::: "memory");
#pragma unroll
    for (int r = 0; r < XR; ++r) xstore(r * XV * nthreads, xvr[r]);  // waits for the token codes only: the oldest requests
    for (int v0 = XR * XV * nthreads; v0 < nvec; v0 += XV * nthreads) {  // still longer rows
      xload(v0, xvr[0]);
      xstore(v0, xvr[0]);
    }
  }
  // LDS writes done, then a barrier without a memory fence: the weight loads stay in flight
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  if constexpr (FQ > 0 && !FP8) sxv = sx_lds[tok < M ? tok : 0];
  GV_STAMP(4);

  // Four independent accumulators (summed at the end: int32, exact in any order) and a batch's token
  // fragments read from LDS up front: one chain of 16 dependent read -> MFMA steps took 0.6 us after the
  // token codes had landed, which is all on the kernel's critical path.
  using accv = std::conditional_t<FP8, v4f, v4i>;
  accv accs[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) accs[i] = accv{0, 0, 0, 0};
  // MFMA step (t, e) of line t takes, for weight row r = lane % 16 and token lane % 16, the line's piece
  // 2 (lane / 16) + e: K bytes t 128 + (2 q + e) 16 of the wavefront's part.  (Any assignment of K bytes to the
  // steps' k slots is a valid product as long as both operands use the same one.)  Lane l holds piece l / 8 of
  // row l % 8 (register lo) and of row 8 + l % 8 (register hi), so lanes 0..7 of each row of 16 lanes have
  // their operand of step e = 0 in lo, and lanes 8..15 find theirs in hi of lane l - 8; for e = 1 it is lo of
  // lane l + 8 and the own hi: one rotation by 8 within the row of 16 lanes, written into half of the lanes.
  const uint8_t* xl = xs + (FQ > 0 && tok >= M ? 0 : tok) * pitch + kh * khalf + (lane >> 4) * 32;
  auto consume = [&](int line0, const uint4 (&wc)[GM_BATCH]) {
    v4i x[GM_BATCH];
#pragma unroll
    for (int t = 0; t < GM_LINES; ++t) {
      const int ln = (line0 + t) < nline ? (line0 + t) : 0;  // lines past the end multiply zero weights
      x[2 * t] = *reinterpret_cast<const v4i*>(xl + ln * 128);
      x[2 * t + 1] = *reinterpret_cast<const v4i*>(xl + ln * 128 + 16);
    }
#pragma unroll
    for (int t = 0; t < GM_LINES; ++t) {
      const uint4 lo = wc[2 * t], hi = wc[2 * t + 1];
      constexpr int ROR8 = 0x128;  // DPP row_ror:8
      // e = 0: lanes 8..15 of each row (banks 2, 3) take hi from lane l - 8, the others keep lo
      const v4i w0 = {__builtin_amdgcn_update_dpp((int)lo.x, (int)hi.x, ROR8, 0xf, 0xc, false),
                      __builtin_amdgcn_update_dpp((int)lo.y, (int)hi.y, ROR8, 0xf, 0xc, false),
                      __builtin_amdgcn_update_dpp((int)lo.z, (int)hi.z, ROR8, 0xf, 0xc, false),
                      __builtin_amdgcn_update_dpp((int)lo.w, (int)hi.w, ROR8, 0xf, 0xc, false)};
      // e = 1: lanes 0..7 of each row (banks 0, 1) take lo from lane l + 8, the others keep hi
      const v4i w1 = {__builtin_amdgcn_update_dpp((int)hi.x, (int)lo.x, ROR8, 0xf, 0x3, false),
                      __builtin_amdgcn_update_dpp((int)hi.y, (int)lo.y, ROR8, 0xf, 0x3, false),
                      __builtin_amdgcn_update_dpp((int)hi.z, (int)lo.z, ROR8, 0xf, 0x3, false),
                      __builtin_amdgcn_update_dpp((int)hi.w, (int)lo.w, ROR8, 0xf, 0x3, false)};
      if constexpr (!FP8) {
        accs[(2 * t) & 3] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w0, x[2 * t], accs[(2 * t) & 3], 0, 0, 0);
        accs[(2 * t + 1) & 3] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w1, x[2 * t + 1], accs[(2 * t + 1) & 3], 0, 0, 0);
      } else {
        // the line's pieces 2q and 2q + 1 are the 32 K bytes lane (row, q) feeds one 16x16x128 product
        const v8i wl = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
        const v4i xa = x[2 * t], xb = x[2 * t + 1];
        const v8i xl8 = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
        accs[t & 3] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wl, xl8, accs[t & 3], 0, 0, 0, 0, 0, 0);
      }
    }
  };
  for (int l0 = 0; l0 < nline; l0 += 2 * GM_LINES) {
    consume(l0, wa);
    if (l0 + 2 * GM_LINES < nline) wload(l0 + 2 * GM_LINES, wa);
    if (l0 + GM_LINES < nline) consume(l0 + GM_LINES, wb);
    if (l0 + 3 * GM_LINES < nline) wload(l0 + 3 * GM_LINES, wb);
  }

  accv acc = (accs[0] + accs[1]) + (accs[2] + accs[3]);
  GV_STAMP(5);
  // sum the K parts: all but the first wavefront of each group park their 4 sums in LDS
  __syncthreads();  // everyone is done reading the token codes: the buffer is reused
  int* part = reinterpret_cast<int*>(xs) + grp * (ksplit - 1) * 256;
  if (kh != 0) {
    *reinterpret_cast<accv*>(part + (kh - 1) * 256 + lane * 4) = acc;
  }
  __syncthreads();
  if constexpr (SWI) {
    // every wavefront stays for the exchange: gate sums -> LDS (behind the K-part area) -> the up wavefronts
    float* const ex = reinterpret_cast<float*>(xs) + groups * (ksplit - 1) * 256 + (gsub * 64 + lane) * 4;
    const bool live = kh == 0;
    float u[4];
    if (live) {
      for (int k = 0; k < ksplit - 1; ++k) acc += *reinterpret_cast<const accv*>(part + k * 256 + lane * 4);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        u[r] = __fmul_rn(__fmul_rn((float)acc[r], sxv), swv[r]);
        if (p.bias) u[r] = __fadd_rn(u[r], bv[r]);
        if (p.y_dtype == AQ_BF16) u[r] = bf16_bits_to_f32(f32_to_bf16_bits(u[r]));  // as the projection would be stored
      }
      if (ghalf == 1) *reinterpret_cast<float4*>(ex) = make_float4(u[0], u[1], u[2], u[3]);
    }
    __syncthreads();
    if (!live || ghalf == 1 || tok >= M) return;
    const float4 g4 = *reinterpret_cast<const float4*>(ex);
    const float g[4] = {g4.x, g4.y, g4.z, g4.w};
    float h[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) h[r] = swiglu_repro(u[r], g[r]);
    const int64_t o = (int64_t)tok * FH + rbase;  // rbase lies in the up half: the column of h
    if (p.y_dtype == AQ_BF16) {
      uint16_t* dst = reinterpret_cast<uint16_t*>(p.y) + o;
      if ((FH & 3) == 0 && rbase + 3 < FH) {
        uint2 pk;
        pk.x = pack_bf16x2(h[0], h[1]);
        pk.y = pack_bf16x2(h[2], h[3]);
        *reinterpret_cast<uint2*>(dst) = pk;
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (rbase + r < FH) dst[r] = (uint16_t)f32_to_bf16_bits(h[r]);
      }
    } else {
      float* dst = reinterpret_cast<float*>(p.y) + o;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (rbase + r < FH) dst[r] = h[r];
    }
    return;
  }
  if (kh != 0) return;
  for (int k = 0; k < ksplit - 1; ++k) acc += *reinterpret_cast<const accv*>(part + k * 256 + lane * 4);  // fp32: a fixed order

  if (tok >= M) return;
  float y[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    y[r] = __fmul_rn(__fmul_rn((float)acc[r], sxv), swv[r]);
    if (p.bias) y[r] = __fadd_rn(y[r], bv[r]);
    if constexpr (RES) y[r] = p.y_dtype == AQ_BF16 ? add_residual_bf16(y[r], rv[r]) : __fadd_rn(y[r], __uint_as_float(rv[r]));
  }
  const int64_t o = (int64_t)tok * N + rbase;
  if (p.y_dtype == AQ_BF16) {
    uint16_t* dst = reinterpret_cast<uint16_t*>(p.y) + o;
    if ((N & 3) == 0 && rbase + 3 < N) {  // 8-byte aligned and fully inside
      uint2 pk;
      pk.x = pack_bf16x2(y[0], y[1]);
      pk.y = pack_bf16x2(y[2], y[3]);
      *reinterpret_cast<uint2*>(dst) = pk;
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (rbase + r < N) dst[r] = (uint16_t)f32_to_bf16_bits(y[r]);
    }
  } else {
    float* dst = reinterpret_cast<float*>(p.y) + o;
    if ((N & 3) == 0 && rbase + 3 < N) {
      *reinterpret_cast<float4*>(dst) = make_float4(y[0], y[1], y[2], y[3]);
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (rbase + r < N) dst[r] = y[r];
    }
  }
  GV_STAMP(6);
}

// the streaming MFMA variant needs K in whole 256-byte steps (two K parts of whole 128-byte lines)
// and its padded codes to fit LDS
static bool gemv_mfma_ok(int64_t M, int64_t K) {
  return M > GV_MFMA_MIN_M && (K % 256) == 0 && 16 * (K + 16) + 64 + 16 <= GV_MAX_LDS;
}

static int launch_gemv_mfma(GemvArgs a, hipStream_t st, bool fp8 = false) {
  // 2 row groups x 2 K parts per workgroup by default; with too few rows for that to give every
  // compute unit a workgroup, one row group per workgroup and up to 8 K parts
  a.ksplit = 2;
  a.groups = 2;
  const int cus = device_cus();
  if ((a.N + 31) / 32 < cus) {
    a.groups = 1;
    while (a.ksplit < GM_MAX_WAVES && (a.N + 15) / 16 * (a.ksplit / 2) < cus && a.K % (256 * a.ksplit) == 0 &&
           a.K / (2 * a.ksplit) >= 512)
      a.ksplit *= 2;
  }
  const unsigned grid = (unsigned)((a.N + GM_ROWS * a.groups - 1) / (GM_ROWS * a.groups));
  const size_t lds = (size_t)16 * (a.K + 16) + 16 * sizeof(float) + 16;
  const bool fixed = a.ksplit == 2 && a.groups == 2, res = a.res != nullptr;
  // one round of token-code loads ahead of the weights covers 8 vectors per thread; longer rows take three
  const bool long_rows = (int64_t)16 * (a.K / 16) > (int64_t)8 * a.ksplit * a.groups * 64;
  using kern_t = void (*)(GemvArgs);
  static const kern_t table[2][2][2][2] = {
      {{{gemv_mfma_kernel<0, 0, false, 1>, gemv_mfma_kernel<0, 0, false, 3>},
        {gemv_mfma_kernel<0, 0, true, 1>, gemv_mfma_kernel<0, 0, true, 3>}},
       {{gemv_mfma_kernel<2, 2, false, 1>, gemv_mfma_kernel<2, 2, false, 3>},
        {gemv_mfma_kernel<2, 2, true, 1>, gemv_mfma_kernel<2, 2, true, 3>}}},
      {{{gemv_mfma_kernel<0, 0, false, 1, 0, false, true>, gemv_mfma_kernel<0, 0, false, 3, 0, false, true>},
        {gemv_mfma_kernel<0, 0, true, 1, 0, false, true>, gemv_mfma_kernel<0, 0, true, 3, 0, false, true>}},
       {{gemv_mfma_kernel<2, 2, false, 1, 0, false, true>, gemv_mfma_kernel<2, 2, false, 3, 0, false, true>},
        {gemv_mfma_kernel<2, 2, true, 1, 0, false, true>, gemv_mfma_kernel<2, 2, true, 3, 0, false, true>}}}};
  const kern_t fn = table[fp8][fixed][res][long_rows];
  if (lds > 64 * 1024) {
    static LdsOptIn opted[16];
    const int e = opted[fp8 * 8 + fixed * 4 + res * 2 + long_rows].ensure(reinterpret_cast<const void*>(fn));
    if (e) return e;
  }
  hipLaunchKernelGGL(fn, dim3(grid), dim3(a.ksplit * a.groups * 64), lds, st, a);
  return (int)hipGetLastError();
}

// The matrix-core variant that quantises its token rows itself (8 wavefronts per workgroup, a row -- two above
// 8 tokens -- per wavefront), where it measured faster than the alternatives (bf16 rows of K = 2048, one launch):
//   9..16 tokens: always (N = 8192: 7.6 us against 8.4 us for row quantiser + GEMV; N = 2048: 6.6 against 7.1);
//   5..8 tokens: from N = 8192 on (6.45 us against 7.4 us for the dot-product kernel, which is bound by its
//                vector ALU there; at N = 4096 the dot-product kernel still wins, 4.8 against 5.2 us);
//                with the norm folded in, whose arithmetic weighs on the dot-product kernel's fewer wavefronts,
//                from N = 6144 on (7.2 -> 6.5 us there; level at N = 3072);
//   3..4 tokens: only for matrices with more 32-row blocks than compute units (N = 11264: 7.0 against 7.6 us).
static bool gemv_mfma_fq_ok(int64_t M, int64_t N, int64_t K, bool norm = false) {
  if (K > 2048 || (K % 512) != 0) return false;
  const bool wide = (N + 31) / 32 > device_cus();
  return M >= 9 || (M >= 5 && N >= (norm ? 6144 : 8192)) || (M >= 3 && wide);
}

static int launch_gemv_mfma_fq(GemvArgs a, hipStream_t st, bool fp8 = false) {
  // 32 weight rows per workgroup (2 row groups x 4 K parts) while that gives every workgroup a compute unit
  // of its own; beyond that 64 rows (4 row groups x 2 K parts): a second round of workgroups would repeat
  // the row quantisation behind the first (N = 11264, 8 tokens: 9.9 -> 7.1 us).
  const bool wide = (a.N + 31) / 32 > device_cus();
  a.ksplit = wide ? 2 : 4;
  a.groups = wide ? 4 : 2;
  const unsigned grid = (unsigned)((a.N + GM_ROWS * a.groups - 1) / (GM_ROWS * a.groups));
  const size_t lds = (size_t)16 * (a.K + 16) + 16 * sizeof(float) + 16;
  const bool res = a.res != nullptr, many = a.M > 8, norm = a.gamma != nullptr;
  using kern_t = void (*)(GemvArgs);
#define AQ_FQ_TABLE(KS, GR)                                                                                  \
  {{{gemv_mfma_kernel<KS, GR, false, 1, 8, false>, gemv_mfma_kernel<KS, GR, false, 1, 8, true>},             \
    {gemv_mfma_kernel<KS, GR, false, 1, 16, false>, gemv_mfma_kernel<KS, GR, false, 1, 16, true>}},          \
   {{gemv_mfma_kernel<KS, GR, true, 1, 8, false>, gemv_mfma_kernel<KS, GR, true, 1, 8, true>},               \
    {gemv_mfma_kernel<KS, GR, true, 1, 16, false>, gemv_mfma_kernel<KS, GR, true, 1, 16, true>}}}
  static const kern_t table[2][2][2][2] = {AQ_FQ_TABLE(4, 2), AQ_FQ_TABLE(2, 4)};
#undef AQ_FQ_TABLE
#define AQ_FQ8_TABLE(KS, GR)                                                                                       \
  {{gemv_mfma_kernel<KS, GR, false, 1, 8, false, true>, gemv_mfma_kernel<KS, GR, false, 1, 16, false, true>},      \
   {gemv_mfma_kernel<KS, GR, true, 1, 8, false, true>, gemv_mfma_kernel<KS, GR, true, 1, 16, false, true>}}
  static const kern_t table8[2][2][2] = {AQ_FQ8_TABLE(4, 2), AQ_FQ8_TABLE(2, 4)};
#undef AQ_FQ8_TABLE
  const kern_t fn = fp8 ? table8[wide][res][many] : table[wide][res][many][norm];
  hipLaunchKernelGGL(fn, dim3(grid), dim3(8 * 64), lds, st, a);
  return (int)hipGetLastError();
}

// up/gate + SwiGLU in one launch: bf16 rows of K <= 2048 in whole 512-byte steps, F a multiple of 16.
static bool gemv_mfma_swiglu_ok(int64_t M, int64_t F, int64_t K) {
  return M >= 1 && M <= 16 && F > 0 && (F % 16) == 0 && K <= 2048 && (K % 512) == 0;
}

// a.N = 2 F.  A workgroup holds 16 (2 x 4 wavefronts: up block, gate block) or, once F has more 16-row blocks than the
// device has compute units, 32 columns of h (4 x 2 wavefronts).
static int launch_gemv_mfma_swiglu(GemvArgs a, hipStream_t st) {
  const int F = a.N / 2;
  const bool wide = (F + 15) / 16 > device_cus();
  a.ksplit = wide ? 2 : 4;
  a.groups = wide ? 4 : 2;
  const int per_wg = GM_ROWS * (a.groups / 2);
  const unsigned grid = (unsigned)((F + per_wg - 1) / per_wg);
  const size_t lds = (size_t)16 * (a.K + 16) + 16 * sizeof(float) + 16;
  const bool many = a.M > 8, norm = a.gamma != nullptr;
  using kern_t = void (*)(GemvArgs);
#define AQ_SWI_TABLE(KS, GR)                                                                                   \
  {{gemv_mfma_kernel<KS, GR, false, 1, 8, false, false, true>, gemv_mfma_kernel<KS, GR, false, 1, 8, true, false, true>},   \
   {gemv_mfma_kernel<KS, GR, false, 1, 16, false, false, true>, gemv_mfma_kernel<KS, GR, false, 1, 16, true, false, true>}}
  static const kern_t table[2][2][2] = {AQ_SWI_TABLE(4, 2), AQ_SWI_TABLE(2, 4)};
#undef AQ_SWI_TABLE
  hipLaunchKernelGGL(table[wide][many][norm], dim3(grid), dim3(8 * 64), lds, st, a);
  return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------
// 17..32 tokens on codes: the same weight stream (every weight byte HBM -> registers once, operands assembled by
// one DPP rotation per dword) with TG = 2 groups of 16 tokens multiplied against each weight fragment.  Between the
// decode batch sizes above and the tiled GEMM (whose smallest tile, 64 x 32, spends the matrix-core time of 64
// rows whatever M is: 32 x 8192 x 2048 in 6.9 us with the weights streamed from HBM) this kernel stays a
// bandwidth-bound launch (6.0 us); from 33 tokens on, with a third and fourth token group, it was the slower one
// (48 rows: 6.1 us, 64 rows: 7.6 us with the weights in the last-level cache, where a 128 x 32 tile took 5.8 us),
// so those go to the tiles.  Same integer sums, same epilogue: the bits of the tiled GEMM.
// K is walked in chunks of 1024 bytes per wavefront (KS wavefronts per row group: 1024-, 2048- or 4096-byte chunks
// per workgroup), the token codes of one chunk at a time in LDS, so that rows of any length are taken (an MLP's
// down projection) and the LDS of a compute unit holds several workgroups.  A chunk's codes are requested into
// registers while the chunk before is multiplied and stored between two barriers; the weight stream runs through
// the chunk boundaries untouched (two register batches, each reloaded as soon as it has been consumed).  GRP row
// groups of 16 rows per workgroup (every workgroup copies all token codes from L2: more rows per workgroup for
// matrices of more 32-row blocks than compute units); rows must be whole 128-byte lines (K % 128 == 0).
// FP8: e4m3 codes with one scale per tensor and fp32 accumulation, as in gemv_mfma_kernel (chunks and K parts
// summed in a fixed order).
template <int TG, int KS, bool RES, int GRP = 2, bool FP8 = false>
__global__ __launch_bounds__(KS * GRP * 64) void gemv_mfma_tokens_kernel(GemvArgs p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t xs[];  // [16 TG][KC + 16] codes of one chunk; later the partial sums
  constexpr int MTOK = 16 * TG, NTHREADS = KS * GRP * 64;
  constexpr int KC = 1024 * KS;            // K bytes of a chunk
  constexpr int PITCH = KC + 16;
  constexpr int XV = MTOK * (KC / 16) / NTHREADS;  // 16-byte vectors of a chunk's codes per thread: 16 / GRP per token group
  static_assert(XV * NTHREADS == MTOK * (KC / 16) && MTOK * PITCH <= 150 * 1024 && KS * GRP <= GM_MAX_WAVES,
                "a chunk's codes: whole vectors per thread, within LDS");
  static_assert(GRP * (KS - 1) * TG * 1024 <= MTOK * PITCH, "the partial sums reuse the codes' LDS");
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = wave / KS, kh = wave % KS;
  const int K = p.K, N = p.N, M = p.M;
  const int n0 = __builtin_amdgcn_readfirstlane((blockIdx.x * GRP + grp) * GM_ROWS);
  const int nchunk = (K + KC - 1) / KC;

  const int tok = lane & 15;
  const int rbase = n0 + (lane >> 4) * 4;
  float swv[4], bv[4], sxv[TG];
  uint32_t rv[TG][4];
  const EpiOperands epi(p, kh == 0, true, RES);

  const int rows = n0 < N ? ((N - n0) < GM_ROWS ? (N - n0) : GM_ROWS) : 0;
  const __amdgpu_buffer_rsrc_t Wr = make_rsrc(p.wq + (int64_t)(n0 < N ? n0 : 0) * K, (uint32_t)rows * (uint32_t)K);
  const uint32_t woff = (uint32_t)(lane & 7) * (uint32_t)K + (uint32_t)((lane >> 3) * 16);
  const uint32_t woff8 = 8u * (uint32_t)K;
  constexpr int GM_LINES = GM_BATCH / 2;
  uint4 wa[GM_BATCH], wb[GM_BATCH];
  // lines line0 .. line0+3 of this wavefront's 1024 bytes of chunk c (columns past K read zeros: an offset there
  // would alias the next row, so it is pushed outside the descriptor)
  auto wload = [&](int c, int line0, uint4 (&dst)[GM_BATCH]) {
#pragma unroll
    for (int t = 0; t < GM_LINES; ++t) {
      const int col = c * KC + kh * 1024 + (line0 + t) * 128;
      const bool ok = col < K;
      const uint32_t o = woff + (uint32_t)col;
      dst[2 * t] = GV_WLOAD(Wr, ok ? o : OOB_OFFSET);
      dst[2 * t + 1] = GV_WLOAD(Wr, ok ? o + woff8 : OOB_OFFSET);
    }
  };
  const __amdgpu_buffer_rsrc_t Xr = make_rsrc(p.xq, (uint32_t)M * (uint32_t)K);
  uint4 xvr[XV];
  auto xload = [&](int c) {
#pragma unroll
    for (int i = 0; i < XV; ++i) {
      const int v = i * NTHREADS + tid;
      const int m = v / (KC / 16), cc = v - m * (KC / 16);
      const int col = c * KC + cc * 16;
      xvr[i] = buffer_load_16(Xr, (m < M && col < K) ? (uint32_t)m * (uint32_t)K + (uint32_t)col : OOB_OFFSET);
    }
  };
  auto xstore = [&]() {
#pragma unroll
    for (int i = 0; i < XV; ++i) {
      const int v = i * NTHREADS + tid;
      const int m = v / (KC / 16), cc = v - m * (KC / 16);
      *reinterpret_cast<uint4*>(xs + m * PITCH + cc * 16) = xvr[i];
    }
  };

  xload(0);
  asm volatile("" ::: "memory");  // request order: token codes, epilogue operands, the weight stream
#pragma unroll
  for (int g = 0; g < TG; ++g) sxv[g] = epi.load_sx(FP8 ? 0 : tok + 16 * g, FP8 || tok + 16 * g < M);
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int n = rbase + r;
    swv[r] = epi.load_sw(FP8 ? 0 : n, FP8 || n < N);
    bv[r] = epi.load_bias(n, n < N);
#pragma unroll
    for (int g = 0; g < TG; ++g) rv[g][r] = RES ? epi.load_res(tok + 16 * g, n, tok + 16 * g < M && n < N, (int)p.ldr) : 0u;
  }
  asm volatile("" ::: "memory");
  wload(0, 0, wa);
  wload(0, GM_LINES, wb);
  asm volatile("" ::: "memory");

  using accv = std::conditional_t<FP8, v4f, v4i>;
  accv accs[TG][2];
#pragma unroll
  for (int g = 0; g < TG; ++g) accs[g][0] = accs[g][1] = accv{0, 0, 0, 0};
  const uint8_t* xl = xs + tok * PITCH + kh * 1024 + (lane >> 4) * 32;
  auto consume = [&](int line0, const uint4 (&wc)[GM_BATCH]) {
#pragma unroll
    for (int t = 0; t < GM_LINES; ++t) {
      v4i x0[TG], x1[TG];
#pragma unroll
      for (int g = 0; g < TG; ++g) {
        x0[g] = *reinterpret_cast<const v4i*>(xl + g * 16 * PITCH + (line0 + t) * 128);
        x1[g] = *reinterpret_cast<const v4i*>(xl + g * 16 * PITCH + (line0 + t) * 128 + 16);
      }
      const uint4 lo = wc[2 * t], hi = wc[2 * t + 1];
      constexpr int ROR8 = 0x128;  // DPP row_ror:8 (see gemv_mfma_kernel)
      const v4i w0 = {__builtin_amdgcn_update_dpp((int)lo.x, (int)hi.x, ROR8, 0xf, 0xc, false),
                      __builtin_amdgcn_update_dpp((int)lo.y, (int)hi.y, ROR8, 0xf, 0xc, false),
                      __builtin_amdgcn_update_dpp((int)lo.z, (int)hi.z, ROR8, 0xf, 0xc, false),
                      __builtin_amdgcn_update_dpp((int)lo.w, (int)hi.w, ROR8, 0xf, 0xc, false)};
      const v4i w1 = {__builtin_amdgcn_update_dpp((int)hi.x, (int)lo.x, ROR8, 0xf, 0x3, false),
                      __builtin_amdgcn_update_dpp((int)hi.y, (int)lo.y, ROR8, 0xf, 0x3, false),
                      __builtin_amdgcn_update_dpp((int)hi.z, (int)lo.z, ROR8, 0xf, 0x3, false),
                      __builtin_amdgcn_update_dpp((int)hi.w, (int)lo.w, ROR8, 0xf, 0x3, false)};
#pragma unroll
      for (int g = 0; g < TG; ++g) {
        if constexpr (!FP8) {
          accs[g][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w0, x0[g], accs[g][0], 0, 0, 0);
          accs[g][1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w1, x1[g], accs[g][1], 0, 0, 0);
        } else {  // the line's two pieces are the 32 K bytes a lane feeds one 16x16x128 product
          const v8i wl = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
          const v8i xl8 = {x0[g].x, x0[g].y, x0[g].z, x0[g].w, x1[g].x, x1[g].y, x1[g].z, x1[g].w};
          accs[g][t & 1] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wl, xl8, accs[g][t & 1], 0, 0, 0, 0, 0, 0);
        }
      }
    }
  };
  // barriers without a memory fence (LDS traffic only has to be complete): the weight loads stay in flight
  auto lds_barrier = [&]() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  for (int c = 0; c < nchunk; ++c) {
    if (c > 0) lds_barrier();  // every wavefront is done with the codes of the chunk before
    xstore();                  // waits for this chunk's codes only: they are older than the weight loads in flight
    lds_barrier();
    if (c + 1 < nchunk) xload(c + 1);
    consume(0, wa);
    if (c + 1 < nchunk) wload(c + 1, 0, wa);
    consume(GM_LINES, wb);
    if (c + 1 < nchunk) wload(c + 1, GM_LINES, wb);
  }

  // sum the K parts through LDS (int32: exact; fp32: in a fixed order)
  __syncthreads();
  int* part = reinterpret_cast<int*>(xs) + (grp * (KS - 1)) * TG * 256;
  accv acc[TG];
#pragma unroll
  for (int g = 0; g < TG; ++g) acc[g] = accs[g][0] + accs[g][1];
  if (kh != 0) {
#pragma unroll
    for (int g = 0; g < TG; ++g) *reinterpret_cast<accv*>(part + ((kh - 1) * TG + g) * 256 + lane * 4) = acc[g];
  }
  __syncthreads();
  if (kh != 0) return;
  for (int k = 0; k < KS - 1; ++k)
#pragma unroll
    for (int g = 0; g < TG; ++g) acc[g] += *reinterpret_cast<const accv*>(part + (k * TG + g) * 256 + lane * 4);

#pragma unroll
  for (int g = 0; g < TG; ++g) {
    const int tk = tok + 16 * g;
    if (tk >= M) continue;
    float y[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      y[r] = __fmul_rn(__fmul_rn((float)acc[g][r], sxv[g]), swv[r]);
      if (p.bias) y[r] = __fadd_rn(y[r], bv[r]);
      if constexpr (RES) y[r] = p.y_dtype == AQ_BF16 ? add_residual_bf16(y[r], rv[g][r]) : __fadd_rn(y[r], __uint_as_float(rv[g][r]));
    }
    const int64_t o = (int64_t)tk * N + rbase;
    if (p.y_dtype == AQ_BF16) {
      uint16_t* dst = reinterpret_cast<uint16_t*>(p.y) + o;
      if ((N & 3) == 0 && rbase + 3 < N) {
        uint2 pk;
        pk.x = pack_bf16x2(y[0], y[1]);
        pk.y = pack_bf16x2(y[2], y[3]);
        *reinterpret_cast<uint2*>(dst) = pk;
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (rbase + r < N) dst[r] = (uint16_t)f32_to_bf16_bits(y[r]);
      }
    } else {
      float* dst = reinterpret_cast<float*>(p.y) + o;
      if ((N & 3) == 0 && rbase + 3 < N) {
        *reinterpret_cast<float4*>(dst) = make_float4(y[0], y[1], y[2], y[3]);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (rbase + r < N) dst[r] = y[r];
      }
    }
  }
}

// Shapes the token-group kernel takes: 17..32 rows of whole 128-byte lines, and the decode batch sizes whose rows
// are too long for the GEMV kernels' own LDS budget (9..16 rows beyond 10 096 bytes, 5..8 beyond 20 208, ...),
// where the tiles were the only path (12 x 4096 x 11008: 41 us against 19 us).  int8 and FP8 codes alike.
bool gemv_tokens_ok(int64_t M, int64_t N, int64_t K) {
  if (M < 1 || M > 32 || N <= 0 || (K % 128) != 0 || K > (1 << 22)) return false;
  if (M <= 16) {
    const int64_t mt = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16;
    return mt * K + 64 + 2048 > GV_MAX_LDS;  // the GEMV kernels' own limit (gemv_check)
  }
  return true;
}

template <int KS, int GRP>
static int launch_gemv_tokens_shape(const GemvArgs& a, hipStream_t st, bool fp8) {
  constexpr int TG = 2;
  const unsigned grid = (unsigned)((a.N + GRP * GM_ROWS - 1) / (GRP * GM_ROWS));
  const size_t lds = (size_t)16 * TG * (1024 * KS + 16) + 16;
  using kern_t = void (*)(GemvArgs);
  const kern_t fn = fp8 ? (a.res ? gemv_mfma_tokens_kernel<TG, KS, true, GRP, true> : gemv_mfma_tokens_kernel<TG, KS, false, GRP, true>)
                        : (a.res ? gemv_mfma_tokens_kernel<TG, KS, true, GRP> : gemv_mfma_tokens_kernel<TG, KS, false, GRP>);
  static LdsOptIn opted[4];
  const int e = opted[(fp8 ? 2 : 0) + (a.res ? 1 : 0)].ensure(reinterpret_cast<const void*>(fn));
  if (e) return e;
  hipLaunchKernelGGL(fn, dim3(grid), dim3(KS * GRP * 64), lds, st, a);
  return (int)hipGetLastError();
}

// Chunk and workgroup shapes, from timings of 17..32 rows over N = 256..16384, K = 512..4096:
//   * chunks no longer than the rows, or wavefronts idle: 1024 bytes up to K = 1024, else 2048; 4096 over 8
//     wavefronts for K >= 4096 while every compute unit gets at most one workgroup (32 x 6144 x 4096: 7.5 us
//     against 8.5 us), on 16 rows per workgroup while that still gives no compute unit a second one (32 x 2048 x
//     5632: 9.5 us against 11.1 us; x 11008: 13.4 us against 16.6 us);
//   * 32 rows per workgroup while there are no more 32-row blocks than compute units (32 x 8192 x 2048: 5.2 us, 64
//     rows 6.8 us), 64 rows beyond (32 x 16384 x 2048: 7.0 us against 7.4 us: half the copies of the token codes).
// (gemv_tokens_ok and gemv_tokens_launch are not static: the tiled GEMM's entry points in gemm_mfma.hip hand these
// shapes over)
int launch_gemv_tokens(const GemvArgs& a, hipStream_t st, bool fp8) {
  const bool wide = (a.N + 31) / 32 > device_cus();
  if (a.K <= 1024) return wide ? launch_gemv_tokens_shape<1, 4>(a, st, fp8) : launch_gemv_tokens_shape<1, 2>(a, st, fp8);
  if (wide) return launch_gemv_tokens_shape<2, 4>(a, st, fp8);
  if (a.K >= 4096) return (a.N + 15) / 16 <= device_cus() ? launch_gemv_tokens_shape<4, 1>(a, st, fp8) : launch_gemv_tokens_shape<4, 2>(a, st, fp8);
  return launch_gemv_tokens_shape<2, 2>(a, st, fp8);
}

int gemv_tokens_launch(const int8_t* xq, const float* sx, const int8_t* wq, const float* sw, const void* bias,
                       int bias_dtype, const void* residual, void* y, int y_dtype, int64_t M, int64_t N, int64_t K,
                       hipStream_t st, bool fp8) {
  GemvArgs a{};
  a.xq = xq;
  a.sx = sx;
  a.wq = wq;
  a.sw = sw;
  a.bias = bias;
  a.res = residual;
  a.ldr = N;
  a.y = y;
  a.M = (int)M;
  a.N = (int)N;
  a.K = (int)K;
  a.bias_dtype = bias_dtype;
  a.y_dtype = y_dtype;
  return launch_gemv_tokens(a, st, fp8);
}

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace aq

extern "C" size_t aq_gemv_w8a8_workspace_bytes(int64_t M, int64_t K) {
  if (M < 0 || K < 0) return 0;
  return aq::align256((size_t)(M * K)) + aq::align256((size_t)M * sizeof(float));
}

// *mt_out: the token-count bucket of the GEMV kernels, or -1 when the activation codes of that bucket do
// not fit the LDS of a compute unit (rows longer than 10 096 bytes at 9..16 tokens, 20 208 at 5..8, ...):
// such a call is served by the tiled MFMA GEMM, which takes any M (same integer sums, same epilogue: same bits).
static int gemv_check(const int8_t* wq, const float* sw, const void* bias, int bias_dtype, const void* residual,
                      const void* y, int y_dtype, int64_t M, int64_t N, int64_t K, int* mt_out) {
  if (y_dtype != AQ_F32 && y_dtype != AQ_BF16) return AQ_E_DTYPE;
  if (bias && bias_dtype != AQ_F32 && bias_dtype != AQ_BF16) return AQ_E_DTYPE;
  if (M < 0 || M > 16 || N < 0 || K <= 0 || (K % 16) != 0) return AQ_E_SHAPE;
  if (M == 0 || N == 0) return AQ_OK;
  if (!wq || !sw || !y) return AQ_E_NULL;
  // matrices on 16 bytes (vector loads and stores), scale and bias vectors on their element size
  if (aq::check_ptr16(wq) || aq::check_ptr16(y) || aq::check_ptr16(residual)) return AQ_E_ALIGN;
  if (aq::check_ptr(sw, 4) || aq::check_ptr(bias, bias_dtype == AQ_BF16 ? 2 : 4)) return AQ_E_ALIGN;
  if (N > (1 << 25) || K > (1 << 22)) return AQ_E_RANGE;  // 16 rows of N outputs are indexed in 32 bits
  const int mt = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16;
  *mt_out = (int64_t)mt * K + 64 + 2048 > aq::GV_MAX_LDS ? -1 : mt;  // codes, scales, K-part sums
  return AQ_OK;
}

static int gemv_dispatch(const aq::GemvArgs& a, int mt, hipStream_t st) {
  // 9..16 rows go to the matrix-core variant, except on a short matrix with long rows (an MLP's down projection):
  // its 16-row wavefronts make N / 16 workgroups, half the device or less, where the dot-product kernel's 4-row
  // wavefronts still reach every compute unit (N = 2048, K = 5632: 7.6-8.0 against 8.5 us; N = 1536, K = 6912:
  // 11.0 against 12.9 us; at K = 2048 or from N = 3072 on the matrix core wins, 4.7 against 5.6 us).
  const bool short_long = (a.N + 15) / 16 * 2 <= aq::device_cus() && a.K >= 4096;
  if (aq::gemv_mfma_ok(a.M, a.K) && !short_long) return aq::launch_gemv_mfma(a, st);
  switch (mt) {
    case 1: return aq::launch_gemv<1, false, 4>(a, st);
    case 2: return aq::launch_gemv<2, false, 4>(a, st);
    case 4: return aq::launch_gemv<4, false, 4>(a, st);
    case 8: return aq::launch_gemv<8, false, 4>(a, st);
    default: return aq::launch_gemv<16, false, 4>(a, st);
  }
}

// One launch for up to 8 bf16 rows that fit the in-kernel quantiser's register
// budget; returns -1 when the shape has to take the two-launch path.  With more
// than 8 rows every workgroup would repeat 2+ row quantisations per wavefront
// on its critical path, which measures no faster than the separate launch.
static int gemv_dispatch_fused(const aq::GemvArgs& a, int mt, hipStream_t st) {
  if (aq::gemv_mfma_fq_ok(a.M, a.N, a.K, a.gamma != nullptr)) return aq::launch_gemv_mfma_fq(a, st);
  const int64_t vpl = (a.K / 8 + 63) / 64;  // 16-byte vectors per lane per bf16 row
  if (mt > 8 || vpl > 16) return -1;
  // A short matrix with long rows (an MLP's down projection): with whole rows per wavefront its N / 32 workgroups
  // would leave most compute units without loads in flight (N = 2048, K = 5632, 8 rows: 11.0 us against 9.1 for
  // the separate row quantiser + the K-split GEMV on codes).  The fused kernel with 4 K parts -- 8 weight rows per
  // workgroup, every wavefront rounding one token row first -- is the fastest form: 8.6 -> 7.15 us for that shape,
  // 8.0 -> 5.7 us for 4 rows of 6912 against 1536 weight rows, 7.0 -> 4.8 us for one row of 5632 (2 parts: 8.0,
  // 8 parts: 12.1 us).  With the norm in front (rows stay short there) the two launches remain.
  if ((a.N + 31) / 32 * 4 <= aq::device_cus() && (a.K > 4096 || (a.M > 4 && a.K >= 4096))) {
    if (a.gamma) return -1;
    switch (mt) {
      case 1: return aq::launch_gemv_fw<1, true, 16, false, 0, aq::GV_WAVES, 4>(a, st);
      case 2: return aq::launch_gemv_fw<2, true, 16, false, 0, aq::GV_WAVES, 4>(a, st);
      case 4: return aq::launch_gemv_fw<4, true, 16, false, 0, aq::GV_WAVES, 4>(a, st);
      default: return aq::launch_gemv_fw<8, true, 16, false, 0, aq::GV_WAVES, 4>(a, st);
    }
  }
  const bool small = vpl <= 4;
  if (a.gamma) {  // with the norm in front: short rows only (the gain's vectors stay in registers too)
    if (!small) return -1;
    switch (mt) {
      case 1: return aq::launch_gemv<1, true, 4, true>(a, st);
      case 2: return aq::launch_gemv<2, true, 4, true>(a, st);
      case 4: return aq::launch_gemv<4, true, 4, true>(a, st);
      default: return aq::launch_gemv<8, true, 4, true>(a, st);
    }
  }
  switch (mt) {
    case 1: return small ? aq::launch_gemv<1, true, 4>(a, st) : aq::launch_gemv<1, true, 16>(a, st);
    case 2: return small ? aq::launch_gemv<2, true, 4>(a, st) : aq::launch_gemv<2, true, 16>(a, st);
    case 4: return small ? aq::launch_gemv<4, true, 4>(a, st) : aq::launch_gemv<4, true, 16>(a, st);
    default: return small ? aq::launch_gemv<8, true, 4>(a, st) : aq::launch_gemv<8, true, 16>(a, st);
  }
}

extern "C" int aq_gemv_w8a8_codes_residual(const int8_t* xq, const float* sx, const int8_t* wq, const float* sw,
                                           const void* bias, int bias_dtype, const void* residual,
                                           void* y, int y_dtype, int64_t M, int64_t N, int64_t K, void* stream) {
  int mt = 0;
  int rc = gemv_check(wq, sw, bias, bias_dtype, residual, y, y_dtype, M, N, K, &mt);
  if (rc || M == 0 || N == 0) return rc;
  if (!xq || !sx) return AQ_E_NULL;
  if (aq::check_ptr16(xq) || aq::check_ptr(sx, 4)) return AQ_E_ALIGN;
  if (mt < 0) return aq_linear_w8a8_residual(xq, sx, wq, sw, bias, bias_dtype, residual, y, y_dtype, M, N, K, stream);
  aq::GemvArgs a{};
  a.xq = xq;
  a.sx = sx;
  a.wq = wq;
  a.sw = sw;
  a.bias = bias;
  a.res = residual;
  a.ldr = N;
  a.y = y;
  a.M = (int)M;
  a.N = (int)N;
  a.K = (int)K;
  a.bias_dtype = bias_dtype;
  a.y_dtype = y_dtype;
  return gemv_dispatch(a, mt, static_cast<hipStream_t>(stream));
}

extern "C" int aq_gemv_w8a8_codes(const int8_t* xq, const float* sx, const int8_t* wq, const float* sw,
                                  const void* bias, int bias_dtype, void* y, int y_dtype, int64_t M,
                                  int64_t N, int64_t K, void* stream) {
  return aq_gemv_w8a8_codes_residual(xq, sx, wq, sw, bias, bias_dtype, nullptr, y, y_dtype, M, N, K, stream);
}

extern "C" int aq_gemv_w8a8_decode_residual(const void* x, int x_dtype, const int8_t* wq, const float* sw,
                                            const void* bias, int bias_dtype, const void* residual,
                                            void* y, int y_dtype, int64_t M, int64_t N, int64_t K, void* ws,
                                            size_t ws_bytes, void* stream) {
  if (x_dtype != AQ_F32 && x_dtype != AQ_BF16) return AQ_E_DTYPE;
  int mt = 0;
  int rc = gemv_check(wq, sw, bias, bias_dtype, residual, y, y_dtype, M, N, K, &mt);
  if (rc || M == 0 || N == 0) return rc;
  if (!x || !ws) return AQ_E_NULL;
  if (aq::check_ptr16(x) || aq::check_ptr16(ws)) return AQ_E_ALIGN;
  if (ws_bytes < aq_gemv_w8a8_workspace_bytes(M, K)) return AQ_E_WORKSPACE;
  if (x_dtype == AQ_BF16 && mt > 0) {  // one launch: the GEMV kernel quantises the rows itself
    aq::GemvArgs a{};
    a.x = x;
    a.wq = wq;
    a.sw = sw;
    a.bias = bias;
    a.res = residual;
    a.ldr = N;
    a.y = y;
    a.M = (int)M;
    a.N = (int)N;
    a.K = (int)K;
    a.bias_dtype = bias_dtype;
    a.y_dtype = y_dtype;
    const int frc = gemv_dispatch_fused(a, mt, static_cast<hipStream_t>(stream));
    if (frc >= 0) return frc;
  }
  int8_t* xq = static_cast<int8_t*>(ws);
  float* sx = reinterpret_cast<float*>(static_cast<char*>(ws) + aq::align256((size_t)(M * K)));
  rc = aq_quant_rowwise_i8(x, x_dtype, M, K, K, xq, sx, stream);
  if (rc) return rc;
  return aq_gemv_w8a8_codes_residual(xq, sx, wq, sw, bias, bias_dtype, residual, y, y_dtype, M, N, K, stream);
}

// ---------------------------------------------------------------------------
// FP8 decode: the same streaming GEMV on e4m3 codes with per-tensor scales.  Shapes the kernel does not take
// (K not in whole 256-byte steps, rows too long for the LDS) go to the tiled FP8 GEMM, which takes any M.
extern "C" size_t aq_gemv_fp8_workspace_bytes(int64_t M, int64_t K) {
  if (M < 0 || K < 0) return 0;
  return aq::align256((size_t)(M * K)) + 256 + AQ_FP8_AMAX_WS_BYTES;  // codes, the scale, the quantiser's partial maxima
}

static int gemv_fp8_check(const uint8_t* wq, const float* sw, const void* bias, int bias_dtype, const void* residual,
                          const void* y, int y_dtype, int64_t M, int64_t N, int64_t K) {
  if (y_dtype != AQ_F32 && y_dtype != AQ_BF16) return AQ_E_DTYPE;
  if (bias && bias_dtype != AQ_F32 && bias_dtype != AQ_BF16) return AQ_E_DTYPE;
  if (M < 0 || M > 16 || N < 0 || K <= 0 || (K % 16) != 0) return AQ_E_SHAPE;
  if (M == 0 || N == 0) return AQ_OK;
  if (!wq || !sw || !y) return AQ_E_NULL;
  if (aq::check_ptr16(wq) || aq::check_ptr16(y) || aq::check_ptr16(residual)) return AQ_E_ALIGN;
  if (aq::check_ptr(sw, 4) || aq::check_ptr(bias, bias_dtype == AQ_BF16 ? 2 : 4)) return AQ_E_ALIGN;
  if (N > (1 << 25) || K > (1 << 22)) return AQ_E_RANGE;
  return AQ_OK;
}

static aq::GemvArgs gemv_fp8_args(const uint8_t* wq, const float* sw, const void* bias, int bias_dtype,
                                  const void* residual, void* y, int y_dtype, int64_t M, int64_t N, int64_t K) {
  aq::GemvArgs a{};
  a.wq = reinterpret_cast<const int8_t*>(wq);
  a.sw = sw;
  a.bias = bias;
  a.res = residual;
  a.ldr = N;
  a.y = y;
  a.M = (int)M;
  a.N = (int)N;
  a.K = (int)K;
  a.bias_dtype = bias_dtype;
  a.y_dtype = y_dtype;
  return a;
}

static bool gemv_fp8_ok(int64_t K) { return (K % 256) == 0 && 16 * (K + 16) + 64 + 16 <= aq::GV_MAX_LDS; }

extern "C" int aq_gemv_fp8_codes_residual(const uint8_t* xq, const float* sx, const uint8_t* wq, const float* sw,
                                          const void* bias, int bias_dtype, const void* residual, void* y, int y_dtype,
                                          int64_t M, int64_t N, int64_t K, void* stream) {
  int rc = gemv_fp8_check(wq, sw, bias, bias_dtype, residual, y, y_dtype, M, N, K);
  if (rc || M == 0 || N == 0) return rc;
  if (!xq || !sx) return AQ_E_NULL;
  if (aq::check_ptr16(xq) || aq::check_ptr(sx, 4)) return AQ_E_ALIGN;
  if (!gemv_fp8_ok(K)) return aq_linear_fp8_residual(xq, sx, wq, sw, bias, bias_dtype, residual, y, y_dtype, M, N, K, stream);
  aq::GemvArgs a = gemv_fp8_args(wq, sw, bias, bias_dtype, residual, y, y_dtype, M, N, K);
  a.xq = reinterpret_cast<const int8_t*>(xq);
  a.sx = sx;
  return aq::launch_gemv_mfma(a, static_cast<hipStream_t>(stream), true);
}

extern "C" int aq_gemv_fp8_decode_residual(const void* x, int x_dtype, const uint8_t* wq, const float* sw,
                                           const void* bias, int bias_dtype, const void* residual, void* y, int y_dtype,
                                           int64_t M, int64_t N, int64_t K, void* ws, size_t ws_bytes, void* stream) {
  if (x_dtype != AQ_F32 && x_dtype != AQ_BF16) return AQ_E_DTYPE;
  int rc = gemv_fp8_check(wq, sw, bias, bias_dtype, residual, y, y_dtype, M, N, K);
  if (rc || M == 0 || N == 0) return rc;
  if (!x || !ws) return AQ_E_NULL;
  if (aq::check_ptr16(x) || aq::check_ptr16(ws)) return AQ_E_ALIGN;
  if (ws_bytes < aq_gemv_fp8_workspace_bytes(M, K)) return AQ_E_WORKSPACE;
  if (x_dtype == AQ_BF16 && K <= 2048 && (K % 512) == 0) {  // one launch: the kernel casts the rows itself
    aq::GemvArgs a = gemv_fp8_args(wq, sw, bias, bias_dtype, residual, y, y_dtype, M, N, K);
    a.x = x;
    return aq::launch_gemv_mfma_fq(a, static_cast<hipStream_t>(stream), true);
  }
  uint8_t* xq = static_cast<uint8_t*>(ws);
  float* sx = reinterpret_cast<float*>(static_cast<char*>(ws) + aq::align256((size_t)(M * K)));
  uint32_t* amax_ws = reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(sx) + 256);
  rc = aq_quant_tensor_fp8(x, x_dtype, M * K, xq, sx, amax_ws, AQ_FP8_AMAX_WS_BYTES, stream);
  if (rc) return rc;
  return aq_gemv_fp8_codes_residual(xq, sx, wq, sw, bias, bias_dtype, residual, y, y_dtype, M, N, K, stream);
}

// ---------------------------------------------------------------------------
// The decode entry point for callers that cannot allocate (code under HIP graph capture, serving loops and
// harnesses that forbid hipMalloc): the workspace of aq_gemv_w8a8_decode_residual -- the activation codes and
// scales that the row quantiser hands to the GEMV when the rows are not quantised inside the GEMV kernel --
// lives in device memory that the library itself owns, one copy per GPU, for the life of the process.
namespace aq {

constexpr size_t NOALLOC_SCRATCH_BYTES = AQ_GEMV_NOALLOC_MAX_MK + 256;  // codes [M, K] then scales [M]
static_assert(AQ_GEMV_NOALLOC_MAX_MK % 256 == 0, "the scales start 256-byte aligned");
static __device__ __align__(256) uint8_t scratch[NOALLOC_SCRATCH_BYTES];

// In host code `scratch` is only a handle: the array's device address is asked of the runtime, once per
// device (each GPU holds its own copy at its own address) with that device current, and kept.  Two threads
// that come first at the same time both store the same address.
static int scratch_of_current_device(void** out) {
  static void* ptrs[64] = {};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= 64) return AQ_E_RANGE;
  void* p = __atomic_load_n(&ptrs[dev], __ATOMIC_ACQUIRE);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!p) return AQ_E_NULL;
    __atomic_store_n(&ptrs[dev], p, __ATOMIC_RELEASE);
  }
  *out = p;
  return AQ_OK;
}

}  // namespace aq

extern "C" int aq_gemv_w8a8_decode_noalloc(const void* x, int x_dtype, const int8_t* wq, const float* sw,
                                           const void* bias, int bias_dtype, const void* residual, void* y,
                                           int y_dtype, int64_t M, int64_t N, int64_t K, void* stream) {
  // sizes beyond the scratch are rejected before anything else is looked at: AQ_E_RANGE, "size beyond ..."
  if (M > 0 && K > 0 && (M > 16 || M * K > (int64_t)AQ_GEMV_NOALLOC_MAX_MK)) return M > 16 ? AQ_E_SHAPE : AQ_E_RANGE;
  void* ws = nullptr;
  const int rc = aq::scratch_of_current_device(&ws);
  if (rc) return rc;
  // The scratch keeps the previous call's contents; nothing in it has to start at zero: the quantiser
  // writes all M rows of codes and all M scales before the GEMV reads exactly those.
  return aq_gemv_w8a8_decode_residual(x, x_dtype, wq, sw, bias, bias_dtype, residual, y, y_dtype, M, N, K, ws,
                                      aq::NOALLOC_SCRATCH_BYTES, stream);
}

extern "C" int aq_gemv_w8a8_decode_attn(const float* partials, int64_t n_slices, int64_t head_dim, const int8_t* wq,
                                        const float* sw, const void* bias, int bias_dtype, const void* residual,
                                        void* y, int y_dtype, int64_t M, int64_t N, int64_t K, void* stream) {
  int mt = 0;
  int rc = gemv_check(wq, sw, bias, bias_dtype, residual, y, y_dtype, M, N, K, &mt);
  if (rc) return rc;
  if ((head_dim != 64 && head_dim != 128) || (K % head_dim) != 0 || n_slices <= 0) return AQ_E_SHAPE;
  // the in-kernel merge keeps every slice of a lane's vectors in registers
  if (M > 8 || K > AQ_GEMV_ATTN_MAX_K || n_slices > AQ_GEMV_ATTN_MAX_SLICES) return AQ_E_RANGE;
  if (M == 0 || N == 0) return AQ_OK;
  if (!partials) return AQ_E_NULL;
  if (aq::check_ptr16(partials)) return AQ_E_ALIGN;
  aq::GemvArgs a{};
  a.parts = partials;
  a.parts_ns = (int)n_slices;
  a.parts_d = (int)head_dim;
  a.wq = wq;
  a.sw = sw;
  a.bias = bias;
  a.res = residual;
  a.ldr = N;
  a.y = y;
  a.M = (int)M;
  a.N = (int)N;
  a.K = (int)K;
  a.bias_dtype = bias_dtype;
  a.y_dtype = y_dtype;
  hipStream_t st = static_cast<hipStream_t>(stream);
  constexpr int NS = AQ_GEMV_ATTN_MAX_SLICES;
  switch (mt) {
    case 1: return aq::launch_gemv<1, true, 4, false, NS>(a, st);
    case 2: return aq::launch_gemv<2, true, 4, false, NS>(a, st);
    case 4: return aq::launch_gemv<4, true, 4, false, NS>(a, st);
    default: return aq::launch_gemv<8, true, 4, false, NS>(a, st);
  }
}

extern "C" int aq_gemv_w8a8_decode_rmsnorm(const void* x, int x_dtype, const void* gamma, float eps, const int8_t* wq,
                                           const float* sw, const void* bias, int bias_dtype, const void* residual,
                                           void* y, int y_dtype, int64_t M, int64_t N, int64_t K, void* ws,
                                           size_t ws_bytes, void* stream) {
  if (x_dtype != AQ_F32 && x_dtype != AQ_BF16) return AQ_E_DTYPE;
  int mt = 0;
  int rc = gemv_check(wq, sw, bias, bias_dtype, residual, y, y_dtype, M, N, K, &mt);
  if (rc || M == 0 || N == 0) return rc;
  if (!x || !gamma || !ws) return AQ_E_NULL;
  if (aq::check_ptr16(x) || aq::check_ptr16(gamma) || aq::check_ptr16(ws)) return AQ_E_ALIGN;
  if (ws_bytes < aq_gemv_w8a8_workspace_bytes(M, K)) return AQ_E_WORKSPACE;
  if (x_dtype == AQ_BF16 && mt > 0) {  // one launch: the GEMV kernel normalises and quantises the rows itself
    aq::GemvArgs a{};
    a.x = x;
    a.gamma = gamma;
    a.eps = eps;
    a.wq = wq;
    a.sw = sw;
    a.bias = bias;
    a.res = residual;
    a.ldr = N;
    a.y = y;
    a.M = (int)M;
    a.N = (int)N;
    a.K = (int)K;
    a.bias_dtype = bias_dtype;
    a.y_dtype = y_dtype;
    const int frc = gemv_dispatch_fused(a, mt, static_cast<hipStream_t>(stream));
    if (frc >= 0) return frc;
  }
  int8_t* xq = static_cast<int8_t*>(ws);
  float* sx = reinterpret_cast<float*>(static_cast<char*>(ws) + aq::align256((size_t)(M * K)));
  rc = aq_rmsnorm_quant_rowwise_i8(x, x_dtype, gamma, x_dtype, eps, M, K, K, xq, sx, stream);
  if (rc) return rc;
  return aq_gemv_w8a8_codes_residual(xq, sx, wq, sw, bias, bias_dtype, residual, y, y_dtype, M, N, K, stream);
}

extern "C" int aq_gemv_w8a8_decode_swiglu_ok(int x_dtype, int64_t M, int64_t F, int64_t K) {
  return x_dtype == AQ_BF16 && aq::gemv_mfma_swiglu_ok(M, F, K) ? 1 : 0;
}

extern "C" int aq_gemv_w8a8_decode_swiglu(const void* x, int x_dtype, const void* gamma, float eps, const int8_t* wq,
                                          const float* sw, const void* bias, int bias_dtype, void* h, int h_dtype,
                                          int64_t M, int64_t F, int64_t K, void* stream) {
  if (x_dtype != AQ_F32 && x_dtype != AQ_BF16) return AQ_E_DTYPE;
  if (F < 0 || F > (1 << 24)) return F < 0 ? AQ_E_SHAPE : AQ_E_RANGE;
  int mt = 0;
  int rc = gemv_check(wq, sw, bias, bias_dtype, nullptr, h, h_dtype, M, 2 * F, K, &mt);
  if (rc || M == 0 || F == 0) return rc;
  if (!x) return AQ_E_NULL;
  if (aq::check_ptr16(x) || aq::check_ptr16(gamma)) return AQ_E_ALIGN;
  if (!aq_gemv_w8a8_decode_swiglu_ok(x_dtype, M, F, K)) return AQ_E_RANGE;  // the caller takes the separate launches
  aq::GemvArgs a{};
  a.x = x;
  a.gamma = gamma;
  a.eps = eps;
  a.wq = wq;
  a.sw = sw;
  a.bias = bias;
  a.y = h;
  a.M = (int)M;
  a.N = (int)(2 * F);
  a.K = (int)K;
  a.bias_dtype = bias_dtype;
  a.y_dtype = h_dtype;
  return aq::launch_gemv_mfma_swiglu(a, static_cast<hipStream_t>(stream));
}

extern "C" int aq_gemv_w8a8_decode(const void* x, int x_dtype, const int8_t* wq, const float* sw,
                                   const void* bias, int bias_dtype, void* y, int y_dtype, int64_t M,
                                   int64_t N, int64_t K, void* ws, size_t ws_bytes, void* stream) {
  return aq_gemv_w8a8_decode_residual(x, x_dtype, wq, sw, bias, bias_dtype, nullptr, y, y_dtype, M, N, K, ws, ws_bytes,
                                      stream);
}

#ifdef AQ_LAB
// Lab build only (see aq_lab.h): the buffer the matrix-core GEMV's wavefronts leave their time stamps in.
extern "C" int aq_lab_set_gemv_timeline(long long* buf) {
  return (int)hipMemcpyToSymbol(HIP_SYMBOL(aq::gv_timeline), &buf, sizeof(buf));
}
extern "C" int aq_lab_set_gemv_skip_weights(int on) {
  return (int)hipMemcpyToSymbol(HIP_SYMBOL(aq::gv_skip_weights), &on, sizeof(on));
}
#endif
