// Prefill GEMMs on the CDNA4 matrix cores: int8 x int8 -> int32
// (v_mfma_i32_32x32x32_i8) and FP8 e4m3 x e4m3 -> fp32
// (v_mfma_scale_f32_32x32x64_f8f6f4 with unit scales), one kernel template.
//
//   C[m, n] = sum_k A[m, k] * B[n, k]     A = activation codes [M, K]
//                                         B = weight codes     [N, K]
// Both operands are K-contiguous, which is exactly the MFMA operand order
// (each lane feeds 16 or 32 consecutive k of one row), so no transpose is ever
// materialised.  A workgroup of 8 wavefronts (two per SIMD) owns a 256 x 128
// tile of C; each wavefront a 64 x 64 sub-tile held as 2 x 2 MFMA 32x32
// accumulators.  (When that gives too few tiles to occupy the device, the
// tile is 128 x 128, 128 x 64, 128 x 32, 64 x 64 or 64 x 32 instead, on four or
// two wavefronts.)  K is walked in 128-byte steps through three to six LDS
// stages that are filled by direct global->LDS loads (no register staging), with an XOR
// permutation of 16-byte pieces that makes the fragment reads bank-conflict
// free; the loop is software-pipelined so that LDS reads and global loads of
// later sub-steps are issued between the MFMAs of the current one, with one
// workgroup barrier per K step.  The epilogue is fused and runs straight from
// the accumulator registers: int32 store, or dequantise (+bias) and cast.
#include <type_traits>

#include "aq_common.h"

namespace aq {

// Shape of a workgroup: WM x WN x WK wavefronts, each accumulating a (32 TM) x (32 TN) sub-tile
// (TM x TN MFMA 32x32 accumulators); K walked in BK-byte steps through NSTAGE LDS stages.
//   <4, 2, 2, 2, 1, 128, 3>  256 x 128 tile, 8 wavefronts (two per SIMD) of 64 x 64, 3 stages of 48 KiB;
//   <2, 2, 2, 2, 1, 128, 3>  128 x 128 tile, 4 wavefronts (one per SIMD) of 64 x 64, 3 stages of 32 KiB (4 fit
//                            and were 1-5 % slower on this tile's shapes);
//   <2, 2, 2, 1, 1, 128, 4>  128 x 64 tile, 4 wavefronts of 64 x 32,
//   <4, 1, 1, 1, 1, 128, 4>  128 x 32 tile, 4 wavefronts of 32 x 32,
//   <2, 2, 1, 1, 1, 128, 4>  64 x 64 tile, 4 wavefronts of 32 x 32, and
//   <2, 1, 1, 1, 1, 128, 6>  64 x 32 tile, 2 wavefronts of 32 x 32 (six stages of 12 KiB: 2-20 % faster than four,
//                            while the other three were fastest with four of the 3..8 that fit, three costing
//                            them 5-25 %: their K loop runs at the latency of its loads): for a few
//                            hundred rows, where wider tiles leave most compute units without one.  A
//                            workgroup's time is the matrix-core time of its whole tile, rows past M included
//                            (128 x 128 x 2048: 16 K steps of 16 MFMAs, 3.9 us per compute unit), so with tiles
//                            to spare the smaller tile is the faster launch (128 x 2048 x 2048, weights from
//                            HBM: 12.4 us on 16 tiles of 128 x 128, 8.7 us on 64 of 128 x 32, 6.9 us on 128 of
//                            64 x 32);
// The same five tiles on twice the wavefronts, the two that share a sub-tile each taking half of every K step
// and exchanging half of their accumulators through LDS at the end (WK = 2, so that each finishes and stores
// half of the sub-tile), were measured against these in one process over 48..512 rows and four weight shapes:
// 2-6 % slower every time (128 x 128 at 512 x 8192 x 2048: 15.0 against 14.1 us; 64 x 64 at 128 x 8192 x 2048:
// 8.8 against 8.4 us).  The lab build keeps the 128 x 128 one (<2, 2, 2, 2, 2, 128, 3>) so that the K-split
// code stays compiled and tested.
// Shapes that (but for the first one on FP8) only the lab build instantiates.  Measured, none faster on int8 with
// real operand data: under a matrix-core load with toggling operands this part runs against its power limit, and
// fewer LDS reads per MFMA buy clock, not rate (8192^3: 2.31-2.42 POP/s for every shape below and for the
// 256 x 128 tile alike, while the clock moves between 1.47 and 1.65 GHz).  FP8, which is throttled less, gains 5 %
// from the first one at 8192^3 (417 against 438 us: its K loop runs at 84 % of the matrix cores' own time with 6 %
// of it waited at the stage barriers, where the 256 x 128 tile waits 40 %; a 64 x 64 sub-tile reads 32 bytes of
// fragments per wavefront and cycle, 128 per compute unit, which is all the LDS delivers, before the fills'
// writes; the 128 x 128 sub-tile needs half); the product takes it for FP8 launches of at least two rounds of
// 256 x 256 tiles.
//   <2, 2, 4, 4, 1, 64, 4>   256 x 256 tile, 4 wavefronts (one per SIMD) of 128 x 128: 256 accumulator
//                            registers per lane (the AGPR half of the register file), 8 fragment reads per
//                            16 MFMAs instead of 16, half the LDS fill per MFMA; 4 stages of 32 KiB; whole K
//                            steps, whole 256-row multiples, even N, no residual (one K-loop and one epilogue
//                            variant: with all three epilogues and both K loops the kernel was 45 000 lines of
//                            machine code whose spilled values came back from scratch one memory round trip at a
//                            time, 45 k cycles of epilogue per tile; now 12-16 k);
//   <4, 2, 2, 4, 1, 64, 4>   256 x 256 tile, 8 wavefronts of 64 x 128: 6 fragment reads per 8 MFMAs;
//   <2, 2, 4, 2, 1, 128, 3>  256 x 128 tile, 4 wavefronts of 128 x 64.
// Two independent 4-wavefront workgroups per compute unit (256 x 128 or 128 x 128 tiles with 64-byte stages, so
// that one's epilogue overlaps the other's loop) were measured too: 8192^3 in 459 and 556 us against 310 us with
// all-zero operands.
template <int WM_, int WN_, int TM_, int TN_, int WK_, int BK_, int NSTAGE_>
struct Shape {
  static constexpr int WM = WM_, WN = WN_, TM = TM_, TN = TN_, WK = WK_, BK = BK_, NSTAGE = NSTAGE_;
  static constexpr int NWAVES = WM * WN * WK, NTHREADS = NWAVES * 64;
  static constexpr int WAVE_M = 32 * TM, WAVE_N = 32 * TN;
  static constexpr int BM = WM * WAVE_M, BN = WN * WAVE_N;
  static constexpr int STAGE = (BM + BN) * BK;
  // Sub-tiles of 16 accumulators (128 x 128 per wavefront): the 256 accumulator registers leave no room to hold a
  // lane's 64 per-row scales through the K loop, so the tile's BM scales wait in LDS behind the stages instead;
  // such shapes also compile one K-loop variant (whole K steps) and one epilogue variant only (see gemm_kernel).
  static constexpr bool BIG = TM * TN >= 16;
  static constexpr int SX_BYTES = BIG ? BM * 4 : 0;
  static constexpr int LDS_BYTES = NSTAGE * STAGE + SX_BYTES;
  static_assert(BK == 64 || BK == 128, "K bytes per stage");
  static_assert(NWAVES % 2 == 0, "the piece permutation assumes a wavefront's row groups share parity");
  static_assert((BM * BK / 1024) % NWAVES == 0 && (BN * BK / 1024) % NWAVES == 0, "whole 1 KiB loads per wavefront");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS of one compute unit");
  static_assert((NSTAGE - 1) * ((BM + BN) * BK / 16 / NTHREADS) <= 63, "the loads in flight fit the 6-bit counter");
};
using ShapeLarge = Shape<4, 2, 2, 2, 1, 128, 3>;
using ShapeSmall = Shape<2, 2, 2, 2, 1, 128, 3>;
using ShapeN64 = Shape<2, 2, 2, 1, 1, 128, 4>;
using ShapeN32 = Shape<4, 1, 1, 1, 1, 128, 4>;
using ShapeM64N64 = Shape<2, 2, 1, 1, 1, 128, 4>;
using ShapeM64N32 = Shape<2, 1, 1, 1, 1, 128, 6>;
using ShapeHuge = Shape<2, 2, 4, 4, 1, 64, 4>;  // product: FP8 launches of two rounds or more (see huge_fp8_ok)
#ifdef AQ_LAB
using ShapeTall = Shape<2, 2, 4, 2, 1, 128, 3>;
using ShapeHuge8 = Shape<4, 2, 2, 4, 1, 64, 4>;
using ShapePair = Shape<2, 2, 2, 2, 2, 128, 3>;
#endif
constexpr int NUM_XCD = 8;
constexpr int GROUP_M = 4;

enum { OUT_I32 = 0, OUT_F32 = 1, OUT_BF16 = 2 };

struct GemmArgs {
  const uint8_t* A;
  const uint8_t* B;
  void* C;
  int M, N, K;
  int tiles_m, tiles_n;
  const float* sx;   // int8: [M]; fp8: [1]
  const float* sw;   // int8: [N]; fp8: [1]
  const void* bias;  // [N] or null
  int bias_dtype;
  const void* res;   // [M, N] residual in the output's type, or null; may be C itself
};

// Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.
// Re-number them so that one XCD owns a contiguous run of tile ids, and walk
// tile ids in GROUP_M-tall column-major groups, so the tiles resident on an
// XCD at one time share A rows and B rows (4 x 8 tiles = 2 MB + 2 MB of
// operands for the 4096 x 2048 x 2048 case).
__device__ __forceinline__ void tile_of_block(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int nt = tiles_m * tiles_n;
  const int per = nt / NUM_XCD, rem = nt % NUM_XCD;
  const int xcd = pid % NUM_XCD, idx = pid / NUM_XCD;
  const int tile = xcd * per + (xcd < rem ? xcd : rem) + idx;
  const int group_sz = GROUP_M * tiles_n;
  const int group = tile / group_sz;
  const int first_m = group * GROUP_M;
  const int gm = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  const int in_group = tile - group * group_sz;
  tm = first_m + in_group % gm;
  tn = in_group / gm;
}

template <bool FP8>
struct Acc {
  using type = v16i;
};
template <>
struct Acc<true> {
  using type = v16f;
};

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding:
// vmcnt in bits 3:0 and 15:14, expcnt 6:4 and lgkmcnt 11:8 left at their maxima).
#define AQ_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0f70 | ((n) & 15) | (((n) >> 4) << 14))
// Workgroup barrier without the memory fence of __syncthreads(): the fence
// would drain every outstanding global->LDS load, including the ones issued
// two K steps ahead on purpose.  The empty asm statements stop the compiler
// from moving LDS accesses across it.
#define AQ_BARRIER()                   \
  do {                                 \
    asm volatile("" ::: "memory");     \
    __builtin_amdgcn_s_barrier();      \
    asm volatile("" ::: "memory");     \
  } while (0)

typedef __attribute__((address_space(3))) void lds_void;


template <bool FP8>
struct Frag {
  using type = v4i;  // 16 bytes of K per lane: v_mfma_i32_32x32x32_i8
};
template <>
struct Frag<true> {
  using type = v8i;  // 32 bytes of K per lane: v_mfma_scale_f32_32x32x64_f8f6f4
};

#ifndef AQ_FP8_SCALE
#define AQ_FP8_SCALE 0
#endif
template <bool FP8>
__device__ __forceinline__ typename Acc<FP8>::type mma(const typename Frag<FP8>::type& a,
                                                       const typename Frag<FP8>::type& b,
                                                       const typename Acc<FP8>::type& c) {
  if constexpr (!FP8) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
  } else {
    // E8M0 scale 127 = 2^0 for both operands: plain e4m3 x e4m3.
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, AQ_FP8_SCALE, 0, AQ_FP8_SCALE);
  }
}

// Issue order of one pipeline slot, as scheduling groups: GROUPS times
// [1 MFMA, NDS LDS reads, this group's share of the NLD global loads].
// (0x008 = MFMA, 0x100 = LDS read, 0x020 = vector-memory read.)
template <int G, int GROUPS, int NDS, int NLD>
__device__ __forceinline__ void sched_pattern() {
  if constexpr (G < GROUPS) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, NDS, 0);
    constexpr int nl = ((G + 1) * NLD) / GROUPS - (G * NLD) / GROUPS;
    if constexpr (nl > 0) __builtin_amdgcn_sched_group_barrier(0x020, nl, 0);
    sched_pattern<G + 1, GROUPS, NDS, NLD>();
  }
}

#ifdef AQ_LAB
__device__ long long aq_lab_clock[16];
#endif
// EXACT: K is a whole number of BK-byte steps, so every 16-byte piece of every step lies inside its row and the
// global->LDS loads need no per-lane range logic: a loop-invariant lane offset per row group and the K step as a
// scalar offset, no vector ALU work per load.
template <bool FP8, int OUT, class S, bool EXACT>
__device__ __forceinline__ void gemm_tile(const GemmArgs& p, uint8_t* smem, int pid) {
  constexpr int WM = S::WM, WN = S::WN, TM = S::TM, TN = S::TN, WK = S::WK, BK = S::BK, NSTAGE = S::NSTAGE;
  constexpr int NWAVES = S::NWAVES, NTHREADS = S::NTHREADS, WAVE_M = S::WAVE_M, WAVE_N = S::WAVE_N;
  constexpr int BM = S::BM, BN = S::BN, STAGE = S::STAGE;
  constexpr bool BIG = S::BIG;
  static_assert(TM % WK == 0, "the K-split pair divides the sub-tile's row blocks");
  static_assert(!BIG || (EXACT && WK == 1), "big sub-tiles: whole K steps, no K-split pair");
  constexpr int TME = TM / WK;  // row blocks a wavefront finishes and stores
  constexpr int A_LOADS = BM * BK / 16 / NTHREADS;  // 16-byte vectors per thread per K step
  constexpr int B_LOADS = BN * BK / 16 / NTHREADS;
  // NSTAGE stages of [A tile BM x BK bytes][B tile BN x BK bytes], rows unpadded.
  // Global->LDS loads land 64 lanes x 16 B contiguously (1 KiB: RPG = 8 rows of
  // 128 B or 16 rows of 64 B), so the bank-conflict-free layout is obtained by
  // permuting which 16-byte piece of its row each lane fetches: piece c of row r
  // is stored at slot c ^ ((r / RPL) % PPR), with PPR = BK / 16 pieces per row and
  // RPL = 256 / BK rows per bank line.  LDS has 64 banks here (256 bytes per bank
  // line) and a 16-byte-per-lane read is served 16 lanes at a time, so 16
  // consecutive rows reading the same piece must land on 16 distinct slots:
  // r % RPL picks the part of the bank line, the permuted piece the slot in it.
  constexpr int PPR = BK / 16, RPL = 256 / BK, RPG = 1024 / BK;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_k = WK == 1 ? 0 : wave / (WM * WN), wave_mn = WK == 1 ? wave : wave % (WM * WN);
  const int wave_m = wave_mn / WN, wave_n = wave_mn % WN;

  int tile_m, tile_n;
  tile_of_block(pid, p.tiles_m, p.tiles_n, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int M = p.M, N = p.N, K = p.K;

  // Tile-local buffer descriptors: rows past the M / N edge fall outside and read as zero.
  const int rows_a = (M - m0) < BM ? (M - m0) : BM;
  const int rows_b = (N - n0) < BN ? (N - n0) : BN;
  const __amdgpu_buffer_rsrc_t Ar = make_rsrc(p.A + (int64_t)m0 * K, (uint32_t)rows_a * (uint32_t)K);
  const __amdgpu_buffer_rsrc_t Br = make_rsrc(p.B + (int64_t)n0 * K, (uint32_t)rows_b * (uint32_t)K);

  const int col = lane & 31;
  const int rq = (lane >> 5) * 4;  // row offset of this lane's half inside each group of 8 rows
  // first row of the part of the sub-tile this wavefront finishes (wavefront-uniform: kept scalar)
  const int mw = __builtin_amdgcn_readfirstlane(m0 + wave_m * WAVE_M + wave_k * (32 * TME));

  // One load instruction of a wavefront fills 1 KiB = RPG tile rows.  Wavefront w
  // owns the row groups w, w+NWAVES, w+2*NWAVES, ... of A and of B.
  // Row of lane l in group j: RPG j + l / PPR; (row / RPL) % PPR is the same for every
  // group of a wavefront because RPG NWAVES / RPL is a multiple of PPR.
  static_assert((RPG * NWAVES / RPL) % PPR == 0, "the piece permutation is the same for all row groups of a wavefront");
  const int ld_row = wave * RPG + lane / PPR;  // + RPG*NWAVES*i
  const int ld_piece = ((lane % PPR) ^ ((ld_row / RPL) % PPR)) * 16;  // piece this lane fetches
  const uint32_t ld_off = (uint32_t)ld_row * (uint32_t)K + ld_piece;
  const uint32_t row32 = (uint32_t)(RPG * NWAVES) * (uint32_t)K;  // byte distance between a wavefront's row groups
  constexpr int NLOADS = A_LOADS + B_LOADS;
  const int nk = (K + BK - 1) / BK;
  uint32_t ld_vo[A_LOADS > B_LOADS ? A_LOADS : B_LOADS];  // EXACT: lane offset of row group i, A and B alike
#pragma unroll
  for (int i = 0; i < (A_LOADS > B_LOADS ? A_LOADS : B_LOADS); ++i) ld_vo[i] = ld_off + (uint32_t)i * row32;
  // load number `idx` (0..NLOADS-1) of K step kt into stage buffer `buf`
  auto issue_load = [&](int kt, int buf, int idx) {
    if constexpr (EXACT) {
      // steps past the last one request the last step again (into a stage nobody reads): in range by construction
      const int k0s = (kt < nk ? kt : nk - 1) * BK;  // wavefront-uniform: a scalar offset
      uint8_t* st = smem + buf * STAGE + wave * 1024;
      if (idx < A_LOADS)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(Ar, (lds_void*)(st + idx * (1024 * NWAVES)), 16, ld_vo[idx], k0s, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(Br, (lds_void*)(st + BM * BK + (idx - A_LOADS) * (1024 * NWAVES)), 16,
                                                 ld_vo[idx - A_LOADS], k0s, 0, 0);
      return;
    }
    const int k0 = kt * BK;
    // K is a multiple of 16: a piece is all in or all out.  Pieces past K would
    // alias the next row, so they are pushed outside the descriptor (-> zeros).
    const uint32_t off = (k0 + ld_piece) < K ? ld_off + (uint32_t)k0 : OOB_OFFSET;
    uint8_t* st = smem + buf * STAGE + wave * 1024;
    if (idx < A_LOADS)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(Ar, (lds_void*)(st + idx * (1024 * NWAVES)), 16,
                                               off == OOB_OFFSET ? OOB_OFFSET : off + idx * row32, 0, 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(Br, (lds_void*)(st + BM * BK + (idx - A_LOADS) * (1024 * NWAVES)), 16,
                                               off == OOB_OFFSET ? OOB_OFFSET : off + (idx - A_LOADS) * row32,
                                               0, 0, 0);
  };

#ifdef AQ_LAB_STALL
  const long long tl_start = clock64();
#endif
  using acc_t = typename Acc<FP8>::type;
  acc_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  // Fragment reads: lane -> tile row lane%32; its K pieces within a row
  // are (ks*2 + lane/32) for int8 (16 B per MFMA) and (ks*4 + (lane/32)*2 + {0,1})
  // for FP8 (32 B per MFMA); slot = piece ^ ((row / RPL) % PPR), which depends on lane%32 only
  // (sub-tile rows start at multiples of 32).
  const int fr_a = (wave_m * WAVE_M + (lane & 31)) * BK;
  const int fr_b = BM * BK + (wave_n * WAVE_N + (lane & 31)) * BK;
  const int fsw = ((lane & 31) / RPL) % PPR;
  constexpr int KSUB = FP8 ? 64 : 32;  // K per MFMA
  constexpr int NKS = BK / KSUB / WK;  // MFMA sub-steps per stage and wavefront: 4 or 2 (int8), 2 or 1 (FP8)
  // this wavefront's sub-steps of a stage start at piece wave_k * NKS * KSUB / 16; NKS is a power
  // of two, so adding the sub-step number to that base is an XOR and folds into the permutation
  const int swz = (FP8 ? ((((lane >> 5) * 2) ^ fsw) << 4) : (((lane >> 5) ^ fsw) << 4)) ^ (wave_k * NKS * KSUB);
  using frag_t = typename Frag<FP8>::type;
  auto load_frags = [&](const uint8_t* st, int ks, frag_t (&a)[TM], frag_t (&b)[TN]) {
    if constexpr (!FP8) {
      const int o = ((ks * 2) << 4) ^ swz;
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = *reinterpret_cast<const v4i*>(st + fr_a + i * 32 * BK + o);
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = *reinterpret_cast<const v4i*>(st + fr_b + j * 32 * BK + o);
    } else {
      const int o0 = ((ks * 4) << 4) ^ swz, o1 = o0 ^ 16;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const v4i lo = *reinterpret_cast<const v4i*>(st + fr_a + i * 32 * BK + o0);
        const v4i hi = *reinterpret_cast<const v4i*>(st + fr_a + i * 32 * BK + o1);
        a[i] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const v4i lo = *reinterpret_cast<const v4i*>(st + fr_b + j * 32 * BK + o0);
        const v4i hi = *reinterpret_cast<const v4i*>(st + fr_b + j * 32 * BK + o1);
        b[j] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      }
    }
  };

  // One pipeline slot = the TM*TN MFMAs of one sub-step, with the LDS reads of
  // the next sub-step's fragments and (LOADS) a share of the global->LDS loads
  // of a later stage interleaved between them, so that a wavefront (the only
  // one on its SIMD) never queues a burst of memory instructions in front of
  // the matrix core.
  frag_t af[2][TM], bf[2][TN];
  // fragment number f of a sub-step, in the order the next sub-step's MFMAs need them: A0, B0 .. B(TN-1), A1 ..
  auto load_frag = [&](const uint8_t* st, int ks, int f, frag_t (&a)[TM], frag_t (&b)[TN]) {
    const bool is_a = f == 0 || f > TN;
    const int idx = f == 0 ? 0 : f <= TN ? f - 1 : f - TN;
    const uint8_t* base = st + (is_a ? fr_a : fr_b) + idx * 32 * BK;
    if constexpr (!FP8) {
      const v4i v = *reinterpret_cast<const v4i*>(base + (((ks * 2) << 4) ^ swz));
      if (is_a) a[idx] = v; else b[idx] = v;
    } else {
      const int o0 = ((ks * 4) << 4) ^ swz;
      const v4i lo = *reinterpret_cast<const v4i*>(base + o0);
      const v4i hi = *reinterpret_cast<const v4i*>(base + (o0 ^ 16));
      const v8i v = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      if (is_a) a[idx] = v; else b[idx] = v;
    }
  };
  // slot number Q (0 = slot A .. NKS-1) issues loads [Q*NLOADS/NKS, (Q+1)*NLOADS/NKS) of its stage.
  // The order is written out and fenced: MFMA, then the fragment read(s) and at most a global load that
  // it covers, so that every memory instruction is issued in the shadow of a running MFMA and no fragment is
  // read right in front of its first use (left to itself the scheduler bunches the reads before the MFMAs
  // that need them).  The last MFMAs of a slot carry no reads: the fragments have landed when the next slot starts.
  auto slot = [&](auto cur_c, const uint8_t* st_next, int ks_next, auto loads_c, int kt_ld, int buf_ld,
                  auto q_c) {
    constexpr int CUR = decltype(cur_c)::value;
    constexpr bool LOADS = decltype(loads_c)::value;
    constexpr int Q = decltype(q_c)::value;
    constexpr int LD0 = (Q * NLOADS) / NKS, LPS = LOADS ? ((Q + 1) * NLOADS) / NKS - LD0 : 0;
    constexpr int NMMA = TM * TN, NFR = TM + TN;
    constexpr int GROUPS = NMMA > 4 ? NMMA - 2 : NMMA;  // MFMAs that carry memory instructions
    if constexpr (NMMA >= 8) {
      // Large sub-tiles (one wavefront per SIMD, or few fragment reads per MFMA): the fragment reads go out in
      // pairs behind every STRIDE-th MFMA and the global loads behind the MFMA after it.  Measured on a loop of
      // independent MFMAs with one wavefront per SIMD: two reads behind every fourth MFMA cost nothing (512.3
      // cycles per 16 MFMAs against 512.4 without reads), one behind every second 24 cycles, all eight first 40.
      constexpr int NPAIR = (NFR + 1) / 2, STRIDE = NMMA / NPAIR;
#pragma unroll
      for (int m = 0; m < NMMA; ++m) {
        acc[m / TN][m % TN] = mma<FP8>(af[CUR][m / TN], bf[CUR][m % TN], acc[m / TN][m % TN]);
        if (m % STRIDE == 0 && m / STRIDE < NPAIR) {
          load_frag(st_next, ks_next, 2 * (m / STRIDE), af[CUR ^ 1], bf[CUR ^ 1]);
          if (2 * (m / STRIDE) + 1 < NFR) load_frag(st_next, ks_next, 2 * (m / STRIDE) + 1, af[CUR ^ 1], bf[CUR ^ 1]);
        } else if (m % STRIDE == 1 && m / STRIDE < NPAIR) {
#pragma unroll
          for (int q = ((m / STRIDE) * LPS) / NPAIR; q < ((m / STRIDE + 1) * LPS) / NPAIR; ++q) issue_load(kt_ld, buf_ld, LD0 + q);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      return;
    }
#pragma unroll
    for (int m = 0; m < NMMA; ++m) {
      acc[m / TN][m % TN] = mma<FP8>(af[CUR][m / TN], bf[CUR][m % TN], acc[m / TN][m % TN]);
      if (m < GROUPS) {
#pragma unroll
        for (int f = (m * NFR) / GROUPS; f < ((m + 1) * NFR) / GROUPS; ++f) load_frag(st_next, ks_next, f, af[CUR ^ 1], bf[CUR ^ 1]);
#pragma unroll
        for (int q = (m * LPS) / GROUPS; q < ((m + 1) * LPS) / GROUPS; ++q) issue_load(kt_ld, buf_ld, LD0 + q);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using std::integral_constant;
  using k0 = integral_constant<int, 0>;
  using k1 = integral_constant<int, 1>;
  using q0 = integral_constant<int, 0>;
  using q1 = integral_constant<int, 1>;
  using q2 = integral_constant<int, 2>;
  using q3 = integral_constant<int, 3>;
  using yes = integral_constant<bool, true>;
  using no = integral_constant<bool, false>;

  // Rotated software pipeline over K steps ("stages" s = 0 .. nk-1):
  //   iteration s:  slots    MFMAs of (s, 0 .. NKS-2)       | read fragments (s, 1 .. NKS-1)
  //                 wait for this wavefront's loads of stage s+1, barrier
  //                 slot A   MFMAs of (s, last sub-step)    | read fragments (s+1, 0)
  // with the loads of stage s+NSTAGE spread from slot A of s over the slots of s+1.
  // At the barrier every wavefront holds the last fragments of stage s in
  // registers, so stage s's LDS buffer is free for the loads of stage s+NSTAGE right
  // after it, and stage s+1 is complete and visible for slot A's fragment reads.
  // Loads past the last K step are still issued (outside the descriptors they
  // write zeros into a stage nobody reads) so that the count of outstanding
  // loads per wavefront is the same at every wait.
  // Epilogue operands, requested right behind stage 0 so that their latency is
  // hidden behind the whole K loop and they never delay the first tile: per-row
  // activation scales as float4 per lane (accumulator register r of lane l
  // belongs to row (r/4)*8 + (l/32)*4 + r%4), per-column weight scale and bias
  // as one scalar per 32x32 tile column.  Nothing is done with the values until
  // the epilogue (bias stays a raw bit pattern), so no wait is placed here.
  float sx1 = 1.0f, sw1 = 1.0f;
  float sxr[BIG ? 1 : TME][4][4];  // [i][g][q]: row mw + i*32 + g*8 + rq + q (big sub-tiles: in LDS instead)
  float* const sx_lds = reinterpret_cast<float*>(smem + NSTAGE * STAGE);  // [BM], big sub-tiles only
  float swn[TN];
  uint32_t bias_raw[TN];
  const bool has_bias = OUT != OUT_I32 && p.bias != nullptr;
  const bool bias_bf16 = p.bias_dtype == AQ_BF16;
  auto load_epilogue_operands = [&]() {
    if constexpr (FP8) {
      sx1 = *p.sx;
      sw1 = *p.sw;
      const __amdgpu_buffer_rsrc_t Bsr =
          make_rsrc(has_bias ? p.bias : (const void*)p.sw, has_bias ? (uint32_t)N * (bias_bf16 ? 2u : 4u) : 0u);
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const uint32_t n = (uint32_t)(n0 + wave_n * WAVE_N + j * 32 + col);  // past N, or no bias: outside -> 0
        bias_raw[j] = bias_bf16 ? (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(Bsr, n * 2u, 0, 0)
                                : (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(Bsr, n * 4u, 0, 0);
      }
    } else if constexpr (OUT != OUT_I32) {
      // rows past M fall outside the descriptor and read as zero (their outputs are never stored)
      const int rows_left = __builtin_amdgcn_readfirstlane((M - mw) > 0 ? (M - mw) : 0);
      const __amdgpu_buffer_rsrc_t Sr =
          make_rsrc(p.sx + (rows_left ? mw : 0), (uint32_t)(rows_left < 32 * TME ? rows_left : 32 * TME) * 4u);
      if constexpr (BIG) {
        // the tile's BM scales straight into LDS, 64 per load instruction; rows past M read as zero
        const __amdgpu_buffer_rsrc_t Tr = make_rsrc(p.sx + m0, (uint32_t)rows_a * 4u);
#pragma unroll
        for (int r = 0; r < BM / 64 / NWAVES; ++r)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(Tr, (lds_void*)(sx_lds + (r * NWAVES + wave) * 64), 4,
                                                   (uint32_t)((r * NWAVES + wave) * 64 + lane) * 4u, 0, 0, 0);
      } else if ((M & 3) == 0) {  // uniform: the 4 rows of a float4 are all in or all out, and 16-byte aligned
#pragma unroll
        for (int i = 0; i < TME; ++i)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const uint4 t = buffer_load_16(Sr, (uint32_t)(i * 32 + g * 8 + rq) * 4u);
            sxr[i][g][0] = __uint_as_float(t.x);
            sxr[i][g][1] = __uint_as_float(t.y);
            sxr[i][g][2] = __uint_as_float(t.z);
            sxr[i][g][3] = __uint_as_float(t.w);
          }
      } else {
#pragma unroll
        for (int i = 0; i < TME; ++i)
#pragma unroll
          for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int q = 0; q < 4; ++q)
              sxr[i][g][q] = __uint_as_float(
                  (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(Sr, (i * 32 + g * 8 + rq + q) * 4, 0, 0));
      }
      const __amdgpu_buffer_rsrc_t Wsr = make_rsrc(p.sw, (uint32_t)N * 4u);
      const __amdgpu_buffer_rsrc_t Bsr =
          make_rsrc(has_bias ? p.bias : p.sw, has_bias ? (uint32_t)N * (bias_bf16 ? 2u : 4u) : 0u);
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const uint32_t n = (uint32_t)(n0 + wave_n * WAVE_N + j * 32 + col);  // past N: outside -> 0
        swn[j] = __uint_as_float((uint32_t)__builtin_amdgcn_raw_buffer_load_b32(Wsr, n * 4u, 0, 0));
        bias_raw[j] = bias_bf16 ? (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(Bsr, n * 2u, 0, 0)
                                : (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(Bsr, n * 4u, 0, 0);
      }
    }
  };
#pragma unroll
  for (int q = 0; q < NLOADS; ++q) issue_load(0, 0, q);
  asm volatile("" ::: "memory");  // keep the request order: stage 0, epilogue operands, the other stages
  load_epilogue_operands();
  asm volatile("" ::: "memory");
#pragma unroll
  for (int st = 1; st < NSTAGE; ++st)
#pragma unroll
    for (int q = 0; q < NLOADS; ++q) issue_load(st, st, q);

  // sub-steps 0 .. NKS-2 of a stage whose first fragments sit in af[C0]
  auto middle_slots = [&](auto c0_c, const uint8_t* stc, auto loads_c, int kt_ld, int buf_ld) {
    constexpr int C0 = decltype(c0_c)::value;
    using c0 = integral_constant<int, C0>;
    using c1 = integral_constant<int, C0 ^ 1>;
    if constexpr (NKS == 4) {
      slot(c0{}, stc, 1, loads_c, kt_ld, buf_ld, q1{});
      slot(c1{}, stc, 2, loads_c, kt_ld, buf_ld, q2{});
      slot(c0{}, stc, 3, loads_c, kt_ld, buf_ld, q3{});
    } else if constexpr (NKS == 2) {
      slot(c0{}, stc, 1, loads_c, kt_ld, buf_ld, q1{});
    }
  };
  // the fragment buffer the last sub-step of such a stage computes from
  auto last_of = [](auto c0_c) { return integral_constant<int, (NKS % 2 == 0) ? (decltype(c0_c)::value ^ 1) : decltype(c0_c)::value>{}; };

  AQ_WAIT_VMCNT((NSTAGE - 1) * NLOADS);  // all but the younger stages: stage 0 (and the operands) have landed
  AQ_BARRIER();
#ifdef AQ_LAB_STALL
  const long long tl_stage0 = clock64();
#endif
  load_frags(smem, 0, af[0], bf[0]);
  middle_slots(k0{}, smem, no{}, 0, 0);  // no loads to issue yet: every stage buffer is in flight
  __builtin_amdgcn_s_waitcnt(0xc07f);        // lgkmcnt(0): the last fragments of stage 0 are in registers
  AQ_WAIT_VMCNT((NSTAGE - 2) * NLOADS);  // stage 1 has landed
  AQ_BARRIER();
  // slot A of stage 0: its buffer (0) is free now and takes stage NSTAGE
  slot(last_of(k0{}), smem + STAGE, 0, yes{}, NSTAGE, 0, q0{});
  int b_prev = 0;  // buffer of stage s-1
#ifdef AQ_LAB_STALL
  long long st_t0 = 0, st_t1 = 0, st_sum = 0;
  const long long st_begin = clock64();
#endif
  auto stage = [&](int s, auto c0_c) {
    const int b_cur = b_prev == NSTAGE - 1 ? 0 : b_prev + 1;
    const int b_next = b_cur == NSTAGE - 1 ? 0 : b_cur + 1;
    // sub-steps 0 .. NKS-2 of stage s; the rest of stage s-1+NSTAGE's loads go into stage s-1's buffer
    middle_slots(c0_c, smem + b_cur * STAGE, yes{}, s - 1 + NSTAGE, b_prev);
#ifdef AQ_LAB_STALL
    const long long st_now = clock64();
#endif
    __builtin_amdgcn_s_waitcnt(0xc07f);        // lgkmcnt(0): the last fragments of stage s are in registers
    AQ_WAIT_VMCNT((NSTAGE - 2) * NLOADS);  // stage s+1 has landed (later ones may still be in flight)
    AQ_BARRIER();
#ifdef AQ_LAB_STALL
    st_sum += st_t1 - st_t0;  // the previous step's wait: both of its clock reads have returned by now
    st_t0 = st_now;
    st_t1 = clock64();
#endif
    // slot A: last sub-step of stage s | first fragments of stage s+1 | first loads of stage s+NSTAGE
    slot(last_of(c0_c), smem + b_next * STAGE, 0, yes{}, s + NSTAGE, b_cur, q0{});
    b_prev = b_cur;
  };
  if constexpr (NKS % 2 == 0) {
    for (int s = 1; s < nk; ++s) stage(s, k0{});
  } else {  // one sub-step per stage: the fragment buffers alternate per stage
    int s = 1;
    for (; s + 1 < nk; s += 2) {
      stage(s, k1{});
      stage(s + 1, k0{});
    }
    if (s < nk) stage(s, k1{});
  }
  AQ_WAIT_VMCNT(0);  // drain the padding loads before the workgroup's LDS can be released or reused
#ifdef AQ_LAB_STALL
  const long long tl_loop_end = clock64();
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    aq_lab_clock[2] = st_sum + (st_t1 - st_t0);
    aq_lab_clock[3] = tl_loop_end - st_begin;
    aq_lab_clock[4] = tl_stage0 - tl_start;   // tile start -> first stage landed and visible
    aq_lab_clock[5] = st_begin - tl_stage0;   // first K step without loads
  }
#endif

  if constexpr (WK == 2) {
    // The two wavefronts of a sub-tile hold the sums over their halves of every K step.  Each
    // keeps half of the row blocks (the first wavefront the upper ones) and parks the other half
    // in LDS for its partner (over the stage buffers, which nobody reads any more once every
    // wavefront is past the barrier); then both add what the partner left for them and run the
    // epilogue on their half.  int32 sums are exact in any order; FP8 partial sums are fp32,
    // inside the stated tolerance.
    __syncthreads();
    using part_t = std::conditional_t<FP8, v4f, v4i>;
    constexpr int SLOT = TME * TN * 4 * 64;  // part_t elements one wavefront parks
    part_t* mine = reinterpret_cast<part_t*>(smem) + (wave_mn * 2 + wave_k) * SLOT + lane;
    part_t* theirs = reinterpret_cast<part_t*>(smem) + (wave_mn * 2 + (wave_k ^ 1)) * SLOT + lane;
    static_assert(NWAVES * SLOT * 16 <= NSTAGE * STAGE, "the parked accumulators fit the stage buffers");
    if (wave_k == 0) {  // uniform
#pragma unroll
      for (int i = 0; i < TME; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g)
            mine[((i * TN + j) * 4 + g) * 64] = part_t{acc[TME + i][j][g * 4], acc[TME + i][j][g * 4 + 1],
                                                       acc[TME + i][j][g * 4 + 2], acc[TME + i][j][g * 4 + 3]};
    } else {
#pragma unroll
      for (int i = 0; i < TME; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
          for (int g = 0; g < 4; ++g)
            mine[((i * TN + j) * 4 + g) * 64] =
                part_t{acc[i][j][g * 4], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2], acc[i][j][g * 4 + 3]};
          acc[i][j] = acc[TME + i][j];  // the lower row blocks move to the front: the epilogue indexes from 0
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TME; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const part_t t = theirs[((i * TN + j) * 4 + g) * 64];
#pragma unroll
          for (int q = 0; q < 4; ++q) acc[i][j][g * 4 + q] += t[q];
        }
  }

  // ---- epilogue, straight from the accumulator registers (no LDS, no barrier).
  // A lane owns one output column per 32x32 tile and 64 of the wavefront's 128
  // rows.  Stores go through a buffer descriptor based at the wavefront's first
  // output: the lane part of the address (its column, its half of the 8-row
  // group) is one VGPR computed once, the row part is a scalar offset, so no
  // vector ALU work is spent on addresses.  Lanes whose column is past N carry
  // an out-of-range offset and their stores are dropped by the hardware.
  // bf16 outputs are paired across neighbouring lanes: each lane converts its
  // two rows (2h, 2h+1) into one packed dword, swaps it with its neighbour
  // (DPP quad_perm [1,0,3,2]) and byte-permutes the two into "my row, both
  // columns": even lanes write row 2h, odd lanes row 2h+1, 4 bytes per lane,
  // 64 contiguous bytes per row segment.
  constexpr int ESZ = (OUT == OUT_BF16) ? 2 : 4;
  const int nw = __builtin_amdgcn_readfirstlane(n0 + wave_n * WAVE_N);  // first column of this wavefront
  const __amdgpu_buffer_rsrc_t Cr =
      make_rsrc(reinterpret_cast<uint8_t*>(p.C) + ((int64_t)mw * N + nw) * ESZ, 0x40000000u);
  // Residual: the same window over the tensor that is added to the rounded output; each lane
  // reads exactly the elements it then writes, so the residual may be the output itself.
  const bool has_res = !BIG && OUT != OUT_I32 && p.res != nullptr;  // uniform (big sub-tiles are not launched with a residual)
  const __amdgpu_buffer_rsrc_t Rr = make_rsrc(
      reinterpret_cast<const uint8_t*>(has_res ? p.res : p.C) + ((int64_t)mw * N + nw) * ESZ, has_res ? 0x40000000u : 0u);
  const bool pair_ok = (N & 1) == 0;  // uniform: bf16 rows start dword-aligned, pairs never straddle N
  const bool odd = lane & 1;
  const uint32_t perm_sel = odd ? 0x03020706u : 0x05040100u;
  const uint32_t rowb = (uint32_t)N * ESZ;
  const bool rows_inside = mw + 32 * TME <= M;  // uniform
  // CHECK_M: some rows of this wavefront are past M.  PAIR: the bf16 dword path.
  auto store_all = [&](auto check_c, auto pair_c) {
    constexpr bool CHECK_M = decltype(check_c)::value;
    constexpr bool PAIR = (OUT == OUT_BF16) && decltype(pair_c)::value;
    // lane part of the byte offset of column j; the pairing path stores at the even column of the pair
    auto lane_offset = [&](int j) -> uint32_t {
      const int cj = j * 32 + col;  // column inside the wavefront's 64
      return nw + cj < N ? (uint32_t)rq * rowb + (uint32_t)(PAIR ? (cj & ~1) : cj) * ESZ + (PAIR && odd ? rowb : 0u)
                         : OOB_OFFSET;
    };
    // The residual elements a lane will add, requested ahead of the arithmetic: all columns at once on
    // the paired bf16 path (32 registers; the stores of one column would otherwise sit between the
    // loads of the next and their use), column by column on the others.
    constexpr int RLD = PAIR ? 2 : 4;  // loads per 4-row group: packed row pairs, or single elements
    constexpr bool HOIST = PAIR && TN * TME <= 4;
    uint32_t rr[HOIST ? TN : 1][TME][4][RLD];
    auto load_residual = [&](int j) {
      const uint32_t vbase = lane_offset(j);
#pragma unroll
      for (int i = 0; i < TME; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
          for (int q = 0; q < RLD; ++q) {
            const int r0 = i * 32 + g * 8;
            const int rowq = PAIR ? 2 * q : q;
            uint32_t vo = vbase;
            if (CHECK_M && mw + r0 + rq + rowq + (PAIR && odd ? 1 : 0) >= M) vo = OOB_OFFSET;
            if constexpr (OUT == OUT_F32 || PAIR)
              rr[HOIST ? j : 0][i][g][q] = __builtin_amdgcn_raw_buffer_load_b32(Rr, vo, (r0 + rowq) * rowb, 0);
            else
              rr[HOIST ? j : 0][i][g][q] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(Rr, vo, (r0 + rowq) * rowb, 0);
          }
    };
    if constexpr (OUT != OUT_I32 && HOIST) {
      if (has_res) {
#pragma unroll
        for (int j = 0; j < TN; ++j) load_residual(j);
      }
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      float bn = 0.0f;
      if constexpr (OUT != OUT_I32)
        bn = !has_bias ? 0.0f : bias_bf16 ? bf16_bits_to_f32(bias_raw[j]) : __uint_as_float(bias_raw[j]);
      const uint32_t vbase = lane_offset(j);
      if constexpr (OUT != OUT_I32 && !HOIST) {
        if (has_res) load_residual(j);
      }
#pragma unroll
      for (int i = 0; i < TME; ++i) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int r0 = i * 32 + g * 8;  // + rq + q : row inside the wavefront's 128
          if constexpr (OUT == OUT_I32) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              uint32_t vo = vbase;
              if (CHECK_M && mw + r0 + rq + q >= M) vo = OOB_OFFSET;
              __builtin_amdgcn_raw_buffer_store_b32((uint32_t)acc[i][j][g * 4 + q], Cr, vo, (r0 + q) * rowb, STORE_WT);
            }
          } else {
            float y[4];
            v4f sxq = {0.0f, 0.0f, 0.0f, 0.0f};
            if constexpr (BIG && !FP8)
              sxq = *reinterpret_cast<const v4f*>(sx_lds + (mw - m0) + r0 + rq);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              if constexpr (FP8) {
                // without a bias bn is +0: it changes no bit unless the product is -0, whose sign a bf16 or
                // fp32 consumer of a Linear output never sees as a different value
                y[q] = __fadd_rn(__fmul_rn(__fmul_rn(acc[i][j][g * 4 + q], sx1), sw1), bn);
              } else {
                // three separately rounded fp32 operations, never contracted.  Without a bias
                // bn is +0: the product of an integer and two positive scales is never -0,
                // so adding it changes no bit.
                y[q] = __fadd_rn(__fmul_rn(__fmul_rn((float)acc[i][j][g * 4 + q], BIG ? sxq[q] : sxr[BIG ? 0 : i][g][q]), swn[j]), bn);
              }
            }
            if constexpr (OUT == OUT_F32) {
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                uint32_t vo = vbase;
                if (CHECK_M && mw + r0 + rq + q >= M) vo = OOB_OFFSET;
                if (has_res) y[q] = __fadd_rn(y[q], __uint_as_float(rr[HOIST ? j : 0][i][g][q]));
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(y[q]), Cr, vo, (r0 + q) * rowb, STORE_WT);
              }
            } else if constexpr (PAIR) {
#pragma unroll
              for (int h = 0; h < 2; ++h) {
                const uint32_t mine = pack_bf16x2(y[2 * h], y[2 * h + 1]);  // lo: row 2h, hi: row 2h+1
                const uint32_t other =
                    (uint32_t)__builtin_amdgcn_mov_dpp((int)mine, 0xB1 /* quad_perm [1,0,3,2] */, 0xf, 0xf, true);
                // even lane: {mine.lo, other.lo} = row 2h, columns (c, c+1)
                // odd lane:  {other.hi, mine.hi} = row 2h+1, columns (c-1, c)
                uint32_t pk = __builtin_amdgcn_perm(other, mine, perm_sel);
                if (has_res) {  // rounded output + residual, rounded again: what a separate add gives
                  const uint32_t r = rr[HOIST ? j : 0][i][g][h];
                  pk = pack_bf16x2(__fadd_rn(__uint_as_float(pk << 16), __uint_as_float(r << 16)),
                                   __fadd_rn(__uint_as_float(pk & 0xffff0000u), __uint_as_float(r & 0xffff0000u)));
                }
                uint32_t vo = vbase;
                if (CHECK_M && mw + r0 + rq + 2 * h + (odd ? 1 : 0) >= M) vo = OOB_OFFSET;
                __builtin_amdgcn_raw_buffer_store_b32(pk, Cr, vo, (r0 + 2 * h) * rowb, STORE_WT);
              }
            } else {
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                uint32_t vo = vbase;
                if (CHECK_M && mw + r0 + rq + q >= M) vo = OOB_OFFSET;
                uint32_t ob = f32_to_bf16_bits(y[q]);
                if (has_res) ob = f32_to_bf16_bits(__fadd_rn(__uint_as_float(ob << 16), __uint_as_float(rr[HOIST ? j : 0][i][g][q] << 16)));
                __builtin_amdgcn_raw_buffer_store_b16((uint16_t)ob, Cr, vo, (r0 + q) * rowb, STORE_WT);
              }
            }
          }
        }
      }
    }
  };
  if constexpr (BIG) {
    store_all(no{}, yes{});  // one variant (256 outputs per lane): the launcher sends ragged M and odd N to another shape
  } else {
    if (rows_inside && pair_ok)
      store_all(no{}, yes{});   // interior tiles: straight-line, no per-row checks
    else if (pair_ok)
      store_all(yes{}, yes{});
    else
      store_all(yes{}, no{});
  }
#ifdef AQ_LAB_STALL
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    aq_lab_clock[6] = clock64() - tl_loop_end;  // accumulator exchange (split K steps) + epilogue issue
    aq_lab_clock[7] = clock64() - tl_start;     // the whole tile as wavefront 0 sees it
  }
#endif
}

// A workgroup walks tiles pid, pid + gridDim.x, ...: with more tiles than compute units the launch is one
// resident workgroup per compute unit instead of a queue of short-lived ones (the LDS stages allow one at a time).
template <bool FP8, int OUT, class S>
__global__ __launch_bounds__(S::NTHREADS) void gemm_kernel(GemmArgs p) {
  __shared__ __attribute__((aligned(1024))) uint8_t smem[S::LDS_BYTES];
  const int nt = p.tiles_m * p.tiles_n;
#ifdef AQ_LAB
  struct Clk {
    long long c0, w0;
    __device__ Clk() : c0(clock64()), w0(wall_clock64()) {}
    __device__ ~Clk() {
      if (blockIdx.x == 0 && threadIdx.x == 0) {
        aq_lab_clock[0] = clock64() - c0;
        aq_lab_clock[1] = wall_clock64() - w0;
      }
    }
  } clk;
#endif
  const bool exact = (p.K % S::BK) == 0;  // uniform
  for (int pid = blockIdx.x; pid < nt; pid += gridDim.x) {
    if constexpr (S::BIG)
      gemm_tile<FP8, OUT, S, true>(p, smem, pid);  // launched for whole K steps and even N only
    else if (exact)
      gemm_tile<FP8, OUT, S, true>(p, smem, pid);
    else
      gemm_tile<FP8, OUT, S, false>(p, smem, pid);
    if (pid + (int)gridDim.x < nt) __syncthreads();  // every wavefront is done with the stages before they are refilled
  }
}

// Tile shape by the number of rounds over the compute units a launch needs: a workgroup per compute unit at a
// time, so the cost of a launch is its number of rounds times the cost of a round of that shape (us at K = 2048
// with the weights streamed from HBM, on top of 4 us of launch and pipeline fill; every term scales with K alike):
//   256 x 128: 15.0   128 x 128: 10.8   128 x 64: 7.0   128 x 32: 5.0   64 x 64: 4.6   64 x 32: 3.5
// After a full round, a last round of the two wide shapes that fills only part of the device costs about half a
// round plus half its fill (384 large tiles, 1.5 rounds, take 1.74 times as long as 256); a first round runs at the
// latency of its K loop whatever the fill (128 x 128: 64 tiles 12.3-14.8 us, 256 tiles 14.5 us), and so does every
// round of the small shapes (64 x 32: 64 tiles 6.9 us, 256 tiles 7.0 us, 352 tiles 12.0 us), whose rounds count
// whole.  Fitted on
// 33..2048 rows against N = 1024..16384 and K = 1024..5632, where the rule picks the fastest shape or one within
// 6 % of it.  The small tiles are for launches of a few rounds only.
enum TileKind {
  TILE_AUTO = 0, TILE_N32 = 32, TILE_M64N32 = 33, TILE_N64 = 64, TILE_M64N64 = 65, TILE_SMALL = 128, TILE_PAIR = 129,
  TILE_LARGE = 256, TILE_TALL = 257, TILE_HUGE = 512, TILE_HUGE8 = 513
};
#ifdef AQ_LAB
static int g_forced_tile = 0;  // lab build only: TILE_AUTO = by shape, otherwise forced (tuning and tests)
#endif

static int choose_tile_for(int64_t M, int64_t N, int64_t cus) {
  auto rounds = [cus](int64_t tiles) {
    const int64_t full = tiles / cus, rest = tiles % cus;
    if (full == 0) return 1.0;
    return (double)full + (rest ? 0.5 + 0.5 * (double)rest / cus : 0.0);
  };
  struct Cand {
    int kind, bm, bn;
    double round_us;
    bool small;
  };
  static const Cand cands[] = {{TILE_LARGE, 256, 128, 15.0, false}, {TILE_SMALL, 128, 128, 10.8, false},
                               {TILE_N64, 128, 64, 7.0, true},      {TILE_N32, 128, 32, 5.0, true},
                               {TILE_M64N64, 64, 64, 4.6, true},    {TILE_M64N32, 64, 32, 3.5, true}};
  int best = TILE_LARGE;
  double cost = 0.0;
  for (const Cand& c : cands) {
    const int64_t tiles = ((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn);
    if (c.small && tiles > 4 * cus) continue;
    const double us = c.round_us * (c.small ? (double)((tiles + cus - 1) / cus) : rounds(tiles));
    if (c.kind == TILE_LARGE || us < cost) {
      cost = us;
      best = c.kind;
    }
  }
  return best;
}

static int choose_tile(int64_t M, int64_t N) {
#ifdef AQ_LAB
  if (g_forced_tile) return g_forced_tile;
#endif
  return choose_tile_for(M, N, device_cus());
}

template <bool FP8, int OUT, class S>
static int launch_shape(GemmArgs& a, hipStream_t st) {
  a.tiles_m = (a.M + S::BM - 1) / S::BM;
  a.tiles_n = (a.N + S::BN - 1) / S::BN;
  // one resident workgroup per compute unit walks the tiles (a workgroup's LDS stages fill a compute unit):
  // 3-5 % faster than queueing a workgroup per tile once there are more tiles than compute units
  const int64_t ntiles = (int64_t)a.tiles_m * a.tiles_n, cus = device_cus();
  const unsigned grid = (unsigned)(ntiles < cus ? ntiles : cus);
  hipLaunchKernelGGL((gemm_kernel<FP8, OUT, S>), dim3(grid), dim3(S::NTHREADS), 0, st, a);
  return (int)hipGetLastError();
}

// FP8 launches the 256 x 256 tile serves and gains on: whole 256-row multiples, even N, whole 64-byte K steps, no
// residual (the tile's one K-loop and epilogue variant), and at least two rounds of such tiles over the compute
// units (one round -- 4096^3 -- measured level with the 256 x 128 tile, 57.0 against 57.7 us).
static bool huge_fp8_ok(const GemmArgs& a) {
  if ((a.K % ShapeHuge::BK) != 0 || (a.N % 2) != 0 || (a.M % ShapeHuge::BM) != 0 || a.res != nullptr) return false;
  const int64_t tiles = (int64_t)(a.M / ShapeHuge::BM) * ((a.N + ShapeHuge::BN - 1) / ShapeHuge::BN);
  return tiles >= 2 * (int64_t)device_cus();
}

template <bool FP8, int OUT>
static int launch(GemmArgs& a, hipStream_t st) {
#ifdef AQ_LAB
  const bool forced = g_forced_tile != 0;
#else
  const bool forced = false;
#endif
  if constexpr (FP8 && OUT != OUT_I32) {
    if (!forced && huge_fp8_ok(a)) return launch_shape<FP8, OUT, ShapeHuge>(a, st);
  }
  switch (choose_tile(a.M, a.N)) {
    case TILE_SMALL: return launch_shape<FP8, OUT, ShapeSmall>(a, st);
    case TILE_N64: return launch_shape<FP8, OUT, ShapeN64>(a, st);
    case TILE_N32: return launch_shape<FP8, OUT, ShapeN32>(a, st);
    case TILE_M64N64: return launch_shape<FP8, OUT, ShapeM64N64>(a, st);
    case TILE_M64N32: return launch_shape<FP8, OUT, ShapeM64N32>(a, st);
#ifdef AQ_LAB
    case TILE_TALL: return launch_shape<FP8, OUT, ShapeTall>(a, st);
    case TILE_HUGE:
      if ((a.K % ShapeHuge::BK) == 0 && (a.N % 2) == 0 && (a.M % ShapeHuge::BM) == 0 && a.res == nullptr)
        return launch_shape<FP8, OUT, ShapeHuge>(a, st);
      return launch_shape<FP8, OUT, ShapeLarge>(a, st);
    case TILE_HUGE8: return launch_shape<FP8, OUT, ShapeHuge8>(a, st);
    case TILE_PAIR: return launch_shape<FP8, OUT, ShapePair>(a, st);
#endif
    default: return launch_shape<FP8, OUT, ShapeLarge>(a, st);
  }
}

static int check_gemm(const void* A, const void* B, const void* C, int64_t M, int64_t N, int64_t K) {
  if (M < 0 || N < 0 || K <= 0 || (K % 16) != 0) return AQ_E_SHAPE;
  if (M == 0 || N == 0) return AQ_OK;
  if (!A || !B || !C) return AQ_E_NULL;
  if (check_ptr16(A) || check_ptr16(B) || check_ptr16(C)) return AQ_E_ALIGN;
  // 32-bit tile-relative offsets: 256 rows * K bytes of an operand and 256 rows * N * 4 bytes of the
  // output window of a workgroup must fit 31 bits
  if (K > (1 << 22) || M > (1 << 30) || N > (1 << 20)) return AQ_E_RANGE;
  if (((M + 127) / 128) * ((N + 127) / 128) > (int64_t)0x7fffffff) return AQ_E_RANGE;
  return AQ_OK;
}

static GemmArgs make_args(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K) {
  GemmArgs a{};
  a.A = static_cast<const uint8_t*>(A);
  a.B = static_cast<const uint8_t*>(B);
  a.C = C;
  a.M = (int)M;
  a.N = (int)N;
  a.K = (int)K;
  return a;
}

}  // namespace aq

#ifdef AQ_LAB
extern "C" int aq_lab_read_clock(long long* host2) {
  return (int)hipMemcpyFromSymbol(host2, HIP_SYMBOL(aq::aq_lab_clock), 64);
}
extern "C" int aq_lab_set_gemm_tile(int rows) {
  if (rows != 0 && rows != 129 && rows != 33 && rows != 65 && rows != 64 && rows != 32 && rows != 128 && rows != 256 && rows != 257 && rows != 512 && rows != 513) return AQ_E_SHAPE;
  aq::g_forced_tile = rows;
  return AQ_OK;
}
extern "C" int aq_lab_choose_gemm_tile(int64_t M, int64_t N, int compute_units) {
  if (M <= 0 || N <= 0 || compute_units <= 0) return AQ_E_SHAPE;
  return aq::choose_tile_for(M, N, compute_units);
}
#endif

extern "C" int aq_gemm_i8_i32(const int8_t* xq, const int8_t* wq, int32_t* acc, int64_t M, int64_t N,
                              int64_t K, void* stream) {
  int rc = aq::check_gemm(xq, wq, acc, M, N, K);
  if (rc || M == 0 || N == 0) return rc;
  aq::GemmArgs a = aq::make_args(xq, wq, acc, M, N, K);
  return aq::launch<false, aq::OUT_I32>(a, static_cast<hipStream_t>(stream));
}

extern "C" int aq_linear_w8a8(const int8_t* xq, const float* sx, const int8_t* wq, const float* sw,
                              const void* bias, int bias_dtype, void* y, int y_dtype, int64_t M,
                              int64_t N, int64_t K, void* stream) {
  return aq_linear_w8a8_residual(xq, sx, wq, sw, bias, bias_dtype, nullptr, y, y_dtype, M, N, K, stream);
}

namespace aq {
// gemv.hip: the weight-streaming kernel for 17..32 rows (same sums, same epilogue: same bits)
bool gemv_tokens_ok(int64_t M, int64_t N, int64_t K);
int gemv_tokens_launch(const int8_t* xq, const float* sx, const int8_t* wq, const float* sw, const void* bias,
                       int bias_dtype, const void* residual, void* y, int y_dtype, int64_t M, int64_t N, int64_t K,
                       hipStream_t st, bool fp8);
}  // namespace aq

extern "C" int aq_linear_w8a8_residual(const int8_t* xq, const float* sx, const int8_t* wq, const float* sw,
                                       const void* bias, int bias_dtype, const void* residual, void* y, int y_dtype,
                                       int64_t M, int64_t N, int64_t K, void* stream) {
  if (y_dtype != AQ_F32 && y_dtype != AQ_BF16) return AQ_E_DTYPE;
  if (bias && bias_dtype != AQ_F32 && bias_dtype != AQ_BF16) return AQ_E_DTYPE;
  int rc = aq::check_gemm(xq, wq, y, M, N, K);
  if (rc || M == 0 || N == 0) return rc;
  if (!sx || !sw) return AQ_E_NULL;
  if (aq::check_ptr(sx, 4) || aq::check_ptr(sw, 4) || aq::check_ptr(bias, bias_dtype == AQ_BF16 ? 2 : 4) ||
      aq::check_ptr(residual, 4))
    return AQ_E_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // 17..32 rows (and decode batches of rows too long for the GEMV kernels): the weight-streaming kernel takes
  // them (not when a test has forced a tile shape)
#ifdef AQ_LAB
  const bool tile_forced = aq::g_forced_tile != 0;
#else
  const bool tile_forced = false;
#endif
  if (!tile_forced && aq::gemv_tokens_ok(M, N, K) && aq::check_ptr16(residual) == 0)
    return aq::gemv_tokens_launch(xq, sx, wq, sw, bias, bias_dtype, residual, y, y_dtype, M, N, K, st, false);
  aq::GemmArgs a = aq::make_args(xq, wq, y, M, N, K);
  a.sx = sx;
  a.sw = sw;
  a.bias = bias;
  a.bias_dtype = bias_dtype;
  a.res = residual;
  return y_dtype == AQ_BF16 ? aq::launch<false, aq::OUT_BF16>(a, st) : aq::launch<false, aq::OUT_F32>(a, st);
}

extern "C" int aq_linear_fp8(const uint8_t* xq, const float* sx, const uint8_t* wq, const float* sw,
                             void* y, int y_dtype, int64_t M, int64_t N, int64_t K, void* stream) {
  return aq_linear_fp8_residual(xq, sx, wq, sw, nullptr, AQ_F32, nullptr, y, y_dtype, M, N, K, stream);
}

extern "C" int aq_linear_fp8_residual(const uint8_t* xq, const float* sx, const uint8_t* wq, const float* sw,
                                      const void* bias, int bias_dtype, const void* residual, void* y, int y_dtype,
                                      int64_t M, int64_t N, int64_t K, void* stream) {
  if (y_dtype != AQ_F32 && y_dtype != AQ_BF16) return AQ_E_DTYPE;
  if (bias && bias_dtype != AQ_F32 && bias_dtype != AQ_BF16) return AQ_E_DTYPE;
  int rc = aq::check_gemm(xq, wq, y, M, N, K);
  if (rc || M == 0 || N == 0) return rc;
  if (!sx || !sw) return AQ_E_NULL;
  if (aq::check_ptr(sx, 4) || aq::check_ptr(sw, 4) || aq::check_ptr(bias, bias_dtype == AQ_BF16 ? 2 : 4) ||
      aq::check_ptr(residual, 4))
    return AQ_E_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // 17..32 rows: the weight-streaming kernel, as for int8 (fp32 sums in its own fixed order)
#ifdef AQ_LAB
  const bool tile_forced = aq::g_forced_tile != 0;
#else
  const bool tile_forced = false;
#endif
  if (!tile_forced && aq::gemv_tokens_ok(M, N, K) && aq::check_ptr16(residual) == 0)
    return aq::gemv_tokens_launch(reinterpret_cast<const int8_t*>(xq), sx, reinterpret_cast<const int8_t*>(wq), sw, bias,
                                  bias_dtype, residual, y, y_dtype, M, N, K, st, true);
  aq::GemmArgs a = aq::make_args(xq, wq, y, M, N, K);
  a.sx = sx;
  a.sw = sw;
  a.bias = bias;
  a.bias_dtype = bias_dtype;
  a.res = residual;
  return y_dtype == AQ_BF16 ? aq::launch<true, aq::OUT_BF16>(a, st) : aq::launch<true, aq::OUT_F32>(a, st);
}
