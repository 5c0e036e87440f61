// Prefill GEMMs on the CDNA4 matrix cores: int8 x int8 -> int32
// (v_mfma_i32_32x32x32_i8) and FP8 e4m3 x e4m3 -> fp32
// (v_mfma_scale_f32_32x32x64_f8f6f4 with unit scales), one kernel template.
//
//   C[m, n] = sum_k A[m, k] * B[n, k]     A = activation codes [M, K]
//                                         B = weight codes     [N, K]
// Both operands are K-contiguous, which is exactly the MFMA operand order
// (each lane feeds 16 or 32 consecutive k of one row), so no transpose is ever
// materialised.  A workgroup of 4 wavefronts owns a 256 x 128 tile of C; each
// wavefront a 128 x 64 sub-tile held as 4 x 2 MFMA 32x32 accumulators (128
// registers).  K is walked in 128-byte steps: global -> registers -> LDS with
// two LDS stages, one barrier per step; rows are padded by 16 bytes so the
// 16-byte fragment reads of 8 consecutive rows cover all 32 banks.
// The epilogue is fused: int32 store, or dequantise (+bias) and cast.
#include "aq_common.h"

namespace aq {

constexpr int BM = 256, BN = 128, BK = 128;
constexpr int PITCH = BK + 16;
constexpr int WAVE_M = 128, WAVE_N = 64;  // 2 x 2 wavefronts
constexpr int TM = WAVE_M / 32, TN = WAVE_N / 32;
constexpr int A_LOADS = BM * BK / 16 / 256;  // 16-byte vectors per thread per K step
constexpr int B_LOADS = BN * BK / 16 / 256;
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

template <bool FP8, int OUT>
__global__ __launch_bounds__(256) void gemm_kernel(GemmArgs p) {
  __shared__ __attribute__((aligned(16))) uint8_t smem[2 * (BM + BN) * PITCH];
  uint8_t* const sA0 = smem;
  uint8_t* const sB0 = smem + BM * PITCH;
  constexpr int STAGE = (BM + BN) * PITCH;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave >> 1, wave_n = wave & 1;

  int tile_m, tile_n;
  tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int M = p.M, N = p.N, K = p.K;

  // ---- global -> LDS staging assignment: vector c = i*256 + tid, row = c/8
  const int ld_row = tid >> 3;       // + 32*i
  const int ld_kc = (tid & 7) * 16;  // byte offset inside the K step
  // Tile-local buffer descriptors: rows past the M / N edge fall outside and read as zero.
  const int rows_a = (M - m0) < BM ? (M - m0) : BM;
  const int rows_b = (N - n0) < BN ? (N - n0) : BN;
  const __amdgpu_buffer_rsrc_t Ar = make_rsrc(p.A + (int64_t)m0 * K, (uint32_t)rows_a * (uint32_t)K);
  const __amdgpu_buffer_rsrc_t Br = make_rsrc(p.B + (int64_t)n0 * K, (uint32_t)rows_b * (uint32_t)K);
  const uint32_t ld_off = (uint32_t)ld_row * (uint32_t)K + ld_kc;  // + 32*i rows, + k0
  const uint32_t row32 = 32u * (uint32_t)K;

  uint4 ra[A_LOADS], rb[B_LOADS];
  auto gload = [&](int k0) {
    // K is a multiple of 16: a vector is all in or all out.  Vectors past K
    // would alias the next row, so they are pushed out of the descriptor.
    const bool ok = (k0 + ld_kc) < K;
    const uint32_t base = ok ? ld_off + (uint32_t)k0 : OOB_OFFSET;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) ra[i] = buffer_load_16(Ar, ok ? base + i * row32 : OOB_OFFSET);
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) rb[i] = buffer_load_16(Br, ok ? base + i * row32 : OOB_OFFSET);
  };
  const int lds_st = ld_row * PITCH + ld_kc;
  auto lstore = [&](int buf) {
    uint8_t* a = sA0 + buf * STAGE + lds_st;
    uint8_t* b = sB0 + buf * STAGE + lds_st;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) *reinterpret_cast<uint4*>(a + i * 32 * PITCH) = ra[i];
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) *reinterpret_cast<uint4*>(b + i * 32 * PITCH) = rb[i];
  };

  using acc_t = typename Acc<FP8>::type;
  acc_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  // fragment read offsets: lane -> row lane%32, k bytes (lane/32)*FRAG within a sub-step
  constexpr int FRAG = FP8 ? 32 : 16;  // bytes of K per lane per MFMA
  constexpr int KSUB = 2 * FRAG;       // K per MFMA: 32 (int8) or 64 (fp8)
  const int fr_a = (wave_m * WAVE_M + (lane & 31)) * PITCH + (lane >> 5) * FRAG;
  const int fr_b = (wave_n * WAVE_N + (lane & 31)) * PITCH + (lane >> 5) * FRAG;

  const int nk = (K + BK - 1) / BK;
  gload(0);
  lstore(0);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) gload((kt + 1) * BK);
    const uint8_t* a = sA0 + cur * STAGE + fr_a;
    const uint8_t* b = sB0 + cur * STAGE + fr_b;
#pragma unroll
    for (int ks = 0; ks < BK / KSUB; ++ks) {
      if constexpr (!FP8) {
        v4i af[TM], bf[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) af[i] = *reinterpret_cast<const v4i*>(a + i * 32 * PITCH + ks * KSUB);
#pragma unroll
        for (int j = 0; j < TN; ++j) bf[j] = *reinterpret_cast<const v4i*>(b + j * 32 * PITCH + ks * KSUB);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
      } else {
        v8i af[TM], bf[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const v4i lo = *reinterpret_cast<const v4i*>(a + i * 32 * PITCH + ks * KSUB);
          const v4i hi = *reinterpret_cast<const v4i*>(a + i * 32 * PITCH + ks * KSUB + 16);
          af[i] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const v4i lo = *reinterpret_cast<const v4i*>(b + j * 32 * PITCH + ks * KSUB);
          const v4i hi = *reinterpret_cast<const v4i*>(b + j * 32 * PITCH + ks * KSUB + 16);
          bf[j] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        }
        // E8M0 scale 127 = 2^0 for both operands: plain e4m3 x e4m3.
        const int one = 0x7f7f7f7f;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[i], bf[j], acc[i][j], 0, 0, 0,
                                                                        one, 0, one);
      }
    }
    if (kt + 1 < nk) lstore(cur ^ 1);
    __syncthreads();
  }

  // ---- epilogue.  32x32 accumulator: register r of lane l holds
  //      row (r/4)*8 + (l/32)*4 + r%4, column l%32.
  float sx1 = 1.0f, sw1 = 1.0f;
  if constexpr (FP8) {
    sx1 = *p.sx;
    sw1 = *p.sw;
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int n = n0 + wave_n * WAVE_N + j * 32 + (lane & 31);
    const bool n_ok = n < N;
    float swn = 1.0f, bn = 0.0f;
    bool has_bias = false;
    if constexpr (!FP8 && OUT != OUT_I32) {
      if (n_ok) {
        swn = p.sw[n];
        if (p.bias) {
          has_bias = true;
          bn = p.bias_dtype == AQ_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p.bias)[n])
                                       : reinterpret_cast<const float*>(p.bias)[n];
        }
      }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int mb = m0 + wave_m * WAVE_M + i * 32 + (lane >> 5) * 4;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = mb + (r >> 2) * 8 + (r & 3);
        if (m < M && n_ok) {
          const int64_t o = (int64_t)m * N + n;
          if constexpr (OUT == OUT_I32) {
            reinterpret_cast<int32_t*>(p.C)[o] = acc[i][j][r];
          } else {
            float y;
            if constexpr (FP8) {
              y = __fmul_rn(__fmul_rn(acc[i][j][r], sx1), sw1);
            } else {
              // three separately rounded fp32 operations, never contracted
              y = __fmul_rn(__fmul_rn((float)acc[i][j][r], p.sx[m]), swn);
              if (has_bias) y = __fadd_rn(y, bn);
            }
            if constexpr (OUT == OUT_F32)
              reinterpret_cast<float*>(p.C)[o] = y;
            else
              reinterpret_cast<uint16_t*>(p.C)[o] = (uint16_t)f32_to_bf16_bits(y);
          }
        }
      }
    }
  }
}

template <bool FP8, int OUT>
static int launch(const GemmArgs& a, hipStream_t st) {
  const unsigned grid = (unsigned)(a.tiles_m * a.tiles_n);
  hipLaunchKernelGGL((gemm_kernel<FP8, OUT>), dim3(grid), dim3(256), 0, st, a);
  return (int)hipGetLastError();
}

static int check_gemm(const void* A, const void* B, const void* C, int64_t M, int64_t N, int64_t K) {
  if (M < 0 || N < 0 || K <= 0 || (K % 16) != 0) return AQ_E_SHAPE;
  if (M == 0 || N == 0) return AQ_OK;
  if (!A || !B || !C) return AQ_E_NULL;
  if (check_ptr16(A) || check_ptr16(B) || check_ptr16(C)) return AQ_E_ALIGN;
  // 32-bit tile-relative offsets: 256 rows * K bytes must fit an int
  if (K > (1 << 22) || M > (1 << 30) || N > (1 << 30)) return AQ_E_RANGE;
  if (((M + BM - 1) / BM) * ((N + BN - 1) / BN) > (int64_t)0x7fffffff) return AQ_E_RANGE;
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
  a.tiles_m = (int)((M + BM - 1) / BM);
  a.tiles_n = (int)((N + BN - 1) / BN);
  return a;
}

}  // namespace aq

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
  if (y_dtype != AQ_F32 && y_dtype != AQ_BF16) return AQ_E_DTYPE;
  if (bias && bias_dtype != AQ_F32 && bias_dtype != AQ_BF16) return AQ_E_DTYPE;
  int rc = aq::check_gemm(xq, wq, y, M, N, K);
  if (rc || M == 0 || N == 0) return rc;
  if (!sx || !sw) return AQ_E_NULL;
  aq::GemmArgs a = aq::make_args(xq, wq, y, M, N, K);
  a.sx = sx;
  a.sw = sw;
  a.bias = bias;
  a.bias_dtype = bias_dtype;
  hipStream_t st = static_cast<hipStream_t>(stream);
  return y_dtype == AQ_BF16 ? aq::launch<false, aq::OUT_BF16>(a, st) : aq::launch<false, aq::OUT_F32>(a, st);
}

extern "C" int aq_linear_fp8(const uint8_t* xq, const float* sx, const uint8_t* wq, const float* sw,
                             void* y, int y_dtype, int64_t M, int64_t N, int64_t K, void* stream) {
  if (y_dtype != AQ_F32 && y_dtype != AQ_BF16) return AQ_E_DTYPE;
  int rc = aq::check_gemm(xq, wq, y, M, N, K);
  if (rc || M == 0 || N == 0) return rc;
  if (!sx || !sw) return AQ_E_NULL;
  aq::GemmArgs a = aq::make_args(xq, wq, y, M, N, K);
  a.sx = sx;
  a.sw = sw;
  hipStream_t st = static_cast<hipStream_t>(stream);
  return y_dtype == AQ_BF16 ? aq::launch<true, aq::OUT_BF16>(a, st) : aq::launch<true, aq::OUT_F32>(a, st);
}
