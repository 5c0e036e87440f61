// Decode path (M <= 16 tokens): a weight-streaming int8 GEMV.  The weight
// matrix is read exactly once with 16-byte loads, one wavefront reading 1 KiB
// contiguous of a row per instruction; the few activation rows are quantised
// by the row-wise kernel into the caller's workspace, copied to LDS and reused
// by every row of W.  Products are v_dot4_i32_i8 (no MFMA tiles, no LDS
// staging of W); a wavefront reduces its 4 x MT partial sums with a transposed
// butterfly so that each lane ends up owning one output, then applies the same
// dequantising epilogue as the MFMA GEMM.  The int32 sums are exact, so the
// result is bit-identical to quantise + GEMM.
#include "aq_common.h"

namespace aq {

constexpr int GV_ROWS = 4;        // weight rows per wavefront pass
constexpr int GV_WAVES = 4;       // wavefronts per workgroup
constexpr int GV_CHUNK = 64 * 16; // K bytes one wavefront covers per load

// Reduce V values per lane across the 64 lanes.  While more than one value is
// live, partners exchange halves (reduce-scatter); afterwards plain butterfly
// adds.  On return v[0] of lane l is the full sum of value index
// l >> (6 - log2 V).
template <int CUR, int OFF>
struct Butterfly {
  template <int V>
  __device__ static __forceinline__ void run(int (&v)[V], int lane) {
    if constexpr (CUR > 1) {
      constexpr int H = CUR / 2;
      const bool up = (lane & OFF) != 0;
#pragma unroll
      for (int i = 0; i < H; ++i) {
        const int lo = v[i], hi = v[i + H];
        const int send = up ? lo : hi;
        const int keep = up ? hi : lo;
        v[i] = keep + __shfl_xor(send, OFF, AQ_WAVE);
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
  const int8_t* xq;   // [M, K] codes (workspace)
  const float* sx;    // [M]
  const int8_t* wq;   // [N, K]
  const float* sw;    // [N]
  const void* bias;   // [N] or null
  void* y;            // [M, N]
  int M, N, K;
  int bias_dtype, y_dtype;
};

template <int MT>
__global__ __launch_bounds__(GV_WAVES * 64) void gemv_w8a8_kernel(GemvArgs p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t xs[];  // [MT][K]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int K = p.K, N = p.N, M = p.M;
  // wavefront-uniform first row, made scalar so the buffer descriptor lives in SGPRs
  const int n0 = __builtin_amdgcn_readfirstlane((blockIdx.x * GV_WAVES + wave) * GV_ROWS);

  // Issue the first weight loads before anything else: they are the long pole.
  // The descriptor spans this wavefront's rows only; rows past N and bytes
  // past K fall outside it and read as zero.
  const int nchunk = (K + GV_CHUNK - 1) / GV_CHUNK;
  const int rows = n0 < N ? ((N - n0) < GV_ROWS ? (N - n0) : GV_ROWS) : 0;
  const __amdgpu_buffer_rsrc_t Wr =
      make_rsrc(p.wq + (int64_t)(n0 < N ? n0 : 0) * K, (uint32_t)rows * (uint32_t)K);
  const uint4 zero = make_uint4(0, 0, 0, 0);
  auto wload = [&](int c, uint4 (&dst)[GV_ROWS]) {
    const int kb = c * GV_CHUNK + lane * 16;
    const bool ok = kb < K;  // past K the offset would alias the next row
#pragma unroll
    for (int r = 0; r < GV_ROWS; ++r)
      dst[r] = buffer_load_16(Wr, ok ? (uint32_t)r * (uint32_t)K + (uint32_t)kb : OOB_OFFSET);
  };
  uint4 w[GV_ROWS];
  wload(0, w);

  // activation codes -> LDS, rows >= M zero
  const int nvec_row = K / 16;
  for (int v = tid; v < MT * nvec_row; v += GV_WAVES * 64) {
    const int m = v / nvec_row;
    uint4 val = zero;
    if (m < M) val = reinterpret_cast<const uint4*>(p.xq)[v];
    reinterpret_cast<uint4*>(xs)[v] = val;
  }
  __syncthreads();

  int acc[GV_ROWS * MT];
#pragma unroll
  for (int i = 0; i < GV_ROWS * MT; ++i) acc[i] = 0;

  for (int c = 0; c < nchunk; ++c) {
    const int kb = c * GV_CHUNK + lane * 16;
    uint4 wn[GV_ROWS];
    if (c + 1 < nchunk) {
      wload(c + 1, wn);
    } else {
#pragma unroll
      for (int r = 0; r < GV_ROWS; ++r) wn[r] = zero;
    }
    const int kx = kb < K ? kb : 0;  // lanes past the end multiply zeros; keep the LDS read in range
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const uint4 x = *reinterpret_cast<const uint4*>(xs + m * K + kx);
#pragma unroll
      for (int r = 0; r < GV_ROWS; ++r) {
        int a = acc[r * MT + m];
        a = __builtin_amdgcn_sdot4((int)w[r].x, (int)x.x, a, false);
        a = __builtin_amdgcn_sdot4((int)w[r].y, (int)x.y, a, false);
        a = __builtin_amdgcn_sdot4((int)w[r].z, (int)x.z, a, false);
        a = __builtin_amdgcn_sdot4((int)w[r].w, (int)x.w, a, false);
        acc[r * MT + m] = a;
      }
    }
#pragma unroll
    for (int r = 0; r < GV_ROWS; ++r) w[r] = wn[r];
  }

  constexpr int V = GV_ROWS * MT;
  Butterfly<V, 32>::run(acc, lane);
  constexpr int SH = 6 - ilog2(V);
  if ((lane & ((1 << SH) - 1)) != 0) return;
  const int idx = lane >> SH;
  const int r = idx / MT, m = idx % MT;
  const int n = n0 + r;
  if (m >= M || n >= N) return;
  float y = __fmul_rn(__fmul_rn((float)acc[0], p.sx[m]), p.sw[n]);
  if (p.bias) {
    const float b = p.bias_dtype == AQ_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p.bias)[n])
                                            : reinterpret_cast<const float*>(p.bias)[n];
    y = __fadd_rn(y, b);
  }
  const int64_t o = (int64_t)m * N + n;
  if (p.y_dtype == AQ_BF16)
    reinterpret_cast<uint16_t*>(p.y)[o] = (uint16_t)f32_to_bf16_bits(y);
  else
    reinterpret_cast<float*>(p.y)[o] = y;
}

template <int MT>
static int launch_gemv(const GemvArgs& a, hipStream_t st) {
  const unsigned grid = (unsigned)((a.N + GV_ROWS * GV_WAVES - 1) / (GV_ROWS * GV_WAVES));
  const size_t lds = (size_t)MT * a.K;
  if (lds > 64 * 1024) {  // beyond the default dynamic-LDS limit: opt this kernel in (idempotent)
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_w8a8_kernel<MT>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  hipLaunchKernelGGL((gemv_w8a8_kernel<MT>), dim3(grid), dim3(GV_WAVES * 64), lds, st, a);
  return (int)hipGetLastError();
}

constexpr int64_t GV_MAX_LDS = 160 * 1024;  // LDS of one gfx950 CU

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace aq

extern "C" size_t aq_gemv_w8a8_workspace_bytes(int64_t M, int64_t K) {
  if (M < 0 || K < 0) return 0;
  return aq::align256((size_t)(M * K)) + aq::align256((size_t)M * sizeof(float));
}

static int gemv_check(const int8_t* wq, const float* sw, const void* bias, int bias_dtype, const void* y,
                      int y_dtype, int64_t M, int64_t N, int64_t K, int* mt_out) {
  if (y_dtype != AQ_F32 && y_dtype != AQ_BF16) return AQ_E_DTYPE;
  if (bias && bias_dtype != AQ_F32 && bias_dtype != AQ_BF16) return AQ_E_DTYPE;
  if (M < 0 || M > 16 || N < 0 || K <= 0 || (K % 16) != 0) return AQ_E_SHAPE;
  if (M == 0 || N == 0) return AQ_OK;
  if (!wq || !sw || !y) return AQ_E_NULL;
  if (aq::check_ptr16(wq)) return AQ_E_ALIGN;
  if (N > (1 << 30)) return AQ_E_RANGE;
  const int mt = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16;
  if ((int64_t)mt * K > aq::GV_MAX_LDS) return AQ_E_RANGE;
  *mt_out = mt;
  return AQ_OK;
}

static int gemv_dispatch(const aq::GemvArgs& a, int mt, hipStream_t st) {
  switch (mt) {
    case 1: return aq::launch_gemv<1>(a, st);
    case 2: return aq::launch_gemv<2>(a, st);
    case 4: return aq::launch_gemv<4>(a, st);
    case 8: return aq::launch_gemv<8>(a, st);
    default: return aq::launch_gemv<16>(a, st);
  }
}

extern "C" int aq_gemv_w8a8_codes(const int8_t* xq, const float* sx, const int8_t* wq, const float* sw,
                                  const void* bias, int bias_dtype, void* y, int y_dtype, int64_t M,
                                  int64_t N, int64_t K, void* stream) {
  int mt = 0;
  int rc = gemv_check(wq, sw, bias, bias_dtype, y, y_dtype, M, N, K, &mt);
  if (rc || M == 0 || N == 0) return rc;
  if (!xq || !sx) return AQ_E_NULL;
  if (aq::check_ptr16(xq)) return AQ_E_ALIGN;
  aq::GemvArgs a{};
  a.xq = xq;
  a.sx = sx;
  a.wq = wq;
  a.sw = sw;
  a.bias = bias;
  a.y = y;
  a.M = (int)M;
  a.N = (int)N;
  a.K = (int)K;
  a.bias_dtype = bias_dtype;
  a.y_dtype = y_dtype;
  return gemv_dispatch(a, mt, static_cast<hipStream_t>(stream));
}

extern "C" int aq_gemv_w8a8_decode(const void* x, int x_dtype, const int8_t* wq, const float* sw,
                                   const void* bias, int bias_dtype, void* y, int y_dtype, int64_t M,
                                   int64_t N, int64_t K, void* ws, size_t ws_bytes, void* stream) {
  if (x_dtype != AQ_F32 && x_dtype != AQ_BF16) return AQ_E_DTYPE;
  int mt = 0;
  int rc = gemv_check(wq, sw, bias, bias_dtype, y, y_dtype, M, N, K, &mt);
  if (rc || M == 0 || N == 0) return rc;
  if (!x || !ws) return AQ_E_NULL;
  if (aq::check_ptr16(x) || aq::check_ptr16(ws)) return AQ_E_ALIGN;
  if (ws_bytes < aq_gemv_w8a8_workspace_bytes(M, K)) return AQ_E_WORKSPACE;
  int8_t* xq = static_cast<int8_t*>(ws);
  float* sx = reinterpret_cast<float*>(static_cast<char*>(ws) + aq::align256((size_t)(M * K)));
  rc = aq_quant_rowwise_i8(x, x_dtype, M, K, K, xq, sx, stream);
  if (rc) return rc;
  return aq_gemv_w8a8_codes(xq, sx, wq, sw, bias, bias_dtype, y, y_dtype, M, N, K, stream);
}
