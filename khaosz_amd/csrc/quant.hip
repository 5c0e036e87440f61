// Activation / weight quantisation kernels for gfx950: symmetric absmax int8
// per row and per-tensor FP8 (OCP e4m3fn).  Both are HBM-bound streaming
// kernels: 16-byte loads per lane, one wavefront per row, wavefront-wide
// absmax through cross-lane shuffles, no LDS.
#include "aq_common.h"

namespace aq {

// ---------------------------------------------------------------- int8 rows

template <bool BF16>
struct RowIn;
template <>
struct RowIn<true> {  // 8 bf16 per 16-byte vector
  static constexpr int EPV = 8;
  __device__ static __forceinline__ void unpack(const uint4& v, float* f) {
    f[0] = __uint_as_float(v.x << 16);
    f[1] = __uint_as_float(v.x & 0xffff0000u);
    f[2] = __uint_as_float(v.y << 16);
    f[3] = __uint_as_float(v.y & 0xffff0000u);
    f[4] = __uint_as_float(v.z << 16);
    f[5] = __uint_as_float(v.z & 0xffff0000u);
    f[6] = __uint_as_float(v.w << 16);
    f[7] = __uint_as_float(v.w & 0xffff0000u);
  }
};
template <>
struct RowIn<false> {  // 4 fp32 per 16-byte vector
  static constexpr int EPV = 4;
  __device__ static __forceinline__ void unpack(const uint4& v, float* f) {
    f[0] = __uint_as_float(v.x);
    f[1] = __uint_as_float(v.y);
    f[2] = __uint_as_float(v.z);
    f[3] = __uint_as_float(v.w);
  }
};

template <int EPV>
__device__ __forceinline__ float vec_amax(const float* f) {
  float m = 0.0f;
#pragma unroll
  for (int i = 0; i < EPV; ++i) m = fmaxf(m, fabsf(f[i]));
  return m;
}

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
  return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) | ((uint32_t)(c & 0xff) << 16) |
         ((uint32_t)(d & 0xff) << 24);
}

template <bool BF16>
__device__ __forceinline__ void quant_store(const uint4& v, float s, float rs, int8_t* dst) {
  float f[RowIn<BF16>::EPV];
  RowIn<BF16>::unpack(v, f);
  if constexpr (BF16) {
    uint2 o;
    o.x = pack4(quant_code(f[0], s, rs), quant_code(f[1], s, rs), quant_code(f[2], s, rs),
                quant_code(f[3], s, rs));
    o.y = pack4(quant_code(f[4], s, rs), quant_code(f[5], s, rs), quant_code(f[6], s, rs),
                quant_code(f[7], s, rs));
    *reinterpret_cast<uint2*>(dst) = o;
  } else {
    *reinterpret_cast<uint32_t*>(dst) = pack4(quant_code(f[0], s, rs), quant_code(f[1], s, rs),
                                              quant_code(f[2], s, rs), quant_code(f[3], s, rs));
  }
}

// One wavefront per row.  The first NC vectors of the lane stay in registers
// between the absmax pass and the rounding pass; longer rows are re-read
// (from L2) for the part that does not fit.
template <bool BF16, int NC>
__global__ __launch_bounds__(256) void quant_rowwise_i8_kernel(const void* __restrict__ x, int64_t M,
                                                                 int K, int64_t ldx,
                                                                 int8_t* __restrict__ q,
                                                                 float* __restrict__ scale) {
  constexpr int EPV = RowIn<BF16>::EPV;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const int nvec = K / EPV;  // 16-byte vectors per row
  const uint4* src =
      reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(x) + row * ldx * (BF16 ? 2 : 4));
  int8_t* dst = q + row * (int64_t)K;

  uint4 cache[NC];
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int v = i * 64 + lane;
    if (v < nvec) {
      cache[i] = src[v];
      float f[EPV];
      RowIn<BF16>::unpack(cache[i], f);
      amax = fmaxf(amax, vec_amax<EPV>(f));
    }
  }
  for (int v = NC * 64 + lane; v < nvec; v += 64) {
    float f[EPV];
    RowIn<BF16>::unpack(src[v], f);
    amax = fmaxf(amax, vec_amax<EPV>(f));
  }
  amax = wave_max(amax);
  float s = __fdiv_rn(amax, 127.0f);
  if (amax == 0.0f) s = 1.0f;
  const float rs = __builtin_amdgcn_rcpf(s);
  if (lane == 0) scale[row] = s;
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int v = i * 64 + lane;
    if (v < nvec) quant_store<BF16>(cache[i], s, rs, dst + (int64_t)v * EPV);
  }
  for (int v = NC * 64 + lane; v < nvec; v += 64) quant_store<BF16>(src[v], s, rs, dst + (int64_t)v * EPV);
}

// ---------------------------------------------------------------- FP8 tensor

__global__ void fill_u32_kernel(uint32_t* p, uint32_t v) {
  if (threadIdx.x == 0 && blockIdx.x == 0) *p = v;
}

template <bool BF16>
__global__ __launch_bounds__(256) void amax_kernel(const void* __restrict__ x, int64_t nvec,
                                                    uint32_t* __restrict__ amax_bits) {
  constexpr int EPV = RowIn<BF16>::EPV;
  const uint4* src = reinterpret_cast<const uint4*>(x);
  float amax = 0.0f;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < nvec; v += stride) {
    float f[EPV];
    RowIn<BF16>::unpack(src[v], f);
    amax = fmaxf(amax, vec_amax<EPV>(f));
  }
  amax = wave_max(amax);
  // |x| >= 0, so the IEEE bit patterns order like unsigned integers.
  if ((threadIdx.x & 63) == 0 && amax > 0.0f) atomicMax(amax_bits, __float_as_uint(amax));
}

__device__ __forceinline__ float fp8_prescale(float a, float s) {
  float v = __fdiv_rn(a, s);
  return fminf(fmaxf(v, -448.0f), 448.0f);
}

template <bool BF16>
__global__ __launch_bounds__(256) void cast_fp8_kernel(const void* __restrict__ x, int64_t nvec,
                                                        const uint32_t* __restrict__ amax_bits,
                                                        uint8_t* __restrict__ q,
                                                        float* __restrict__ scale) {
  constexpr int EPV = RowIn<BF16>::EPV;
  const float amax = __uint_as_float(*amax_bits);
  float s = __fdiv_rn(amax, 448.0f);
  if (amax == 0.0f) s = 1.0f;
  if (blockIdx.x == 0 && threadIdx.x == 0) *scale = s;
  const uint4* src = reinterpret_cast<const uint4*>(x);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < nvec; v += stride) {
    float f[EPV];
    RowIn<BF16>::unpack(src[v], f);
#pragma unroll
    for (int i = 0; i < EPV; ++i) f[i] = fp8_prescale(f[i], s);
    // v_cvt_pk_fp8_f32: two fp32 -> two OCP e4m3fn codes, round to nearest even.
    int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false);
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w0, true);
    if constexpr (BF16) {
      int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], 0, false);
      w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], w1, true);
      uint2 o;
      o.x = (uint32_t)w0;
      o.y = (uint32_t)w1;
      *reinterpret_cast<uint2*>(q + v * EPV) = o;
    } else {
      *reinterpret_cast<uint32_t*>(q + v * EPV) = (uint32_t)w0;
    }
  }
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
  const unsigned grid = (unsigned)((M + 3) / 4);
  if (x_dtype == AQ_BF16)
    hipLaunchKernelGGL((aq::quant_rowwise_i8_kernel<true, 16>), dim3(grid), dim3(256), 0, st, x, M,
                       (int)K, ldx, q, scale);
  else
    hipLaunchKernelGGL((aq::quant_rowwise_i8_kernel<false, 16>), dim3(grid), dim3(256), 0, st, x, M,
                       (int)K, ldx, q, scale);
  return (int)hipGetLastError();
}

extern "C" int aq_quant_tensor_fp8(const void* x, int x_dtype, int64_t numel, uint8_t* q,
                                   float* scale, uint32_t* amax_ws, void* stream) {
  if (x_dtype != AQ_F32 && x_dtype != AQ_BF16) return AQ_E_DTYPE;
  if (numel < 0 || (numel % 16) != 0) return AQ_E_SHAPE;
  if (!scale || !amax_ws) return AQ_E_NULL;
  if (numel > 0 && (!x || !q)) return AQ_E_NULL;
  if (aq::check_ptr16(x) || aq::check_ptr16(q)) return AQ_E_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int epv = x_dtype == AQ_BF16 ? 8 : 4;
  const int64_t nvec = numel / epv;
  int64_t blocks = (nvec + 255) / 256;
  if (blocks > 2048) blocks = 2048;  // 8 workgroups per CU, grid-stride beyond
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(aq::fill_u32_kernel, dim3(1), dim3(64), 0, st, amax_ws, 0u);
  if (x_dtype == AQ_BF16) {
    hipLaunchKernelGGL((aq::amax_kernel<true>), dim3((unsigned)blocks), dim3(256), 0, st, x, nvec, amax_ws);
    hipLaunchKernelGGL((aq::cast_fp8_kernel<true>), dim3((unsigned)blocks), dim3(256), 0, st, x, nvec,
                       amax_ws, q, scale);
  } else {
    hipLaunchKernelGGL((aq::amax_kernel<false>), dim3((unsigned)blocks), dim3(256), 0, st, x, nvec, amax_ws);
    hipLaunchKernelGGL((aq::cast_fp8_kernel<false>), dim3((unsigned)blocks), dim3(256), 0, st, x, nvec,
                       amax_ws, q, scale);
  }
  return (int)hipGetLastError();
}
