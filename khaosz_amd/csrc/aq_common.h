// Shared device helpers for the gfx950 quantized-Linear kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/astrai_q.h"

// Results are compared bit for bit with a CPU restatement that rounds every
// fp32 operation separately, so a*b+c must never be contracted into an FMA
// (__fmul_rn / __fadd_rn are plain operators in HIP and do not prevent it).
#pragma clang fp contract(off)

#define AQ_WAVE 64

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

namespace aq {

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// fp32 -> bf16 bit pattern, round to nearest even (NaN stays quiet NaN).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
  if ((u & 0x7fffffffu) > 0x7f800000u) r = (u >> 16) | 0x40u;
  return r & 0xffffu;
}

// two fp32 -> packed bf16 pair (lo in bits 15:0) with the hardware converter
// (v_cvt_pk_bf16_f32: round to nearest even, NaN stays NaN).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef float f2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  const f2 v = {lo, hi};
  const bf2 b = __builtin_convertvector(v, bf2);
  return *reinterpret_cast<const uint32_t*>(&b);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, AQ_WAVE));
  return v;
}

// q = clamp(rint(a / s), -127, 127) with a correctly rounded divide.
// Fast path: a * (1/s) is within 127 * 3 ulp of the true quotient, so whenever
// it is further than 2^-6 from a rounding boundary the rounded integer is
// already decided; only the rare near-tie lanes pay for the IEEE divide.
__device__ __forceinline__ int quant_code(float a, float s, float rs) {
  float t = a * rs;
  float n = rintf(t);
  float d = fabsf(t - n);
  if (__builtin_expect(!(d <= 0.484375f), 0)) n = rintf(__fdiv_rn(a, s));  // also taken for inf/NaN
  n = fminf(fmaxf(n, -127.0f), 127.0f);
  return (int)n;
}

// Raw buffer descriptor over [base, base + bytes): loads whose byte offset
// falls outside return zero, which is how tile edges are handled without
// branches.  0x00020000 is the gfx9 32-bit data-format dword.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ uint4 buffer_load_16(__amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
  v4i v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 0);
  return make_uint4((uint32_t)v.x, (uint32_t)v.y, (uint32_t)v.z, (uint32_t)v.w);
}
constexpr uint32_t OOB_OFFSET = 0x7ffffff0u;  // beyond every descriptor built here

inline int check_ptr16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) ? AQ_E_ALIGN : AQ_OK; }

}  // namespace aq
