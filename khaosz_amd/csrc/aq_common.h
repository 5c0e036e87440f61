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

// Maximum of a non-negative value over the 64 lanes, returned in every lane
// (as a wavefront-uniform scalar).  Four DPP steps (quad swaps, then the
// half-row and row mirrors) leave each row of 16 lanes holding its maximum;
// the four row results are read out and combined on the scalar unit, where
// non-negative floats order like their bit patterns.
__device__ __forceinline__ float wave_max(float v) {
  int x = __float_as_int(v);
#define AQ_DPP_MAX(ctrl)                                                                      \
  x = __float_as_int(fmaxf(__int_as_float(x),                                                 \
                           __int_as_float(__builtin_amdgcn_update_dpp(x, x, ctrl, 0xf, 0xf, false))))
  AQ_DPP_MAX(0xB1);   // quad_perm [1,0,3,2]
  AQ_DPP_MAX(0x4E);   // quad_perm [2,3,0,1]
  AQ_DPP_MAX(0x141);  // row_half_mirror
  AQ_DPP_MAX(0x140);  // row_mirror
#undef AQ_DPP_MAX
  const uint32_t a = (uint32_t)__builtin_amdgcn_readlane(x, 0), b = (uint32_t)__builtin_amdgcn_readlane(x, 16);
  const uint32_t c = (uint32_t)__builtin_amdgcn_readlane(x, 32), d = (uint32_t)__builtin_amdgcn_readlane(x, 48);
  const uint32_t ab = a > b ? a : b, cd = c > d ? c : d;
  return __uint_as_float(ab > cd ? ab : cd);
}

// Exact definition: q = clamp(rint(a / s), -127, 127), correctly rounded divide,
// round-half-to-even.  Returned as a 32-bit pattern whose low byte is the code.
__device__ __forceinline__ uint32_t quant_code_exact(float a, float s) {
  float n = rintf(__fdiv_rn(a, s));
  n = fminf(fmaxf(n, -127.0f), 127.0f);
  return (uint32_t)(int)n;
}

// The same codes for N values of one row without the range handling of a
// general divide.  With STEPS = 2, rs must be the once-refined reciprocal of s,
//   y0 = rcp(s), rs = fma(fma(-s, y0, 1), y0, y0),
// and then   q0 = a * rs,  q1 = fma(fma(-s, q0, a), rs, q0),  q2 = fma(fma(-s, q1, a), rs, q1)
// is, operation for operation, the sequence the compiler emits for a correctly
// rounded fp32 divide once its operands are in range (its scaling and fix-up
// steps are the identity there): q2 = fl(a / s).  Adding 1.5 * 2^23 rounds q2 to
// the nearest-even integer n and leaves it in the low mantissa bits, so the low
// byte of the sum IS the two's-complement code; |a| never exceeds the row's
// amax = 127 s, so no clamp is needed.  No branch, no per-value fallback: bf16
// inputs hit exact ties (a = amax / 2 ...) once in 400 values, which makes any
// "fast path unless near a tie" scheme take its slow path in most wavefronts.
// With STEPS = 1, for values that ARE bf16 numbers (8 significant bits, and so is
// their row maximum): rs must be the correctly rounded reciprocal fl(1 / s), and
// the first correction alone, q1 = fma(fma(-s, q0, a), rs, q0), already rounds
// to the same integer as fl(a / s) for every pair (row maximum, value) of bf16
// numbers with |value| <= maximum and s = fl(maximum / 127) in range -- 2.8e8
// pairs, evaluated one by one on the CPU with the same IEEE operations
// (oq_one_step_divide_mismatches in the oracle and the test that runs it).
// With STEPS = 0, for the int8 codes of such rows: no correction at all, q0 = a * rs rounds to the same integer
// as fl(a / s) for every value of the row, PROVIDED rs is fl(1 / s) moved by at most one unit in the last place
// in a direction that depends on the 7 mantissa bits of the row maximum alone (reciprocal_for_bf16_rows below:
// 104 of the 128 mantissas keep fl(1 / s), 18 take the next float up, 6 the next one down; which is which was found
// by trying all three for every maximum, and the choice does not depend on the exponent).  The claim is evaluated
// for every pair like the one above (oq_one_step_divide_mismatches with steps = -1, on the oracle's own copy of the
// table) and on the shipped kernels over every value of rows with every mantissa.
// `lean_ok` must be false for rows whose scale is outside [2^-64, 2^64], where
// the residuals could leave the normal range; those rows take the full divide.
//
// Two bits per mantissa of the row maximum (mantissa m in bits 2 (m % 16) of word m / 16): 0 keep fl(1 / s), 1 one
// unit up, 2 one unit down.
__device__ __forceinline__ float reciprocal_for_bf16_rows(float amax, float s) {
  const uint32_t m = (__float_as_uint(amax) >> 16) & 127u;
  const uint32_t i = m >> 4;
  const uint32_t w = (i & 4u) ? ((i & 2u) ? ((i & 1u) ? 0x00000105u : 0x40000004u) : ((i & 1u) ? 0x40014442u : 0x00000000u))
                              : ((i & 2u) ? ((i & 1u) ? 0x10004480u : 0x80000000u) : ((i & 1u) ? 0x05015a02u : 0x00000000u));
  const uint32_t adj = (w >> (2u * (m & 15u))) & 3u;
  return __uint_as_float(__float_as_uint(__fdiv_rn(1.0f, s)) + (adj & 1u) - (adj >> 1));
}

template <int N, int STEPS = 2>
__device__ __forceinline__ void quant_codes(const float* a, float s, float rs, bool lean_ok, uint32_t* out) {
  const float magic = 12582912.0f;  // 1.5 * 2^23
  if (__builtin_expect(lean_ok, 1)) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      float q = a[i] * rs;
      if constexpr (STEPS >= 1) q = __builtin_fmaf(__builtin_fmaf(-s, q, a[i]), rs, q);
      if constexpr (STEPS == 2) q = __builtin_fmaf(__builtin_fmaf(-s, q, a[i]), rs, q);
      out[i] = __float_as_uint(q + magic);
    }
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) out[i] = quant_code_exact(a[i], s);
  }
}

// exp(x) for |x| <= 87 from operations that round identically on every IEEE
// machine (products, fused multiply-adds, rint, an exponent-field add), so that
// the CPU oracle reproduces it bit for bit; library exponentials differ in their
// last bits between implementations.  n = rint(x log2 e), r = x - n ln 2 in two
// pieces, e^r = 1 + r + r^2 P(r) with the classic degree-5 minimax P (error below
// 2 ulp), scaled by 2^n through the exponent field.
template <bool CLAMP = true>
__device__ __forceinline__ float exp_repro(float x) {
  if constexpr (CLAMP) x = fminf(fmaxf(x, -87.0f), 87.0f);  // CLAMP = false: the caller knows |x| <= 87
  const float n = rintf(__fmul_rn(x, 1.44269504088896341f));
  float r = __builtin_fmaf(n, -0.693359375f, x);
  r = __builtin_fmaf(n, 2.12194440e-4f, r);
  float p = 1.9875691500e-4f;
  p = __builtin_fmaf(p, r, 1.3981999507e-3f);
  p = __builtin_fmaf(p, r, 8.3334519073e-3f);
  p = __builtin_fmaf(p, r, 4.1665795894e-2f);
  p = __builtin_fmaf(p, r, 1.6666665459e-1f);
  p = __builtin_fmaf(p, r, 5.0000001201e-1f);
  const float y = __fadd_rn(__builtin_fmaf(p, __fmul_rn(r, r), r), 1.0f);
  return __int_as_float(__float_as_int(y) + ((int)n << 23));
}

// SwiGLU on fp32 values: u * (g / (1 + exp(-g))), a correctly rounded divide and one product.
__device__ __forceinline__ float swiglu_repro(float u, float g) {
  return __fmul_rn(u, __fdiv_rn(g, __fadd_rn(1.0f, exp_repro(-g))));
}

// n / d, correctly rounded, for operands in the middle of the range: the compiler's own sequence for an fp32
// divide (hardware reciprocal, one refinement, quotient, two residual corrections) without the scaling of
// extreme operands in front (v_div_scale) and the special-case selection behind (v_div_fixup) -- both the
// identity when 2^-62 <= |n|, |d| <= 2^62, where no intermediate leaves the normal range.  11 instead of 14
// operation slots (the reciprocal counts four).
__device__ __forceinline__ float div_midrange(float n, float d) {
  const float y0 = __builtin_amdgcn_rcpf(d);
  const float y = __builtin_fmaf(__builtin_fmaf(-d, y0, 1.0f), y0, y0);
  float q = n * y;
  q = __builtin_fmaf(__builtin_fmaf(-d, q, n), y, q);
  return __builtin_fmaf(__builtin_fmaf(-d, q, n), y, q);
}

// The same quotient two operation slots cheaper, for ONE family of operands only: n = g and d = 1 + exp_repro(-g)
// with g a bf16 number the test below lets through.  The quotient corrections use the hardware reciprocal as it
// comes (no refinement of it).  For general operands that is only almost always the correctly rounded quotient; for
// this family there are fewer than 65536 operand pairs, one per gate, and every one of them goes through the shipped
// kernel against the CPU oracle's true divide in the tests (all bf16 gate patterns, bit for bit).
__device__ __forceinline__ float div_bf16_gate(float n, float d) {
  const float y = __builtin_amdgcn_rcpf(d);
  float q = n * y;
  q = __builtin_fmaf(__builtin_fmaf(-d, q, n), y, q);
  return __builtin_fmaf(__builtin_fmaf(-d, q, n), y, q);
}

// The gates div_midrange may be used for: zero (0 / d = 0, with a sign that no code and no maximum depends on) or
// 2^-62 <= |g| <= 80, so that 1 + exp(-g) < 2^116 and every intermediate of the short divide stays a normal
// number.  Exact zeros must pass: rows of real bf16 activations hold a few per ten million values, and a row sent
// through the general divide takes three times as long as its neighbours and holds up the launch.
// For bf16 gates the test runs on the raw pairs with packed 16-bit integer operations, two gates per operation:
// |g| as a 16-bit pattern orders like the number; pattern - 1 wraps a zero to 0xffff, above every bound.
struct GateRangeBf16 {
  typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
  u16x2 lo = {0xffff, 0xffff}, hi = {0, 0};
  __device__ __forceinline__ void add(uint32_t pair) {
    const uint32_t a = pair & 0x7fff7fffu;
    const u16x2 av = __builtin_bit_cast(u16x2, a);
    lo = __builtin_elementwise_min(lo, av - (u16x2){1, 1});
    hi = __builtin_elementwise_max(hi, av);
  }
  __device__ __forceinline__ void add(const uint4& v) {
    add(v.x);
    add(v.y);
    add(v.z);
    add(v.w);
  }
  __device__ __forceinline__ bool ok() const {
    const unsigned l = lo.x < lo.y ? lo.x : lo.y, h = hi.x > hi.y ? hi.x : hi.y;
    return l >= 0x2080u - 1u && h <= 0x42a0u;  // bf16 patterns of 2^-62 and 80
  }
};
// the same test on fp32 gates
template <int N>
__device__ __forceinline__ bool gates_midrange(const float* g) {
  float lo = 1.0f, hi = 0.0f;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const float a = fabsf(g[i]);
    lo = fminf(lo, a == 0.0f ? 1.0f : a);
    hi = fmaxf(hi, a);
  }
  return lo >= 2.168404344971009e-19f && hi <= 80.0f;  // 2^-62
}

// SwiGLU of N pairs with div_midrange: the bits of swiglu_repro when the gates pass the test above (zeros aside).
// Four chains at a time: enough to cover the arithmetic's latency, few enough temporaries for a caller to keep a
// whole row of h in registers next to them.
// CLAMP = false drops the exponential's own argument clamp, the identity for such gates (|g| <= 80 < 87): one
// operation less per product where the vector ALU is the bound (4096 x 5632: 27.9 -> 27.1 us); the one-row-per-
// workgroup kernel, which is not, measured 0.2 us slower without it and keeps it.
// BF16_GATES: the gates are bf16 numbers, for which div_bf16_gate is certified.
template <int N, bool CLAMP = true, bool BF16_GATES = false>
__device__ __forceinline__ void swiglu_group_midrange(const float* u, const float* g, float* h) {
#pragma unroll
  for (int i = 0; i < N; ++i) {
    if (i > 0 && (i & 3) == 0) __builtin_amdgcn_sched_barrier(0);
    const float d = __fadd_rn(1.0f, exp_repro<CLAMP>(-g[i]));
    h[i] = __fmul_rn(u[i], BF16_GATES ? div_bf16_gate(g[i], d) : div_midrange(g[i], d));
  }
}

// low bytes of four 32-bit patterns -> one dword (a in bits 7:0 .. d in bits 31:24)
__device__ __forceinline__ uint32_t pack_low_bytes(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  const uint32_t ab = __builtin_amdgcn_perm(b, a, 0x0c0c0400u);  // {a.b0, b.b0, 0, 0}
  const uint32_t cd = __builtin_amdgcn_perm(d, c, 0x0c0c0400u);
  return __builtin_amdgcn_perm(cd, ab, 0x05040100u);             // {ab.b0, ab.b1, cd.b0, cd.b1}
}

// quant_codes with the N codes delivered packed, four to a dword (code i in byte i % 4 of out[i / 4]).  On the lean
// path the rounding add writes its low byte -- which IS the code -- straight into its byte of the result
// (v_add_f32 in its sub-dword-addressing form, destination byte selected, the other bytes kept), so rounding and
// packing cost one operation per value instead of one and three quarters.  This part wants one instruction (or
// one idle slot) between such a write and the next instruction that touches the same register; the compiler does
// not see inside the statement, so the slots are written out: two dwords are filled alternately where there are
// eight values, and a pause closes the sequence.
template <int N, int STEPS = 2>
__device__ __forceinline__ void quant_codes_packed(const float* a, float s, float rs, bool lean_ok, uint32_t* out) {
  static_assert(N == 4 || N == 8, "one or two dwords of codes");
  const float magic = 12582912.0f;  // 1.5 * 2^23
  if (__builtin_expect(lean_ok, 1)) {
    float q[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
      q[i] = a[i] * rs;
      if constexpr (STEPS >= 1) q[i] = __builtin_fmaf(__builtin_fmaf(-s, q[i], a[i]), rs, q[i]);
      if constexpr (STEPS == 2) q[i] = __builtin_fmaf(__builtin_fmaf(-s, q[i], a[i]), rs, q[i]);
    }
    if constexpr (N == 8) {
      uint32_t r0 = __float_as_uint(q[0] + magic), r1 = __float_as_uint(q[4] + magic);
      asm("v_add_f32_sdwa %0, %2, %8 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD\n\t"
          "v_add_f32_sdwa %1, %5, %8 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD\n\t"
          "v_add_f32_sdwa %0, %3, %8 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD\n\t"
          "v_add_f32_sdwa %1, %6, %8 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD\n\t"
          "v_add_f32_sdwa %0, %4, %8 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD\n\t"
          "v_add_f32_sdwa %1, %7, %8 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD\n\t"
          "s_nop 0"
          : "+v"(r0), "+v"(r1)
          : "v"(q[1]), "v"(q[2]), "v"(q[3]), "v"(q[5]), "v"(q[6]), "v"(q[7]), "v"(magic));
      out[0] = r0;
      out[1] = r1;
    } else {
      uint32_t r0 = __float_as_uint(q[0] + magic);
      asm("v_add_f32_sdwa %0, %1, %4 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD\n\t"
          "s_nop 0\n\t"
          "v_add_f32_sdwa %0, %2, %4 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD\n\t"
          "s_nop 0\n\t"
          "v_add_f32_sdwa %0, %3, %4 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD\n\t"
          "s_nop 0"
          : "+v"(r0)
          : "v"(q[1]), "v"(q[2]), "v"(q[3]), "v"(magic));
      out[0] = r0;
    }
  } else {
    uint32_t c[N];
#pragma unroll
    for (int i = 0; i < N; ++i) c[i] = quant_code_exact(a[i], s);
#pragma unroll
    for (int i = 0; i < N / 4; ++i) out[i] = pack_low_bytes(c[4 * i], c[4 * i + 1], c[4 * i + 2], c[4 * i + 3]);
  }
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
// the same load marked as streaming (nt): data that is read exactly once, such as a decode step's weights
__device__ __forceinline__ uint4 buffer_load_16_stream(__amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
  v4i v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 2);
  return make_uint4((uint32_t)v.x, (uint32_t)v.y, (uint32_t)v.z, (uint32_t)v.w);
}
constexpr uint32_t OOB_OFFSET = 0x7ffffff0u;  // beyond every descriptor built here

// Write-through stores for bulk outputs.  With the default write-back policy
// the dirty lines of a kernel's output sit in its XCD's L2 until the end-of-
// kernel release writes them all back at once, after the last wavefront has
// finished; written through, they drain while the rest of the kernel still
// runs (measured: 1.9 us of a 21.4 us GEMM with a 16 MB output).
// STORE_WT is the cache-policy operand of the buffer-store builtins (sc0 | sc1).
#ifndef AQ_STORE_WT
#define AQ_STORE_WT 17
#endif
constexpr int STORE_WT = AQ_STORE_WT;
__device__ __forceinline__ void store_wt(uint32_t* p, uint32_t v) {
#if AQ_STORE_WT
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
#else
  *p = v;
#endif
}
__device__ __forceinline__ void store_wt(uint2* p, uint2 v) {
#if AQ_STORE_WT
  __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), ((unsigned long long)v.y << 32) | v.x, __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_SYSTEM);
#else
  *p = v;
#endif
}

inline int check_ptr16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) ? AQ_E_ALIGN : AQ_OK; }
inline int check_ptr(const void* p, unsigned align) { return (reinterpret_cast<uintptr_t>(p) & (align - 1u)) ? AQ_E_ALIGN : AQ_OK; }

// Compute units of the current device, asked of the runtime once per device (launch shapes are
// sized by it: a partition mode that exposes fewer compute units per device gets fewer workgroups).
// The cache is written with the same value by whichever thread comes first: a benign race.
inline int device_cus() {
  static int cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int v = cached[dev];
  if (v <= 0) {
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
    cached[dev] = v;
  }
  return v;
}

}  // namespace aq
