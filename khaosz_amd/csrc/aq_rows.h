// Row-wise int8 quantisation pieces shared by the stand-alone quantise kernels
// and the decode kernels that quantise their few activation rows themselves.
#pragma once
#include "aq_common.h"

namespace aq {

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

// Symmetric absmax scale of one row from its wavefront-wide maximum:
// s = amax / 127 (1 for an all-zero row), rs = the reciprocal of s in the form
// quant_codes<N, STEPS> expects (STEPS = 2: the once-refined hardware reciprocal;
// STEPS = 1: the correctly rounded one, a full divide once per row; STEPS = 0,
// rows of bf16 numbers: that one moved as the row maximum's mantissa asks), and
// whether s is in the range where the short sequence may be used.
struct RowScale {
  float s, rs;
  bool fast_ok;
};
template <int STEPS = 2>
__device__ __forceinline__ RowScale row_scale(float amax) {
  RowScale r;
  r.s = __fdiv_rn(amax, 127.0f);
  if (amax == 0.0f) r.s = 1.0f;
  if constexpr (STEPS == 0) {
    r.rs = reciprocal_for_bf16_rows(amax, r.s);
  } else if constexpr (STEPS == 1) {
    r.rs = __fdiv_rn(1.0f, r.s);
  } else {
    const float y0 = __builtin_amdgcn_rcpf(r.s);
    r.rs = __builtin_fmaf(__builtin_fmaf(-r.s, y0, 1.0f), y0, y0);
  }
  r.fast_ok = r.s >= 5.421010862427522e-20f && r.s <= 1.8446744073709552e19f;  // [2^-64, 2^64]
  return r;
}
// correction steps for rows that are read as they are (bf16 numbers: none) or computed in fp32 (two)
template <bool BF16, bool COMPUTED>
constexpr int quant_steps() { return BF16 && !COMPUTED ? 0 : 2; }

// Sum across the wavefront in a fixed order: p[l] += p[l ^ 1], ^2, ^4, ^8, ^16, ^32, every add
// rounded.  After the xor-1 and xor-2 steps a quad holds one value, after the half-row mirror a
// half row does, after the row mirror a row does: the mirrors pair the same partial sums as
// xor 4 and xor 8 would.
__device__ __forceinline__ float wave_sum_butterfly(float v) {
  v = __fadd_rn(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, false)));
  v = __fadd_rn(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, false)));
  v = __fadd_rn(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, false)));
  v = __fadd_rn(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, false)));
  v = __fadd_rn(v, __shfl_xor(v, 16, 64));
  v = __fadd_rn(v, __shfl_xor(v, 32, 64));
  return v;
}

// 1 / sqrt(mean(x^2) + eps) of a row from its sum of squares: correctly rounded divide, add,
// square root (sqrtf; the __fsqrt_rn intrinsic is the 1-ulp native root) and divide.
__device__ __forceinline__ float rms_scale(float ss, float k, float eps) {
  return __fdiv_rn(1.0f, sqrtf(__fadd_rn(__fdiv_rn(ss, k), eps)));
}

// One wavefront quantises RPW rows of the activation straight into LDS.
// Wavefront `wave` of `nwaves` owns rows wave, wave + nwaves, ...; a lane holds
// VPL 16-byte vectors per row (vector lane + 64*i), all requested by issue()
// before anything is waited for, so the caller can queue other loads behind
// them.  finish() reduces, rounds and writes the codes of row m to
// xs + m*pitch and its scale to sx[m]; rows >= M (up to MT) are zero-filled.
// With NORM the rows are RMS-normalised first, y = (x * r) * gamma with
// r = rms_scale(sum of squares in the fixed order: a lane adds the rounded
// squares of its vectors lane, lane + 64, ... in ascending order, elements in
// memory order, then the butterfly): the arithmetic of the stand-alone
// norm-and-quantise kernel, bit for bit.  gamma is requested by issue_gamma().
template <bool BF16, int RPW, int VPL>
struct RowsToLds {
  static constexpr int EPV = RowIn<BF16>::EPV;
  uint4 c[RPW][VPL];
  uint4 gv[VPL];

  __device__ __forceinline__ void issue_gamma(const void* gamma, int K, int lane) {
    const int nvec = K / EPV;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int v = i * 64 + lane;
      gv[i] = make_uint4(0, 0, 0, 0);
      if (v < nvec) gv[i] = reinterpret_cast<const uint4*>(gamma)[v];
    }
  }

  __device__ __forceinline__ void issue(const void* x, int M, int K, int64_t ldx, int wave, int nwaves, int lane) {
    const int nvec = K / EPV;
#pragma unroll
    for (int j = 0; j < RPW; ++j) {
      const int m = wave + j * nwaves;
      const uint4* src =
          reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(x) + (int64_t)m * ldx * (BF16 ? 2 : 4));
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        const int v = i * 64 + lane;
        c[j][i] = make_uint4(0, 0, 0, 0);
        if (m < M && v < nvec) c[j][i] = src[v];
      }
    }
  }

  // vector i of row j as the values to quantise
  template <bool NORM>
  __device__ __forceinline__ void values(int j, int i, float r, float* f) const {
    RowIn<BF16>::unpack(c[j][i], f);  // vectors past the row or of rows >= M are zero
    if constexpr (NORM) {
      float g[EPV];
      RowIn<BF16>::unpack(gv[i], g);
#pragma unroll
      for (int e = 0; e < EPV; ++e) f[e] = __fmul_rn(__fmul_rn(f[e], r), g[e]);
    }
  }

  template <bool NORM = false>
  __device__ __forceinline__ void finish(int M, int MT, int K, uint8_t* xs, int pitch, float* sx, int wave,
                                         int nwaves, int lane, float eps = 0.0f) {
    const int nvec = K / EPV;
#pragma unroll
    for (int j = 0; j < RPW; ++j) {
      const int m = wave + j * nwaves;
      if (m >= MT) continue;  // uniform
      float r = 1.0f;
      if constexpr (NORM) {
        float ss = 0.0f;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
          float f[EPV];
          RowIn<BF16>::unpack(c[j][i], f);
#pragma unroll
          for (int e = 0; e < EPV; ++e) ss = __fadd_rn(ss, __fmul_rn(f[e], f[e]));
        }
        r = rms_scale(wave_sum_butterfly(ss), (float)K, eps);
      }
      float amax = 0.0f;
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        float f[EPV];
        values<NORM>(j, i, r, f);
        amax = fmaxf(amax, vec_amax<EPV>(f));
      }
      constexpr int STEPS = quant_steps<BF16, NORM>();
      const RowScale rsc = row_scale<STEPS>(wave_max(amax));
      if (lane == 0 && m < M) sx[m] = rsc.s;
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        const int v = i * 64 + lane;
        if (v < nvec) {
          float f[EPV];
          uint32_t code[EPV / 4];
          values<NORM>(j, i, r, f);
          quant_codes_packed<EPV, STEPS>(f, rsc.s, rsc.rs, rsc.fast_ok, code);  // zero rows give zero codes
          uint8_t* dst = xs + m * pitch + v * EPV;
          if constexpr (BF16) {
            *reinterpret_cast<uint2*>(dst) = make_uint2(code[0], code[1]);
          } else {
            *reinterpret_cast<uint32_t*>(dst) = code[0];
          }
        }
      }
    }
  }
};

// Rows of a decode step's attention output taken straight from the attention kernel's per-slice partial
// results instead of from a merged bf16 tensor.  Layout [row][head][slice][D + 4] floats: D numerators,
// the slice's maximum (log2 domain), its denominator, 2 floats of padding.  Element k of row m belongs to
// head k / D.  issue() requests, for each of the lane's 16-byte output vectors, the 8 numerators and the
// (maximum, denominator) pair of every slice; merge() combines them with the arithmetic of the separate
// merge kernel (weights exp2(maximum - overall maximum), numerators and denominator accumulated by fma in
// slice order from zero, product with the denominator's reciprocal, rounded to bf16) and leaves the packed bf16 vectors where
// RowsToLds::issue() would have put the loaded ones, so the quantiser that follows sees the same bits.
// The two operations every place that combines attention slices shares (the merge kernel, the
// attention kernel's own single-slice output, AttnRows below), so that they give the same bits:
// a slice's weight 2^(its maximum - the overall maximum) and the reciprocal of the combined
// denominator, both the hardware's approximations (1 ulp), outputs = numerator * reciprocal.
__device__ __forceinline__ float attn_slice_weight(float m, float mm) { return __builtin_amdgcn_exp2f(m - mm); }
__device__ __forceinline__ float attn_inv_denominator(float den) { return __builtin_amdgcn_rcpf(den); }

template <int RPW, int VPL, int NSMAX>
struct AttnRows;
template <int RPW, int VPL>
struct AttnRows<RPW, VPL, 0> {};  // kernels that do not merge
template <int RPW, int VPL, int NSMAX>
struct AttnRows {
  uint4 num[RPW][VPL][NSMAX][2];
  float2 md[RPW][VPL][NSMAX];

  __device__ __forceinline__ void issue(const float* parts, int M, int K, int D, int NS, int wave, int nwaves,
                                        int lane) {
    const int nvec = K / 8, part = D + 4, dshift = D == 64 ? 6 : 7;
#pragma unroll
    for (int j = 0; j < RPW; ++j) {
      const int m = wave + j * nwaves;
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        const int v = i * 64 + lane, k = v * 8;
        const bool ok = m < M && v < nvec;
        // (row, head) index = (m * K + k) / D; rows and vectors that are not there read element 0
        const int64_t rh = ok ? ((int64_t)m * K + k) >> dshift : 0;
        const float* src = parts + rh * NS * part;
        const int d = ok ? k & (D - 1) : 0;
#pragma unroll
        for (int s = 0; s < NSMAX; ++s) {
          if (s < NS) {  // uniform
            num[j][i][s][0] = *reinterpret_cast<const uint4*>(src + s * part + d);
            num[j][i][s][1] = *reinterpret_cast<const uint4*>(src + s * part + d + 4);
            md[j][i][s] = *reinterpret_cast<const float2*>(src + s * part + D);
          }
        }
      }
    }
  }

  __device__ __forceinline__ void merge(uint4 (&c)[RPW][VPL], int M, int K, int NS, int wave, int nwaves,
                                        int lane) const {
    const int nvec = K / 8;
#pragma unroll
    for (int j = 0; j < RPW; ++j) {
      const int m = wave + j * nwaves;
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        const int v = i * 64 + lane;
        float mm = -INFINITY;
#pragma unroll
        for (int s = 0; s < NSMAX; ++s)
          if (s < NS) mm = fmaxf(mm, md[j][i][s].x);
        float n[8], den = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) n[e] = 0.0f;
#pragma unroll
        for (int s = 0; s < NSMAX; ++s) {
          if (s < NS) {
            const float a = attn_slice_weight(md[j][i][s].x, mm);
            const uint4 lo = num[j][i][s][0], hi = num[j][i][s][1];
            n[0] = __builtin_fmaf(__uint_as_float(lo.x), a, n[0]);
            n[1] = __builtin_fmaf(__uint_as_float(lo.y), a, n[1]);
            n[2] = __builtin_fmaf(__uint_as_float(lo.z), a, n[2]);
            n[3] = __builtin_fmaf(__uint_as_float(lo.w), a, n[3]);
            n[4] = __builtin_fmaf(__uint_as_float(hi.x), a, n[4]);
            n[5] = __builtin_fmaf(__uint_as_float(hi.y), a, n[5]);
            n[6] = __builtin_fmaf(__uint_as_float(hi.z), a, n[6]);
            n[7] = __builtin_fmaf(__uint_as_float(hi.w), a, n[7]);
            den = __builtin_fmaf(md[j][i][s].y, a, den);
          }
        }
        const float r = attn_inv_denominator(den);
        uint4 o;
        o.x = pack_bf16x2(__fmul_rn(n[0], r), __fmul_rn(n[1], r));
        o.y = pack_bf16x2(__fmul_rn(n[2], r), __fmul_rn(n[3], r));
        o.z = pack_bf16x2(__fmul_rn(n[4], r), __fmul_rn(n[5], r));
        o.w = pack_bf16x2(__fmul_rn(n[6], r), __fmul_rn(n[7], r));
        c[j][i] = (m < M && v < nvec) ? o : make_uint4(0, 0, 0, 0);
      }
    }
  }
};

}  // namespace aq
