// Measurement probes and test hooks of the lab library (libastrai_q_lab.so): what the matrix cores
// and HBM of this particular part deliver, so that kernel figures can be read against measured
// ceilings as well as the published ones.  Not on the Linear path and not in the product library.
#include "aq_common.h"
#include "aq_lab.h"

namespace aq {

__device__ __forceinline__ uint32_t lab_hash(uint32_t h) {
  h ^= h >> 15;
  h *= 2246822519u;
  h ^= h >> 13;
  h *= 3266489917u;
  h ^= h >> 16;
  return h;
}

// Every wavefront issues `iters` rounds of 8 independent MFMAs (no memory traffic, no
// dependencies closer than 8 instructions apart).  DATA 0: one constant operand pair;
// DATA 1: four random operand sets per lane, cycled so that consecutive instructions see
// different bits on the operand buses, as a GEMM's fragment stream does.
template <int KIND, int DATA>
__global__ __launch_bounds__(256) void probe_mfma_kernel(int iters, int* sink, long long* clocks) {
  const int lane = threadIdx.x & 63;
  const uint32_t gid = blockIdx.x * 256 + threadIdx.x;
  v4i a[4], b[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    if constexpr (DATA == 0) {
      a[s] = v4i{lane, lane + 1, lane + 2, lane + 3};
      b[s] = v4i{lane * 3, 1, 2, 3};
    } else {
      // FP8: exponents kept low (no NaN, no overflow of the fp32 sums)
      const uint32_t mask = KIND == 2 ? 0x77777777u : 0xffffffffu;
      a[s] = v4i{(int)(lab_hash(gid * 32 + s * 8 + 0) & mask), (int)(lab_hash(gid * 32 + s * 8 + 1) & mask),
                 (int)(lab_hash(gid * 32 + s * 8 + 2) & mask), (int)(lab_hash(gid * 32 + s * 8 + 3) & mask)};
      b[s] = v4i{(int)(lab_hash(gid * 32 + s * 8 + 4) & mask), (int)(lab_hash(gid * 32 + s * 8 + 5) & mask),
                 (int)(lab_hash(gid * 32 + s * 8 + 6) & mask), (int)(lab_hash(gid * 32 + s * 8 + 7) & mask)};
    }
  }
  long long c0 = 0, w0 = 0;
  if (clocks && gid == 0) {
    c0 = clock64();
    w0 = wall_clock64();
  }
  if constexpr (KIND == 0) {  // v_mfma_i32_32x32x32_i8
    v16i c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) c[i][r] = 0;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        c[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i & 3], b[(i + (i >> 2)) & 3], c[i], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += c[i][0] + c[i][15];
    if (s == 0x12345678) sink[0] = s;
  } else if constexpr (KIND == 1) {  // v_mfma_i32_16x16x64_i8
    v4i c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) c[i] = v4i{0, 0, 0, 0};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        c[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[i & 3], b[(i + (i >> 2)) & 3], c[i], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += c[i][0] + c[i][3];
    if (s == 0x12345678) sink[0] = s;
  } else {  // v_mfma_scale_f32_32x32x64_f8f6f4, e4m3 x e4m3, unit scales
    v16f c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) c[i][r] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const v4i x = a[i & 3], y = a[(i + 1) & 3], u = b[(i + (i >> 2)) & 3], w = b[(i + 2) & 3];
        const v8i aa = {x.x, x.y, x.z, x.w, y.x, y.y, y.z, y.w}, bb = {u.x, u.y, u.z, u.w, w.x, w.y, w.z, w.w};
        c[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(aa, bb, c[i], 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
      }
    }
    float s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += c[i][0] + c[i][15];
    if (s == 1.2345f) sink[0] = 1;
  }
  if (clocks && gid == 0) {
    clocks[0] = clock64() - c0;
    clocks[1] = wall_clock64() - w0;
  }
}

// Plain streaming copy, 16 bytes per lane, grid-stride: the known-size kernel
// that HBM counters and achieved bandwidth are calibrated against.
__global__ __launch_bounds__(256) void probe_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                         int64_t nvec) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride) dst[i] = src[i];
}

// Read-only stream: sums every 16-byte vector (keeps the loads alive).
__global__ __launch_bounds__(256) void probe_read_kernel(const uint4* __restrict__ src, int64_t nvec, int* sink) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  uint32_t s = 0;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride) {
    const uint4 v = src[i];
    s += v.x ^ v.y ^ v.z ^ v.w;
  }
  if (s == 0x12345678u) sink[0] = 1;
}

// The same read with every load of a lane issued before any is used: a wavefront owns L KiB contiguous
// (its L loads are 1 KiB apart), so the whole buffer is requested at once and the kernel is one memory
// latency plus the stream -- the shape of the decode GEMV's weight read.
template <int L, bool NT>
__global__ __launch_bounds__(256) void probe_read_upfront_kernel(const uint4* __restrict__ src, int* sink) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 6;
  uint4 v[L];
#pragma unroll
  for (int j = 0; j < L; ++j) {
    const uint4* p = src + (wave * L + j) * 64 + lane;
    if constexpr (NT) {
      const uint32_t* q = reinterpret_cast<const uint32_t*>(p);
      v[j] = make_uint4(__builtin_nontemporal_load(q), __builtin_nontemporal_load(q + 1), __builtin_nontemporal_load(q + 2),
                        __builtin_nontemporal_load(q + 3));
    } else {
      v[j] = *p;
    }
  }
  uint32_t s = 0;
#pragma unroll
  for (int j = 0; j < L; ++j) s += v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
  if (s == 0x12345678u) sink[0] = 1;
}

__global__ void probe_empty_kernel(int* sink) {
  if (threadIdx.x == 9999) sink[0] = 1;
}

template <int L>
static int launch_read_upfront(const void* src, int64_t bytes, bool nt, int* sink, hipStream_t st) {
  const int64_t per_wg = (int64_t)256 * 16 * L;
  if (bytes % per_wg) return AQ_E_SHAPE;
  const unsigned grid = (unsigned)(bytes / per_wg);
  if (nt)
    hipLaunchKernelGGL((probe_read_upfront_kernel<L, true>), dim3(grid), dim3(256), 0, st, static_cast<const uint4*>(src), sink);
  else
    hipLaunchKernelGGL((probe_read_upfront_kernel<L, false>), dim3(grid), dim3(256), 0, st, static_cast<const uint4*>(src), sink);
  return (int)hipGetLastError();
}


// What fragment reads cost the matrix pipe with ONE wavefront per SIMD, by where they are issued.  Every wavefront
// runs `iters` iterations of 32 MFMAs (v_mfma_i32_32x32x32_i8, 8 accumulators in AGPRs) and 16 ds_read_b128 in a
// ping-pong of two register sets: the MFMAs of one half consume what the reads of the other half filled, as a
// GEMM's K loop does.  The instruction order is fixed in inline assembly.
//   variant 0: MFMAs only (1024 cycles per iteration is the matrix pipe's own time)
//   variant 1: one read behind every second MFMA
//   variant 2: the eight reads of a half first, then its sixteen MFMAs
//   variant 3: reads in pairs behind every fourth MFMA
// clocks[0] receives the shader-clock cycles wavefront 0 of workgroup 0 spent in the loop.
#define AQ_MF(acc, a, b) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b))
#define AQ_DR(dst, off) asm volatile("ds_read_b128 %0, %1 offset:" #off : "=&v"(dst) : "v"(addr))
#define AQ_LGKM0() asm volatile("s_waitcnt lgkmcnt(0)")
template <int V>
__global__ __launch_bounds__(256) void probe_issue_kernel(int iters, int* sink, long long* clocks) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < 32768 / 4; i += 256) reinterpret_cast<int*>(lds)[i] = 0;
  __syncthreads();
  const unsigned addr = (unsigned)(wave * 1024 + lane * 16);
  v16i c0 = {}, c1 = {}, c2 = {}, c3 = {}, c4 = {}, c5 = {}, c6 = {}, c7 = {};
  v4i a0 = {0, 0, 0, 0}, a1 = a0, a2 = a0, a3 = a0, b0 = a0, b1 = a0, b2 = a0, b3 = a0;
  v4i n0 = a0, n1 = a0, n2 = a0, n3 = a0, n4 = a0, n5 = a0, n6 = a0, n7 = a0;
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
    if constexpr (V == 0) {
      AQ_MF(c0, n0, n4); AQ_MF(c1, n0, n5); AQ_MF(c2, n0, n6); AQ_MF(c3, n0, n7); AQ_MF(c4, n1, n4); AQ_MF(c5, n1, n5); AQ_MF(c6, n1, n6); AQ_MF(c7, n1, n7);
      AQ_MF(c0, n2, n4); AQ_MF(c1, n2, n5); AQ_MF(c2, n2, n6); AQ_MF(c3, n2, n7); AQ_MF(c4, n3, n4); AQ_MF(c5, n3, n5); AQ_MF(c6, n3, n6); AQ_MF(c7, n3, n7);
      AQ_MF(c0, a0, b0); AQ_MF(c1, a0, b1); AQ_MF(c2, a0, b2); AQ_MF(c3, a0, b3); AQ_MF(c4, a1, b0); AQ_MF(c5, a1, b1); AQ_MF(c6, a1, b2); AQ_MF(c7, a1, b3);
      AQ_MF(c0, a2, b0); AQ_MF(c1, a2, b1); AQ_MF(c2, a2, b2); AQ_MF(c3, a2, b3); AQ_MF(c4, a3, b0); AQ_MF(c5, a3, b1); AQ_MF(c6, a3, b2); AQ_MF(c7, a3, b3);
    } else if constexpr (V == 1) {
      AQ_MF(c0, n0, n4); AQ_DR(a0, 0); AQ_MF(c1, n0, n5); AQ_MF(c2, n0, n6); AQ_DR(b0, 16384); AQ_MF(c3, n0, n7); AQ_MF(c4, n1, n4); AQ_DR(a1, 4096); AQ_MF(c5, n1, n5); AQ_MF(c6, n1, n6); AQ_DR(b1, 20480); AQ_MF(c7, n1, n7);
      AQ_MF(c0, n2, n4); AQ_DR(a2, 8192); AQ_MF(c1, n2, n5); AQ_MF(c2, n2, n6); AQ_DR(b2, 24576); AQ_MF(c3, n2, n7); AQ_MF(c4, n3, n4); AQ_DR(a3, 12288); AQ_MF(c5, n3, n5); AQ_MF(c6, n3, n6); AQ_DR(b3, 28672); AQ_MF(c7, n3, n7);
      AQ_LGKM0();
      AQ_MF(c0, a0, b0); AQ_DR(n0, 0); AQ_MF(c1, a0, b1); AQ_MF(c2, a0, b2); AQ_DR(n4, 16384); AQ_MF(c3, a0, b3); AQ_MF(c4, a1, b0); AQ_DR(n1, 4096); AQ_MF(c5, a1, b1); AQ_MF(c6, a1, b2); AQ_DR(n5, 20480); AQ_MF(c7, a1, b3);
      AQ_MF(c0, a2, b0); AQ_DR(n2, 8192); AQ_MF(c1, a2, b1); AQ_MF(c2, a2, b2); AQ_DR(n6, 24576); AQ_MF(c3, a2, b3); AQ_MF(c4, a3, b0); AQ_DR(n3, 12288); AQ_MF(c5, a3, b1); AQ_MF(c6, a3, b2); AQ_DR(n7, 28672); AQ_MF(c7, a3, b3);
    } else if constexpr (V == 2) {
      AQ_DR(a0, 0); AQ_DR(b0, 16384); AQ_DR(a1, 4096); AQ_DR(b1, 20480); AQ_DR(a2, 8192); AQ_DR(b2, 24576); AQ_DR(a3, 12288); AQ_DR(b3, 28672);
      AQ_MF(c0, n0, n4); AQ_MF(c1, n0, n5); AQ_MF(c2, n0, n6); AQ_MF(c3, n0, n7); AQ_MF(c4, n1, n4); AQ_MF(c5, n1, n5); AQ_MF(c6, n1, n6); AQ_MF(c7, n1, n7);
      AQ_MF(c0, n2, n4); AQ_MF(c1, n2, n5); AQ_MF(c2, n2, n6); AQ_MF(c3, n2, n7); AQ_MF(c4, n3, n4); AQ_MF(c5, n3, n5); AQ_MF(c6, n3, n6); AQ_MF(c7, n3, n7);
      AQ_LGKM0();
      AQ_DR(n0, 0); AQ_DR(n4, 16384); AQ_DR(n1, 4096); AQ_DR(n5, 20480); AQ_DR(n2, 8192); AQ_DR(n6, 24576); AQ_DR(n3, 12288); AQ_DR(n7, 28672);
      AQ_MF(c0, a0, b0); AQ_MF(c1, a0, b1); AQ_MF(c2, a0, b2); AQ_MF(c3, a0, b3); AQ_MF(c4, a1, b0); AQ_MF(c5, a1, b1); AQ_MF(c6, a1, b2); AQ_MF(c7, a1, b3);
      AQ_MF(c0, a2, b0); AQ_MF(c1, a2, b1); AQ_MF(c2, a2, b2); AQ_MF(c3, a2, b3); AQ_MF(c4, a3, b0); AQ_MF(c5, a3, b1); AQ_MF(c6, a3, b2); AQ_MF(c7, a3, b3);
    } else {
      AQ_MF(c0, n0, n4); AQ_DR(a0, 0); AQ_DR(b0, 16384); AQ_MF(c1, n0, n5); AQ_MF(c2, n0, n6); AQ_MF(c3, n0, n7); AQ_MF(c4, n1, n4); AQ_DR(a1, 4096); AQ_DR(b1, 20480); AQ_MF(c5, n1, n5); AQ_MF(c6, n1, n6); AQ_MF(c7, n1, n7);
      AQ_MF(c0, n2, n4); AQ_DR(a2, 8192); AQ_DR(b2, 24576); AQ_MF(c1, n2, n5); AQ_MF(c2, n2, n6); AQ_MF(c3, n2, n7); AQ_MF(c4, n3, n4); AQ_DR(a3, 12288); AQ_DR(b3, 28672); AQ_MF(c5, n3, n5); AQ_MF(c6, n3, n6); AQ_MF(c7, n3, n7);
      AQ_LGKM0();
      AQ_MF(c0, a0, b0); AQ_DR(n0, 0); AQ_DR(n4, 16384); AQ_MF(c1, a0, b1); AQ_MF(c2, a0, b2); AQ_MF(c3, a0, b3); AQ_MF(c4, a1, b0); AQ_DR(n1, 4096); AQ_DR(n5, 20480); AQ_MF(c5, a1, b1); AQ_MF(c6, a1, b2); AQ_MF(c7, a1, b3);
      AQ_MF(c0, a2, b0); AQ_DR(n2, 8192); AQ_DR(n6, 24576); AQ_MF(c1, a2, b1); AQ_MF(c2, a2, b2); AQ_MF(c3, a2, b3); AQ_MF(c4, a3, b0); AQ_DR(n3, 12288); AQ_DR(n7, 28672); AQ_MF(c5, a3, b1); AQ_MF(c6, a3, b2); AQ_MF(c7, a3, b3);
    }
    AQ_LGKM0();
  }
  const long long t1 = clock64();
  if (clocks && threadIdx.x == 0 && blockIdx.x == 0) clocks[0] = t1 - t0;
  int s = n0[0] ^ n1[1] ^ n2[2] ^ n3[3] ^ n4[0] ^ n5[0] ^ n6[0] ^ n7[0] ^ a0[0] ^ a1[0] ^ a2[0] ^ a3[0] ^ b0[0] ^ b1[0] ^ b2[0] ^ b3[0];
#pragma unroll
  for (int i = 0; i < 16; ++i) s ^= c0[i] ^ c1[i] ^ c2[i] ^ c3[i] ^ c4[i] ^ c5[i] ^ c6[i] ^ c7[i];
  if (s == 0x12345678) sink[0] = s;
}
#undef AQ_MF
#undef AQ_DR
#undef AQ_LGKM0

}  // namespace aq

extern "C" int aq_lab_probe_mfma(int kind, int data, int workgroups, int iters, int* sink, long long* clocks, void* stream) {
  if (kind < 0 || kind > 2 || data < 0 || data > 1 || workgroups <= 0 || iters < 0) return AQ_E_SHAPE;
  if (!sink) return AQ_E_NULL;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 g(workgroups), b(256);
#define AQ_LAB_MFMA(K, D) hipLaunchKernelGGL((aq::probe_mfma_kernel<K, D>), g, b, 0, st, iters, sink, clocks)
  if (kind == 0 && data == 0) AQ_LAB_MFMA(0, 0);
  else if (kind == 0) AQ_LAB_MFMA(0, 1);
  else if (kind == 1 && data == 0) AQ_LAB_MFMA(1, 0);
  else if (kind == 1) AQ_LAB_MFMA(1, 1);
  else if (data == 0) AQ_LAB_MFMA(2, 0);
  else AQ_LAB_MFMA(2, 1);
#undef AQ_LAB_MFMA
  return (int)hipGetLastError();
}

extern "C" int aq_lab_probe_copy(const void* src, void* dst, int64_t bytes, int workgroups, void* stream) {
  if (bytes < 0 || (bytes % 16) != 0 || workgroups <= 0) return AQ_E_SHAPE;
  if (bytes == 0) return AQ_OK;
  if (!src || !dst) return AQ_E_NULL;
  if (aq::check_ptr16(src) || aq::check_ptr16(dst)) return AQ_E_ALIGN;
  hipLaunchKernelGGL(aq::probe_copy_kernel, dim3(workgroups), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4*>(src), static_cast<uint4*>(dst), bytes / 16);
  return (int)hipGetLastError();
}

extern "C" int aq_lab_probe_read(const void* src, int64_t bytes, int loads_per_lane, int workgroups, int nontemporal,
                                 int* sink, void* stream) {
  if (bytes < 0 || (bytes % 16) != 0) return AQ_E_SHAPE;
  if (bytes == 0) return AQ_OK;
  if (!src || !sink) return AQ_E_NULL;
  if (aq::check_ptr16(src)) return AQ_E_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (loads_per_lane) {
    case 0:
      if (workgroups <= 0) return AQ_E_SHAPE;
      hipLaunchKernelGGL(aq::probe_read_kernel, dim3(workgroups), dim3(256), 0, st, static_cast<const uint4*>(src),
                         bytes / 16, sink);
      return (int)hipGetLastError();
    case 1: return aq::launch_read_upfront<1>(src, bytes, nontemporal != 0, sink, st);
    case 2: return aq::launch_read_upfront<2>(src, bytes, nontemporal != 0, sink, st);
    case 4: return aq::launch_read_upfront<4>(src, bytes, nontemporal != 0, sink, st);
    case 8: return aq::launch_read_upfront<8>(src, bytes, nontemporal != 0, sink, st);
    case 16: return aq::launch_read_upfront<16>(src, bytes, nontemporal != 0, sink, st);
    default: return AQ_E_SHAPE;
  }
}

namespace aq {
// h[i] = up[i] * silu(gate[i]) for bf16 operands as the row kernel's mid-range path computes it (no clamp in the
// exponential, the two-slot-shorter divide for bf16 gates), and whether the gate passes that path's range test.
__global__ void probe_swiglu_bf16_kernel(const uint16_t* up, const uint16_t* gate, int64_t n, float* h, uint8_t* in_range) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float u = __uint_as_float((uint32_t)up[i] << 16), g = __uint_as_float((uint32_t)gate[i] << 16);
  float out;
  swiglu_group_midrange<1, false, true>(&u, &g, &out);
  h[i] = out;
  GateRangeBf16 r;
  r.add(make_uint4((uint32_t)gate[i] | ((uint32_t)gate[i] << 16), 0x3f803f80u, 0x3f803f80u, 0x3f803f80u));
  in_range[i] = r.ok() ? 1 : 0;
}
}  // namespace aq

extern "C" int aq_lab_probe_swiglu_bf16(const uint16_t* up, const uint16_t* gate, int64_t n, float* h, uint8_t* in_range,
                                        void* stream) {
  if (n < 0 || (n && (!up || !gate || !h || !in_range))) return AQ_E_NULL;
  if (n == 0) return AQ_OK;
  hipLaunchKernelGGL(aq::probe_swiglu_bf16_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), up, gate, n, h, in_range);
  return (int)hipGetLastError();
}

extern "C" int aq_lab_probe_empty(int* sink, void* stream) {
  if (!sink) return AQ_E_NULL;
  hipLaunchKernelGGL(aq::probe_empty_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), sink);
  return (int)hipGetLastError();
}

extern "C" int aq_lab_probe_mfma_lds_issue(int variant, int workgroups, int iters, int* sink, long long* clocks,
                                           void* stream) {
  if (variant < 0 || variant > 3 || workgroups <= 0 || iters <= 0 || !sink) return AQ_E_SHAPE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  using kern_t = void (*)(int, int*, long long*);
  static const kern_t table[4] = {aq::probe_issue_kernel<0>, aq::probe_issue_kernel<1>, aq::probe_issue_kernel<2>,
                                  aq::probe_issue_kernel<3>};
  hipLaunchKernelGGL(table[variant], dim3((unsigned)workgroups), dim3(256), 32768, st, iters, sink, clocks);
  return (int)hipGetLastError();
}

// The one-launch FP8 quantiser with the bound on its wait for the other workgroups given by the caller: 0 makes
// every workgroup give up at once and take the tensor's maximum itself, the path a busy device would take.
namespace aq {
int quant_tensor_fp8_onepass(const void* x, int x_dtype, int64_t numel, uint8_t* q, float* scale, void* ws,
                             size_t ws_bytes, int spin_limit, hipStream_t st);
}
extern "C" int aq_lab_quant_tensor_fp8_onepass_spin(const void* x, int x_dtype, int64_t numel, uint8_t* q, float* scale,
                                                    void* ws, size_t ws_bytes, int spin_limit, void* stream) {
  if (spin_limit < 0) return AQ_E_RANGE;
  return aq::quant_tensor_fp8_onepass(x, x_dtype, numel, q, scale, ws, ws_bytes, spin_limit,
                                      static_cast<hipStream_t>(stream));
}
