// Measurement probes: what the matrix cores and HBM of this particular part
// deliver, so that kernel figures can be read against measured ceilings as well
// as the published ones.  Not on the Linear path.
#include "aq_common.h"

namespace aq {

// Every wavefront issues `iters` rounds of 8 independent MFMAs (no memory
// traffic, no dependencies closer than 8 instructions apart).
template <int KIND>
__global__ __launch_bounds__(256) void probe_mfma_kernel(int iters, int* sink) {
  const int lane = threadIdx.x & 63;
  if constexpr (KIND == 0) {  // v_mfma_i32_32x32x32_i8
    v4i a = {lane, lane + 1, lane + 2, lane + 3}, b = {lane * 3, 1, 2, 3};
    v16i c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) c[i][r] = 0;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i) c[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c[i], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += c[i][0] + c[i][15];
    if (s == 0x12345678) sink[0] = s;
  } else if constexpr (KIND == 1) {  // v_mfma_i32_16x16x64_i8
    v4i a = {lane, lane + 1, lane + 2, lane + 3}, b = {lane * 3, 1, 2, 3};
    v4i c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) c[i] = v4i{0, 0, 0, 0};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i) c[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c[i], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += c[i][0] + c[i][3];
    if (s == 0x12345678) sink[0] = s;
  } else {  // v_mfma_scale_f32_32x32x64_f8f6f4, e4m3 x e4m3, unit scales
    v8i a = {lane, 1, 2, 3, 4, 5, 6, 7}, b = {lane * 3, 1, 2, 3, 4, 5, 6, 7};
    v16f c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) c[i][r] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        c[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c[i], 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
    }
    float s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += c[i][0] + c[i][15];
    if (s == 1.2345f) sink[0] = 1;
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

}  // namespace aq

extern "C" int aq_probe_mfma(int kind, int workgroups, int iters, int* sink, void* stream) {
  if (kind < 0 || kind > 2 || workgroups <= 0 || iters < 0) return AQ_E_SHAPE;
  if (!sink) return AQ_E_NULL;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (kind == 0)
    hipLaunchKernelGGL((aq::probe_mfma_kernel<0>), dim3(workgroups), dim3(256), 0, st, iters, sink);
  else if (kind == 1)
    hipLaunchKernelGGL((aq::probe_mfma_kernel<1>), dim3(workgroups), dim3(256), 0, st, iters, sink);
  else
    hipLaunchKernelGGL((aq::probe_mfma_kernel<2>), dim3(workgroups), dim3(256), 0, st, iters, sink);
  return (int)hipGetLastError();
}

extern "C" int aq_probe_copy(const void* src, void* dst, int64_t bytes, int workgroups, void* stream) {
  if (bytes < 0 || (bytes % 16) != 0 || workgroups <= 0) return AQ_E_SHAPE;
  if (bytes == 0) return AQ_OK;
  if (!src) return AQ_E_NULL;
  if (aq::check_ptr16(src) || aq::check_ptr16(dst)) return AQ_E_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dst)
    hipLaunchKernelGGL(aq::probe_copy_kernel, dim3(workgroups), dim3(256), 0, st,
                       static_cast<const uint4*>(src), static_cast<uint4*>(dst), bytes / 16);
  else
    return AQ_E_NULL;
  return (int)hipGetLastError();
}

extern "C" int aq_probe_read(const void* src, int64_t bytes, int workgroups, int* sink, void* stream) {
  if (bytes < 0 || (bytes % 16) != 0 || workgroups <= 0) return AQ_E_SHAPE;
  if (bytes == 0) return AQ_OK;
  if (!src || !sink) return AQ_E_NULL;
  if (aq::check_ptr16(src)) return AQ_E_ALIGN;
  hipLaunchKernelGGL(aq::probe_read_kernel, dim3(workgroups), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4*>(src), bytes / 16, sink);
  return (int)hipGetLastError();
}
