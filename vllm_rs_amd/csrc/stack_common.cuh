// stack_common.cuh — helpers shared by the operator files of config-driven layer stacks (stack_ops.hip, stack_mixers.hip).
#pragma once
#include <math.h>

#include "common.cuh"
#include "stack_launch.h"

namespace {

template <typename T>
struct El;
template <>
struct El<float> {
  static __device__ __forceinline__ float ld(const float* p) { return *p; }
  static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
  static __device__ __forceinline__ float rnd(float v) { return v; }
};
template <>
struct El<uint16_t> {
  static __device__ __forceinline__ float ld(const uint16_t* p) { return BF16::to_f32(*p); }
  static __device__ __forceinline__ void st(uint16_t* p, float v) { *p = BF16::from_f32(v); }
  static __device__ __forceinline__ float rnd(float v) { return BF16::to_f32(BF16::from_f32(v)); }
};

__device__ __forceinline__ float wave_sum(float v) {
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float sigmoidf_(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

// cos / sin of p * (hi + lo), times mag: the product p * hi is split exactly (fma), the small part enters to first order
__device__ __forceinline__ void rot_cos_sin(const StkRotary& r, int i, float p, float* c, float* s) {
  const float fh = r.freq_hi[i], fl = r.freq_lo ? r.freq_lo[i] : 0.f;
  const float ah = p * fh;
  const float al = fmaf(p, fh, -ah) + p * fl;
  const float c0 = cosf(ah), s0 = sinf(ah);
  *c = (c0 - s0 * al) * r.mag;
  *s = (s0 + c0 * al) * r.mag;
}

template <typename F>
void launch_checked(const char* what, F f) {
  f();
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) vra_set_error("%s: %s", what, hipGetErrorString(e));
}

}  // namespace
