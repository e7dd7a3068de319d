// Shared by every kernel file: element types, conversions, wave reductions.
// gfx950 only: wavefronts are 64 wide.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define DN_WAVE 64

// dtype codes of the C ABI
#define DN_F32 0
#define DN_BF16 1

// error codes of the C ABI (negative: ours; positive: hipError_t)
#define DN_ERR_DTYPE (-1)
#define DN_ERR_SHAPE (-2)

struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) { return __uint_as_float(static_cast<uint32_t>(x.bits) << 16); }

template <typename T>
__device__ __forceinline__ T from_float(float f);
template <>
__device__ __forceinline__ float from_float<float>(float f) {
  return f;
}
// round to nearest even; NaN stays NaN
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return bf16_t{static_cast<uint16_t>((u >> 16) | 0x40u)};
  u += 0x7fffu + ((u >> 16) & 1u);
  return bf16_t{static_cast<uint16_t>(u >> 16)};
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = DN_WAVE / 2; m >= 1; m >>= 1) v += __shfl_xor(v, m, DN_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = DN_WAVE / 2; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, DN_WAVE));
  return v;
}

static inline int dn_launch_status() { return static_cast<int>(hipGetLastError()); }
