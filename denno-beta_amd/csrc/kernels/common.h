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
// round to nearest even; NaN stays NaN: gfx950 has the conversion in hardware (v_cvt_pk_bf16_f32),
// which the compiler picks for a cast to __bf16
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float f) {
  return bf16_t{__builtin_bit_cast(uint16_t, static_cast<__bf16>(f))};
}

// Exchanges between lanes without LDS.  A butterfly through ds_bpermute costs a trip to LDS per
// step; these run in the vector ALU: DPP inside a row of 16 lanes (xor 1, xor 2, then the
// mirrors of 8 and of 16 lanes, which pair lanes as well as xor 4 and xor 8 do once the quads
// agree), v_readlane to carry the four rows' results to every lane, and gfx950's
// v_permlane32_swap where the two halves of a wave exchange a value each.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
#define DN_DPP_XOR1 0xB1          // quad_perm [1,0,3,2]
#define DN_DPP_XOR2 0x4E          // quad_perm [2,3,0,1]
#define DN_DPP_HALF_MIRROR 0x141  // lane i <-> 7 - i of each 8
#define DN_DPP_MIRROR 0x140       // lane i <-> 15 - i of each 16

struct SumOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
struct MaxOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};

// lane `lane`'s value, the same for every lane (lane is a constant)
__device__ __forceinline__ float lane_value(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// every lane of each aligned group of N lanes (N = 2, 4, 8, 16, 32, 64) gets the group's result;
// rows are joined in the order 0, 1, 2, 3
template <int N, typename Op>
__device__ __forceinline__ float group_reduce(float v, Op op) {
  if (N >= 2) v = op(v, dpp_move<DN_DPP_XOR1>(v));
  if (N >= 4) v = op(v, dpp_move<DN_DPP_XOR2>(v));
  if (N >= 8) v = op(v, dpp_move<DN_DPP_HALF_MIRROR>(v));
  if (N >= 16) v = op(v, dpp_move<DN_DPP_MIRROR>(v));
  if (N >= 32) {
    const float lower = op(lane_value(v, 0), lane_value(v, 16));
    const float upper = op(lane_value(v, 32), lane_value(v, 48));
    v = N >= 64 ? op(lower, upper) : ((threadIdx.x & 32) ? upper : lower);
  }
  return v;
}
__device__ __forceinline__ float wave_sum(float v) { return group_reduce<DN_WAVE>(v, SumOp()); }
__device__ __forceinline__ float wave_max(float v) { return group_reduce<DN_WAVE>(v, MaxOp()); }

// The value that the lane 32 away holds.  v_permlane32_swap exchanges the upper half of its
// first register with the lower half of its second; it is written as assembly with both
// registers named as changed (through the compiler's builtin the second result is lost), and
// with the idle cycles that the instruction wants before and after it, which the compiler does
// not add around assembly.
__device__ __forceinline__ float other_half(float v) {
  unsigned a = __builtin_bit_cast(unsigned, v), b = a;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  // a: the lower half's values in both halves; b: the upper half's
  return __builtin_bit_cast(float, (threadIdx.x & 32) ? a : b);
}

static inline int dn_launch_status() { return static_cast<int>(hipGetLastError()); }

// A packed matrix: blocks of 16 rows x 32 columns, 1 KB each and contiguous, block (r / 16, k / 32)
// at ((r / 16) * ksteps + k / 32) * 512 elements; inside it the 8 elements from column k % 32 / 8 * 8
// of row r % 16 lie at ((k % 32 / 8) * 16 + r % 16) * 8: the 16 bytes that lane r % 16 + 16 * (k % 32 / 8)
// feeds to v_mfma_f32_16x16x32_bf16.  Every weight of the MFMA kernels is held so, and so are the
// bfloat16 rows that one kernel hands to the next while a step has at most 64 of them.
__device__ __forceinline__ size_t packed_index(int r, int k, int ksteps) {
  return ((static_cast<size_t>(r / 16) * ksteps + k / 32) * 64 + ((k % 32) / 8) * 16 + r % 16) * 8 + k % 8;
}
