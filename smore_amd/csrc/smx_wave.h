// Wavefront-level helpers for gfx950 (64 lanes).
#pragma once
#include <hip/hip_runtime.h>

namespace smx {

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

// Sum over the 64 lanes, result identical in every lane.  Four DPP steps fold
// each row of 16 lanes (quad swaps, half-row mirror, row mirror); the four row
// sums are then read out and added in a fixed order, so the result does not
// depend on which lane asks.
__device__ __forceinline__ float wave_sum_f32(float v) {
  v += dpp_move<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_move<0x141>(v);  // row_half_mirror
  v += dpp_move<0x140>(v);  // row_mirror
  const int iv = __float_as_int(v);
  const float r0 = __int_as_float(__builtin_amdgcn_readlane(iv, 0));
  const float r1 = __int_as_float(__builtin_amdgcn_readlane(iv, 16));
  const float r2 = __int_as_float(__builtin_amdgcn_readlane(iv, 32));
  const float r3 = __int_as_float(__builtin_amdgcn_readlane(iv, 48));
  return ((r0 + r1) + r2) + r3;
}

// Sum over the 64 lanes, valid in lane 63 only: the four row sums are combined with two more DPP
// steps (row_bcast:15 into rows 1 and 3, row_bcast:31 into rows 2 and 3) instead of being read out
// into scalars, six vector instructions in all.  Order: (r2 + r3) + (r0 + r1).
__device__ __forceinline__ float wave_sum_last_f32(float v) {
  v += dpp_move<0xB1>(v);
  v += dpp_move<0x4E>(v);
  v += dpp_move<0x141>(v);
  v += dpp_move<0x140>(v);
  // rows outside row_mask keep their value; written as the fused instruction (the compiler expands the
  // builtin form into mov 0 + mov_dpp + add); the s_nop cover the VALU-write -> DPP-read wait states
  asm("s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf"
      : "+v"(v));
  return v;
}

// Number of set bits of m at lanes below this one.
__device__ __forceinline__ unsigned lanes_below_in(unsigned long long m) {
  return __builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, 0u));
}

// Makes a value the compiler cannot prove wave-uniform into a scalar.
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

__device__ __forceinline__ long long uniform64(long long v) {
  const int lo = __builtin_amdgcn_readfirstlane((int)(v & 0xffffffffll));
  const int hi = __builtin_amdgcn_readfirstlane((int)(v >> 32));
  return ((long long)hi << 32) | (unsigned int)lo;
}

}  // namespace smx
