// Running sums and maxima over the lanes of a wave with lane moves inside the vector unit (DPP).
//
// A permute through the LDS pipe (__shfl_up and the like) costs a kernel that has a wave or two per
// SIMD, and so nothing to hide a latency behind, some 70 cycles each: six dependent ones per scan.
// These take a handful of vector instructions.  All 64 lanes of the wave must be active.
#ifndef SSPMM_AMD_LANE_OPS_H
#define SSPMM_AMD_LANE_OPS_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sspmm {

// CTRL: 0x110 + n = the value of the lane n below in the same row of 16 lanes; 0x142 = of lane 15 of the row
// below; 0x143 = of lane 31; delivered to the rows ROW_MASK names.  Lanes without a source, and rows not
// named, get 0.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t lanes_below(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xf, true);
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ unsigned long long lanes_below(unsigned long long v) {
  const uint32_t lo = lanes_below<CTRL, ROW_MASK>((uint32_t)v);
  const uint32_t hi = lanes_below<CTRL, ROW_MASK>((uint32_t)(v >> 32));
  return ((unsigned long long)hi << 32) | lo;
}

// Sum of v over lanes 0 .. own lane.  T: uint32_t or unsigned long long.
template <typename T>
__device__ __forceinline__ T wave_inclusive_sum(T v) {
  v += lanes_below<0x111, 0xf>(v);
  v += lanes_below<0x112, 0xf>(v);
  v += lanes_below<0x114, 0xf>(v);
  v += lanes_below<0x118, 0xf>(v);
  v += lanes_below<0x142, 0xa>(v);  // rows 1 and 3 take the sum of the row below
  v += lanes_below<0x143, 0xc>(v);  // rows 2 and 3 take the sum of rows 0 and 1
  return v;
}

// Maximum of v over lanes 0 .. own lane.
__device__ __forceinline__ uint32_t wave_inclusive_max(uint32_t v) {
  v = max(v, lanes_below<0x111, 0xf>(v));
  v = max(v, lanes_below<0x112, 0xf>(v));
  v = max(v, lanes_below<0x114, 0xf>(v));
  v = max(v, lanes_below<0x118, 0xf>(v));
  v = max(v, lanes_below<0x142, 0xa>(v));
  v = max(v, lanes_below<0x143, 0xc>(v));
  return v;
}

// The same moves for floats, with what a lane without a source (or a row not named) gets instead given by the caller.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float lanes_below_or(float v, float otherwise) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(otherwise), __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}
// Maximum / sum of x over all 64 lanes, in every lane (the running value reaches lane 63, which is then read out).
__device__ __forceinline__ float wave_max_all(float x) {
  x = fmaxf(x, lanes_below_or<0x111, 0xf>(x, x));
  x = fmaxf(x, lanes_below_or<0x112, 0xf>(x, x));
  x = fmaxf(x, lanes_below_or<0x114, 0xf>(x, x));
  x = fmaxf(x, lanes_below_or<0x118, 0xf>(x, x));
  x = fmaxf(x, lanes_below_or<0x142, 0xa>(x, x));
  x = fmaxf(x, lanes_below_or<0x143, 0xc>(x, x));
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 63));
}
__device__ __forceinline__ float wave_sum_all(float x) {
  x += lanes_below_or<0x111, 0xf>(x, 0.f);
  x += lanes_below_or<0x112, 0xf>(x, 0.f);
  x += lanes_below_or<0x114, 0xf>(x, 0.f);
  x += lanes_below_or<0x118, 0xf>(x, 0.f);
  x += lanes_below_or<0x142, 0xa>(x, 0.f);
  x += lanes_below_or<0x143, 0xc>(x, 0.f);
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 63));
}

// The value lane 63 holds, in every lane.
__device__ __forceinline__ uint32_t from_last_lane(uint32_t v) { return (uint32_t)__builtin_amdgcn_readlane((int)v, 63); }

}  // namespace sspmm
#endif
