// Cross-row reductions of a 64-lane wave on gfx950 without a trip through the LDS crossbar.
//
// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of
// its second; v_permlane32_swap does the same with the upper and lower 32 lanes. Fed the same
// value x twice, the two results hold {x[l & ~16], x[l | 16]} resp. {x[l & ~32], x[l | 32]} in
// lane l, i.e. x[l] and x[l ^ 16] (x[l ^ 32]) in some order: enough for max and sum.
#pragma once
#include <hip/hip_runtime.h>

namespace pat {

typedef unsigned lane_u32x2 __attribute__((ext_vector_type(2)));

// The two results are copied into scalars before any reinterpretation: __builtin_bit_cast applied
// directly to an element of an ext_vector (r[1]) reads element 0 with hipcc 7.2.
__device__ __forceinline__ void swap16(float x, float& lo, float& hi) {
  const unsigned a = __builtin_bit_cast(unsigned, x);
  const lane_u32x2 r = __builtin_amdgcn_permlane16_swap(a, a, false, false);
  const unsigned r0 = r[0], r1 = r[1];
  lo = __builtin_bit_cast(float, r0);
  hi = __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ void swap32(float x, float& lo, float& hi) {
  const unsigned a = __builtin_bit_cast(unsigned, x);
  const lane_u32x2 r = __builtin_amdgcn_permlane32_swap(a, a, false, false);
  const unsigned r0 = r[0], r1 = r[1];
  lo = __builtin_bit_cast(float, r0);
  hi = __builtin_bit_cast(float, r1);
}

__device__ __forceinline__ float max_xor16(float x) { float a, b; swap16(x, a, b); return fmaxf(a, b); }
__device__ __forceinline__ float max_xor32(float x) { float a, b; swap32(x, a, b); return fmaxf(a, b); }
__device__ __forceinline__ float sum_xor16(float x) { float a, b; swap16(x, a, b); return a + b; }
__device__ __forceinline__ float sum_xor32(float x) { float a, b; swap32(x, a, b); return a + b; }

}  // namespace pat
