// Sums across the lanes of a 64-wide wave, shared by the backward kernels.
#pragma once

#include <hip/hip_runtime.h>

namespace gelib_hip {

namespace {

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// Sum every element of v over aligned groups of n lanes (n a power of two <= 64); all lanes of a group end with
// the totals.  One uniform branch per butterfly step, not per element.
template <int K>
__device__ __forceinline__ void group_sum(float2 (&v)[K], int n) {
#define GELIB_STEP(COND, EXPR_X, EXPR_Y)    \
  if (COND) {                               \
    _Pragma("unroll") for (int k = 0; k < K; k++) { \
      v[k].x += EXPR_X;                     \
      v[k].y += EXPR_Y;                     \
    }                                       \
  }
  GELIB_STEP(n > 1, dpp_move<0xB1>(v[k].x), dpp_move<0xB1>(v[k].y))    // quad_perm [1,0,3,2]
  GELIB_STEP(n > 2, dpp_move<0x4E>(v[k].x), dpp_move<0x4E>(v[k].y))    // quad_perm [2,3,0,1]
  GELIB_STEP(n > 4, dpp_move<0x141>(v[k].x), dpp_move<0x141>(v[k].y))  // row_half_mirror
  GELIB_STEP(n > 8, dpp_move<0x140>(v[k].x), dpp_move<0x140>(v[k].y))  // row_mirror
  GELIB_STEP(n > 16, __shfl_xor(v[k].x, 16), __shfl_xor(v[k].y, 16))
  GELIB_STEP(n > 32, __shfl_xor(v[k].x, 32), __shfl_xor(v[k].y, 32))
#undef GELIB_STEP
}

// Sum every element of v over lanes that differ in the bits from `lo` up to (but not including) `hi`.
template <int K>
__device__ __forceinline__ void stride_sum(float2 (&v)[K], int lo, int hi) {
  for (int s = lo; s < hi; s <<= 1) {
#pragma unroll
    for (int k = 0; k < K; k++) {
      v[k].x += __shfl_xor(v[k].x, s);
      v[k].y += __shfl_xor(v[k].y, s);
    }
  }
}

// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of its second,
// v_permlane32_swap the upper half of the first with the lower half of the second.  The two wait states in front
// cover a vector write of either operand by the instruction just before.
__device__ __forceinline__ void swap_rows16(float &a, float &b) {
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32_e32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap_halves32(float &a, float &b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32_e32 %0, %1" : "+v"(a), "+v"(b));
}

// Sums over the four 16-lane rows of a wave, four values at a time: lane (row k, column c) receives the total of
// v_k over the four lanes of column c, formed as (row0 + row1) + (row2 + row3).  Six instructions for four values,
// against eight shuffles through LDS for the same sums as butterflies.
__device__ __forceinline__ float rows_sum4(float v0, float v1, float v2, float v3) {
  swap_rows16(v0, v1);
  float a = v0 + v1;  // rows: v0 (0+1), v1 (0+1), v0 (2+3), v1 (2+3)
  swap_rows16(v2, v3);
  float b = v2 + v3;
  swap_halves32(a, b);
  return a + b;  // rows: v0, v1, v2, v3
}

}  // namespace

}  // namespace gelib_hip
