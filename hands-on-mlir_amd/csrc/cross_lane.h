// Cross-lane reductions for 64-lane wavefronts on gfx950 that stay in the
// vector ALU: data-parallel-primitive (DPP) operands inside a row of 16 lanes,
// v_permlane16_swap / v_permlane32_swap between rows.  A __shfl_xor is an LDS
// round trip (ds_bpermute) of a hundred cycles or more; these are one
// instruction each.
#pragma once

#include <hip/hip_runtime.h>

namespace hom {

// v + (v of the lane a DPP control selects); CTRL is the dpp_ctrl encoding.
template <int CTRL> __device__ __forceinline__ float addDpp(float v) {
  return v + __int_as_float(__builtin_amdgcn_update_dpp(
                 0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

// Sum over groups of N consecutive lanes (N = 4, 8 or 16, groups aligned to
// N), result in every lane of the group: quad permutes exchange lanes ^1 and
// ^2, the half-row and row mirrors pair each lane with one of the other quad /
// the other half of its row.
template <int N> __device__ __forceinline__ float sumAcrossLanes(float v) {
  static_assert(N == 4 || N == 8 || N == 16, "group size");
  v = addDpp<0xB1>(v); // quad_perm [1,0,3,2]
  v = addDpp<0x4E>(v); // quad_perm [2,3,0,1]
  if (N >= 8)
    v = addDpp<0x141>(v); // row_half_mirror
  if (N >= 16)
    v = addDpp<0x140>(v); // row_mirror
  return v;
}

// v_permlane32_swap exchanges the upper half of its first operand with the
// lower half of its second; given the same value twice it returns (lower-half
// values, upper-half values) in every lane pair (l, l ^ 32).
__device__ __forceinline__ float pairMax(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v),
                                                  __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float pairSum(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v),
                                                  __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// v_permlane16_swap exchanges the odd rows of its first operand with the even
// rows of its second: the same value twice gives (even-row values, odd-row
// values) in every lane pair (l, l ^ 16).
__device__ __forceinline__ float rowPairSum(float v) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v),
                                                  __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Sum over the whole wavefront, result in every lane.
__device__ __forceinline__ float waveSum(float v) {
  return pairSum(rowPairSum(sumAcrossLanes<16>(v)));
}

} // namespace hom
