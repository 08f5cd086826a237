// Sums over neighbouring lanes of a wave by row permutes, for recurrences whose lanes share a state column.
#pragma once
#include "common.h"

// sum over KS neighbouring lanes (from a multiple of KS on); every lane gets it
template <int KS>
__device__ inline float column_sum(float v) {
#define DPP_ADD(ctrl) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, false))
  if (KS >= 2) DPP_ADD(0xB1);    // quad_perm [1, 0, 3, 2]
  if (KS >= 4) DPP_ADD(0x4E);    // quad_perm [2, 3, 0, 1]
  if (KS >= 8) DPP_ADD(0x141);   // row_half_mirror
  if (KS >= 16) DPP_ADD(0x140);  // row_mirror
#undef DPP_ADD
  if (KS >= 32) v += __shfl_xor(v, 16, TP_WAVE);
  return v;
}
