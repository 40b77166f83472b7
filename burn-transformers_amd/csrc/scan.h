// Helpers shared by the kernels that walk a sequence's tokens in order with a state in registers.
#pragma once

#include "common.h"

// Sums over groups of 8 or 16 neighbouring lanes with data-parallel moves between lanes of a row
// (no trip through the LDS crossbar as a shuffle takes; a recurrence pays this once per token): first
// within quads (swap neighbours, swap pairs: then every lane of a quad holds the quad's sum), then
// the mirror image within half a row pairs the two quads of eight lanes, then the mirror image within
// the row pairs its halves.  Every lane of the group ends with the group's sum.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float sum_of_8_lanes(float v) {
  v += dpp_move<0xB1>(v);     // quad_perm [1, 0, 3, 2]
  v += dpp_move<0x4E>(v);     // quad_perm [2, 3, 0, 1]
  v += dpp_move<0x141>(v);    // row_half_mirror
  return v;
}
__device__ __forceinline__ float sum_of_16_lanes(float v) {
  v = sum_of_8_lanes(v);
  v += dpp_move<0x140>(v);    // row_mirror
  return v;
}

__device__ __forceinline__ float silu_f(float v) { return v / (1.0f + expf(-v)); }
__device__ __forceinline__ float softplus_f(float v) { return v > 20.0f ? v : log1pf(expf(v)); }

// Tokens of a run: as many as keep a work-group's LDS at about 24 KiB, at most 64, no more than the step has.
static int scan_chunk(int floats_per_token, int tokens) {
  int chunk = 6144 / floats_per_token;
  chunk = chunk < 1 ? 1 : chunk > 64 ? 64 : chunk;
  return chunk < tokens ? chunk : tokens;
}

