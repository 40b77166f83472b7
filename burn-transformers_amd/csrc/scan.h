// Helpers shared by the kernels that walk a sequence's tokens in order with a state in registers.
#pragma once

#include <hip/hip_runtime.h>

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


// Spans.  A recurrence S_t = a_t S_(t-1) + u_t is linear in S, so a long sequence need not be walked
// by one wave: cut into spans of `span` tokens, (1) every span is scanned from a zero state, side by
// side, and leaves its end state E_k and the sum of its step sizes (its decays multiply up to
// P_k = exp(A * that sum)); (2) a short kernel carries the state across the spans in order,
// C_k = P_k C_(k-1) + E_k, from the slot's state; (3) every span is scanned again, side by side, from
// the state C_(k-1) it really starts with, and writes the outputs.  The carrying kernel also keeps the
// state the sequence came with (as "span -1": the third pass reads only the carry, never the slot, which
// by then holds the state after the sequence's last token, written by the carrying kernel).  Twice the
// arithmetic, on (sequence length / span) times the waves.  Span k of sequence s keeps its block at
// index seq_off[s] / span + 2 s + 1 + k: ranges of different sequences do not meet.
__device__ __forceinline__ int64_t span_block(const int* seq_off, int seq, int span, int part) {
  return (int64_t)(seq_off[seq] / span + 2 * seq + 1 + part);
}


// Sequences of at least this many spans are cut (fewer gain nothing over walking them).
#define MIN_SPANS 3

static int simd_count() {
  static int count = 0;
  if (count == 0) {
    int device = 0, units = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || units <= 0)
      units = 256;
    count = 4 * units;
  }
  return count;
}

// Into spans of how many tokens a step's long sequences are cut, 0 for not at all.  Spans double the
// arithmetic, so they pay only while whole sequences leave the chip short of waves: `waves` (those that
// walk whole sequences) must be at most `fill` to a SIMD, and there are as many spans as bring four
// times that, none shorter than the call's `span`, which its room for the spans' states was sized
// for.  Measured for 2 x 1,024 tokens (us, whole / cut): the head scan with one wave to a SIMD 309 / 205,
// with two 327 / 380; the selective scan with half a wave to a SIMD 334 / 176, with one 369 / 311.
static int span_tokens(int span, int max_count, const float* carry, int64_t waves, int fill) {
  if (span <= 0 || !carry || waves > (int64_t)fill * simd_count()) return 0;
  const int64_t wanted = 4 * (int64_t)fill * simd_count() / waves;
  int tokens = (int)((max_count + wanted - 1) / wanted);
  if (tokens < span) tokens = span;
  return max_count >= MIN_SPANS * tokens ? tokens : 0;
}

