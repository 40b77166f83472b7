// Arguments of the attention kernels (plain and MFMA); mirrored by a ctypes.Structure.
#pragma once

#include "common.h"

struct AttnArgs {
  const void* q;        // [tokens][ldq]; head j at columns j * head_dim
  int64_t ldq;
  void* out;            // [tokens][ldo]
  int64_t ldo;
  const int* tok_seq;   // [tokens]
  const int* tok_pos;   // [tokens]
  const int* seq_off;   // [n_seqs + 1] first token of each sequence in the step
  const int* seq_start; // [n_seqs] position of that first token
  KvView kv;
  int q_heads;
  int n_tokens;
  int n_seqs;
  int max_count;        // most tokens any sequence brings in this step
  int window;           // 0 = all earlier keys
  float scale;
  // With splits > 1 the keys are cut into that many runs, each run is a work-group of its own that
  // leaves (output row, maximum, sum) in `partial` [rows][q_heads][splits][head_dim + 2], and a
  // second kernel joins them into `out`.  Decode: the runs of every sequence's keys, a row is a
  // sequence.  Prompts (bfloat16, heads of 64, no window): the runs of every query tile's keys, a
  // row is a token of the step.
  int splits;
  float* partial;
  // Decode (bfloat16 MFMA kernels) only: 0, or `out` is chunk-major with that many rows
  // (activation_offset in common.h); ldo is then not used.
  int out_rows;
  // 0, or keys are seen in chunks of that many positions, counted from position 0 of the sequence:
  // a query at position p sees the keys from p - p % chunk through p (and, with a window as well,
  // only those the window also holds).
  int chunk;
  // null, or one logit per query head that stands in every softmax's denominator beside the keys a
  // query sees: exp(sink[head]) is added once, unscaled, with no key and no value of its own (the
  // weights of a query's keys then add up to less than one).
  const float* sink;
};

// What a sink adds to a softmax's denominator that is kept relative to the maximum `top`.  The plain and
// the float32 decode kernels keep maxima as natural logarithms, the MFMA kernels in powers of two.
__device__ __forceinline__ float bt_sink_term(const float* sink, int head, float top) {
  return sink ? expf(sink[head] - top) : 0.f;
}
__device__ __forceinline__ float bt_sink_term_pow2(const float* sink, int head, float top) {
  return sink ? exp2f(sink[head] * 1.4426950408889634f - top) : 0.f;
}

// The first position a query at `pos` sees: the later of its window's and its chunk's first key.
// It never decreases as `pos` grows, so the first query of a run of queries has the lowest.
__host__ __device__ __forceinline__ int bt_first_seen(int pos, int window, int chunk) {
  int lo = 0;
  if (window > 0 && pos - window + 1 > lo) lo = pos - window + 1;
  if (chunk > 0 && pos - pos % chunk > lo) lo = pos - pos % chunk;
  return lo;
}
