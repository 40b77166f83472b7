// Kernels of the recurrent (state-space) mixers.  Everything that enters a recurrence is 32-bit:
// step sizes, decays, states, the sums over the state.  A sequence's state lives in its slot's row
// of the cache's per-sequence state area and is carried from step to step; a step may bring any
// number of a sequence's tokens, which are walked in order.
//   * causal convolution per channel with bias and silu; its last taps - 1 inputs are state
//   * dt projection: softplus(W low + b)
//   * selective scan (one state row per channel, one decay per state element), with the output gate
//   * scan with one decay per head and a state of [state, head size] (state-space duality form)
//   * gate, then RMS norm in equal parts
#include "host.h"
#include "scan.h"


// Brings rows t0 .. t0 + count - 1 of B and C (`state` columns each, row pitch `ld`, 32-bit offsets) into LDS
// as pairs, [count][NP] with zeros behind `state`; NP is a power of two.  A pass of the wave covers
// whole rows (64 / NP of them, or 1 / (NP / 64) of one), a lane keeps its column, and thirty-two passes'
// loads are issued before the first is stored: a loop of single loads would wait for memory once per
// element, and one that works its row and column out of a running index spends more instructions on
// that than the recurrence spends on a token.  `lane` numbers the THREADS threads that share the work.
template <int NP, int LOADS, int THREADS>
__device__ __forceinline__ void fill_pairs_ahead(float2* BC, const float* B, const float* C, int ld, int t0, int count,
                                                 int state, int lane) {
  constexpr int ROWS = NP >= THREADS ? 1 : THREADS / NP;     // rows a pass covers
  constexpr int COLS = NP >= THREADS ? NP / THREADS : 1;     // passes a row takes
  constexpr int AHEAD = COLS >= LOADS ? 1 : LOADS / COLS;    // row passes whose loads are in flight together
  const int lane_row = NP >= THREADS ? 0 : lane / NP, lane_col = NP >= THREADS ? lane : lane % NP;
  for (int r0 = 0; r0 < count; r0 += ROWS * AHEAD) {
    float2 got[AHEAD][COLS];
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      const int row = r0 + u * ROWS + lane_row;
      const int at = (t0 + min(row, count - 1)) * ld;
#pragma unroll
      for (int k = 0; k < COLS; ++k) {
        const int n = lane_col + THREADS * k;
        got[u][k] = (row < count && n < state) ? make_float2(B[at + n], C[at + n]) : make_float2(0.f, 0.f);
      }
    }
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      const int row = r0 + u * ROWS + lane_row;
#pragma unroll
      for (int k = 0; k < COLS; ++k)
        if (row < count) BC[row * NP + lane_col + THREADS * k] = got[u][k];
    }
  }
}

// (a step of single tokens has one row to bring: the short form spares it the long one's idle passes)
template <int NP, int THREADS>
__device__ __forceinline__ void fill_pairs(float2* BC, const float* B, const float* C, int ld, int t0, int count,
                                           int state, int lane) {
  constexpr int ROWS = NP >= THREADS ? 1 : THREADS / NP;
  if (count <= 2 * ROWS)
    fill_pairs_ahead<NP, 2, THREADS>(BC, B, C, ld, t0, count, state, lane);
  else
    fill_pairs_ahead<NP, 2048 / THREADS, THREADS>(BC, B, C, ld, t0, count, state, lane);
}

// ---------------------------------------------------------------------------------------------
struct CausalConvCall {
  int cast_dtype;         // element type of `cast`
  int tokens, n_seqs, channels, taps;
  int cast_cols;          // columns of `cast` written: the channels, then zeros
  const float* in;        // [tokens][ld_in]
  int64_t ld_in;
  const float* weight;    // [channels][taps]; the last tap meets the current token
  const float* bias;      // [channels], or null: none
  float* out;             // [tokens][ld_out] float32
  int64_t ld_out;
  void* cast;             // [tokens][ld_cast] the same in the products' type, or null
  int64_t ld_cast;
  float* state;           // slot s: [taps - 1][channels] at state + s * state_stride, oldest first
  int64_t state_stride;
  const int* tok_seq;
  const int* seq_off;     // [n_seqs + 1]
  const int* slots;       // [n_seqs]
  int act;                // what follows the sum: 0 silu, 1 nothing
};

// SHIFT: every sequence of the step brings one token (a decode step), so a (sequence, channel) pair
// belongs to one thread, which can also move the state on: no second kernel.
template <typename T, bool SHIFT>
__global__ void __launch_bounds__(256) causal_conv_kernel(CausalConvCall c) {
  const int t = blockIdx.x;
  const int ch = blockIdx.y * blockDim.x + threadIdx.x;
  T* cast = static_cast<T*>(c.cast);
  if (ch >= c.channels) {
    if (cast && ch < c.cast_cols) cast[(int64_t)t * c.ld_cast + ch] = from_float<T>(0.f);
    return;
  }
  const int seq = c.tok_seq[t];
  const int local = t - c.seq_off[seq];
  float* held = c.state + (int64_t)c.slots[seq] * c.state_stride;
  float sum = c.bias ? c.bias[ch] : 0.f;
  for (int j = 0; j < c.taps; ++j) {
    const int back = c.taps - 1 - j;
    const int src = local - back;
    const float u = src >= 0 ? c.in[(int64_t)(t - back) * c.ld_in + ch]
                             : held[(int64_t)(c.taps - 1 + src) * c.channels + ch];
    sum = fmaf(c.weight[(int64_t)ch * c.taps + j], u, sum);
  }
  const float y = c.act == 0 ? silu_f(sum) : sum;
  c.out[(int64_t)t * c.ld_out + ch] = y;
  if (cast) cast[(int64_t)t * c.ld_cast + ch] = from_float<T>(y);
  if (SHIFT) {
    for (int r = 0; r + 2 < c.taps; ++r) held[(int64_t)r * c.channels + ch] = held[(int64_t)(r + 1) * c.channels + ch];
    if (c.taps > 1) held[(int64_t)(c.taps - 2) * c.channels + ch] = c.in[(int64_t)t * c.ld_in + ch];
  }
}

// After the convolution: the state becomes the last taps - 1 inputs of each sequence.
__global__ void __launch_bounds__(256) conv_state_kernel(CausalConvCall c) {
  const int seq = blockIdx.x;
  const int ch = blockIdx.y * blockDim.x + threadIdx.x;
  if (ch >= c.channels) return;
  const int first = c.seq_off[seq], count = c.seq_off[seq + 1] - first;
  float* held = c.state + (int64_t)c.slots[seq] * c.state_stride;
  for (int r = 0; r < c.taps - 1; ++r) {
    const int src = count - (c.taps - 1) + r;
    // (an older input moves up: row r + count lies behind row r, and is read before it is written)
    held[(int64_t)r * c.channels + ch] = src >= 0 ? c.in[(int64_t)(first + src) * c.ld_in + ch]
                                                  : held[(int64_t)(r + count) * c.channels + ch];
  }
}

BT_EXPORT int bt_causal_conv_call(void* stream, const CausalConvCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->channels <= 0 || c->taps <= 0 || c->n_seqs <= 0)
    BT_REFUSE("causal_conv: %d channels, %d taps, %d sequences: all must be positive", c->channels, c->taps, c->n_seqs);
  if (!c->in || !c->weight || !c->out || !c->tok_seq || !c->seq_off || !c->slots || (c->taps > 1 && !c->state))
    BT_REFUSE("causal_conv: missing operand");
  if (c->act != 0 && c->act != 1) BT_REFUSE("causal_conv: unknown activation %d", c->act);
  if (c->ld_in < c->channels || c->ld_out < c->channels || (c->cast && (c->cast_cols < c->channels || c->ld_cast < c->cast_cols)))
    BT_REFUSE("causal_conv: the rows do not hold %d channels", c->channels);
  if (c->taps > 1 && c->state_stride < (int64_t)(c->taps - 1) * c->channels)
    BT_REFUSE("causal_conv: a slot's state of %lld elements does not hold %d inputs of %d channels",
              (long long)c->state_stride, c->taps - 1, c->channels);
  const int cols = c->cast && c->cast_cols > c->channels ? c->cast_cols : c->channels;
  dim3 grid(c->tokens, (cols + 255) / 256), block(256);
  if (c->tokens == c->n_seqs) {        // one token of every sequence
    if (c->cast_dtype == 0)
      hipLaunchKernelGGL((causal_conv_kernel<float, true>), grid, block, 0, (hipStream_t)stream, *c);
    else
      hipLaunchKernelGGL((causal_conv_kernel<bf16_t, true>), grid, block, 0, (hipStream_t)stream, *c);
    return bt_check_launch("causal_conv");
  }
  if (c->cast_dtype == 0)
    hipLaunchKernelGGL((causal_conv_kernel<float, false>), grid, block, 0, (hipStream_t)stream, *c);
  else
    hipLaunchKernelGGL((causal_conv_kernel<bf16_t, false>), grid, block, 0, (hipStream_t)stream, *c);
  int rc = bt_check_launch("causal_conv");
  if (rc || c->taps == 1) return rc;
  hipLaunchKernelGGL(conv_state_kernel, dim3(c->n_seqs, (c->channels + 255) / 256), block, 0, (hipStream_t)stream, *c);
  return bt_check_launch("causal_conv state");
}

// ---------------------------------------------------------------------------------------------
// out[t][c] = act(sum_r W[c][r] * low[t][r] + bias[c]), act the softplus (`act` 0), the sigmoid (1) or
// nothing (2); the rank is small.
struct DtProjectCall {
  int dtype;              // element type of W
  int tokens, channels, rank;
  const float* low;       // [tokens][ld_low]
  int64_t ld_low;
  const void* W;          // [channels][rank]
  const float* bias;      // [channels], or null: none
  float* out;             // [tokens][ld_out]
  int64_t ld_out;
  int act;                // 0: softplus, 1: sigmoid, 2: none
};

// TOKENS tokens share a work-group (their rows of `low` wait in LDS, every weight is read once for
// all of them); steps of few tokens take one token a work-group, which is more work-groups and a
// shorter chain in each.
template <typename T, int TOKENS>
__global__ void __launch_bounds__(256) dt_project_kernel(DtProjectCall c) {
  extern __shared__ float rows[];      // [TOKENS][rank]
  const int t0 = blockIdx.x * TOKENS;
  for (int e = threadIdx.x; e < TOKENS * c.rank; e += blockDim.x) {
    const int i = e / c.rank, r = e % c.rank;
    rows[e] = t0 + i < c.tokens ? c.low[(int64_t)(t0 + i) * c.ld_low + r] : 0.f;
  }
  __syncthreads();
  const int ch = blockIdx.y * blockDim.x + threadIdx.x;
  if (ch >= c.channels) return;
  const T* w = static_cast<const T*>(c.W) + (int64_t)ch * c.rank;
  float acc[TOKENS];
#pragma unroll
  for (int i = 0; i < TOKENS; ++i) acc[i] = 0.f;
#pragma unroll 8      // (eight of a thread's weights on their way at once)
  for (int r = 0; r < c.rank; ++r) {
    const float wv = to_float(w[r]);
#pragma unroll
    for (int i = 0; i < TOKENS; ++i) acc[i] = fmaf(wv, rows[i * c.rank + r], acc[i]);
  }
  const float b = c.bias ? c.bias[ch] : 0.f;
#pragma unroll
  for (int i = 0; i < TOKENS; ++i)
    if (t0 + i < c.tokens) {
      const float z = acc[i] + b;
      c.out[(int64_t)(t0 + i) * c.ld_out + ch] = c.act == 0 ? softplus_f(z) : (c.act == 1 ? 1.0f / (1.0f + expf(-z)) : z);
    }
}

template <typename T, int TOKENS>
static void launch_dt_project(hipStream_t stream, const DtProjectCall& c) {
  dim3 grid((c.tokens + TOKENS - 1) / TOKENS, (c.channels + 255) / 256), block(256);
  hipLaunchKernelGGL((dt_project_kernel<T, TOKENS>), grid, block, (size_t)TOKENS * c.rank * sizeof(float), stream, c);
}

BT_EXPORT int bt_dt_project_call(void* stream, const DtProjectCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->channels <= 0 || c->rank <= 0 || c->rank > 1024)
    BT_REFUSE("dt_project: %d channels from rank %d (1..1024)", c->channels, c->rank);
  if (!c->low || !c->W || !c->out || c->ld_low < c->rank || c->ld_out < c->channels)
    BT_REFUSE("dt_project: missing operand or rows too short");
  if (c->act < 0 || c->act > 2) BT_REFUSE("dt_project: unknown activation %d", c->act);
  hipStream_t s = (hipStream_t)stream;
  if (c->tokens <= 16) {
    if (c->dtype == 0) launch_dt_project<float, 1>(s, *c);
    else launch_dt_project<bf16_t, 1>(s, *c);
  } else {
    if (c->dtype == 0) launch_dt_project<float, 8>(s, *c);
    else launch_dt_project<bf16_t, 8>(s, *c);
  }
  return bt_check_launch("dt_project");
}

// ---------------------------------------------------------------------------------------------
// Selective scan.  Per channel c and state element n, token after token of a sequence:
//   S[c][n] <- exp(dt_c * A[c][n]) * S[c][n] + dt_c * x_c * B_n,   A = -exp(A_log)
//   y_c = sum_n S[c][n] * C_n + D_c * x_c;   out_c = y_c * silu(z_c)
// One wave per (8 channels, sequence): eight lanes share a channel, lane j of them owns the state
// elements j, j + 8, ... in registers (R of them).
struct SelectiveScanCall {
  int out_dtype;
  int tokens, n_seqs, channels, state;
  int out_cols;           // columns of out written: the channels, then zeros
  const float* x;         // [tokens][ld_x] after convolution and silu
  int64_t ld_x;
  const float* z;         // [tokens][ld_z] gate, pre-activation
  int64_t ld_z;
  const float* dt;        // [tokens][ld_dt] after softplus
  int64_t ld_dt;
  const float* B;         // [tokens][ld_bc]
  const float* C;         // [tokens][ld_bc]
  int64_t ld_bc;
  const float* A_log;     // [channels][state]
  const float* D;         // [channels]
  void* out;              // [tokens][ld_out]
  int64_t ld_out;
  float* S;               // slot s: [channels][state] at S + s * state_stride
  int64_t state_stride;
  const int* seq_off;
  const int* slots;
  // span > 0: long sequences are cut into spans of that many tokens which are scanned side by side
  // (see "Spans" below); max_count is the most tokens a sequence of the step brings, carry the room
  // for the spans' states: (tokens / span + 2 n_seqs + 1) blocks of channels * state + channels floats
  int span;
  int max_count;
  float* carry;
};

// LDS holds a run of `chunk` tokens' inputs (B and C rows padded to 8 R with zeros, and the wave's eight
// channels' dt, x and z), brought in with loads that are all in flight together: one round trip to
// memory per run of tokens instead of one per token, which is what bounds a recurrence.
// phase 0: whole sequences, from and to the slot's state.  1: spans from zero, leaving E_k and the sum
// of dt.  3: spans from the carried states, writing outputs.
template <typename T, int R>
__global__ void __launch_bounds__(64) selective_scan_kernel(SelectiveScanCall c, int chunk, int phase) {
  extern __shared__ float lds[];
  constexpr int NP = 8 * R;
  float2* BC = reinterpret_cast<float2*>(lds);   // [chunk][NP] pairs (B, C): one 8-byte read for both
  float* dts = lds + (size_t)chunk * NP * 2;     // [chunk][8]
  float* xs = dts + (size_t)chunk * 8;
  float* zs = xs + (size_t)chunk * 8;
  const int lane = threadIdx.x, sub = lane & 7, cl = lane >> 3;
  const int ch = blockIdx.x * 8 + cl, seq = blockIdx.y;
  const bool live = ch < c.channels;
  const int chs = live ? ch : c.channels - 1;        // idle lanes read a valid channel and write nothing
  int first = c.seq_off[seq], last = c.seq_off[seq + 1];
  const int seq_last = last, part = blockIdx.z;
  const int64_t per_span = (int64_t)c.channels * c.state + c.channels;
  float* mine = nullptr;                             // this span's block of the carry
  if (phase) {
    first += part * c.span;
    if (first >= seq_last) return;
    last = min(first + c.span, seq_last);
    mine = c.carry + span_block(c.seq_off, seq, c.span, part) * per_span;
  }
  float* held = c.S + (int64_t)c.slots[seq] * c.state_stride + (int64_t)chs * c.state;
  const float* start = phase == 3 ? mine - per_span + (int64_t)chs * c.state : held;
  float A[R], S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int n = sub + 8 * r;
    A[r] = n < c.state ? -expf(c.A_log[(int64_t)chs * c.state + n]) : 0.f;
    S[r] = (n < c.state && phase != 1) ? start[n] : 0.f;
  }
  float dt_sum = 0.f;
  const float Dc = c.D[chs];
  T* out = static_cast<T*>(c.out);
  for (int t0 = first; t0 < last; t0 += chunk) {
    const int count = min(chunk, last - t0);
    __syncthreads();
    // (sixteen elements of a lane at a time, all loads issued before the first is stored; with the
    // short rows of this scan, 8 to 32 pairs, the running index measured faster than `fill_pairs`)
    for (int e0 = lane; e0 < count * NP; e0 += 64 * 16) {
      float2 held_bc[16];
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const int e = e0 + 64 * k, i = e / NP, n = e % NP;
        held_bc[k] = (e < count * NP && n < c.state)
                         ? make_float2(c.B[(int64_t)(t0 + i) * c.ld_bc + n], c.C[(int64_t)(t0 + i) * c.ld_bc + n])
                         : make_float2(0.f, 0.f);
      }
#pragma unroll
      for (int k = 0; k < 16; ++k)
        if (e0 + 64 * k < count * NP) BC[e0 + 64 * k] = held_bc[k];
    }
    {
      float held_in[8][3];
#pragma unroll
      for (int k = 0; k < 8; ++k) {          // count <= 64 tokens of 8 channels: at most eight elements a lane
        const int e = lane + 64 * k, i = min(e >> 3, count - 1);
        const int q = min((int)blockIdx.x * 8 + (e & 7), c.channels - 1);
        held_in[k][0] = c.dt[(int64_t)(t0 + i) * c.ld_dt + q];
        held_in[k][1] = c.x[(int64_t)(t0 + i) * c.ld_x + q];
        held_in[k][2] = c.z[(int64_t)(t0 + i) * c.ld_z + q];
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int e = lane + 64 * k;
        if (e < count * 8) {
          dts[e] = held_in[k][0];
          xs[e] = held_in[k][1];
          zs[e] = held_in[k][2];
        }
      }
    }
    __syncthreads();
    auto token = [&](int i) {
      const float dt = dts[i * 8 + cl], xv = xs[i * 8 + cl];
      const float dx = dt * xv;
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const float2 bc = BC[i * NP + sub + 8 * r];
        S[r] = expf(dt * A[r]) * S[r] + dx * bc.x;
        acc = fmaf(S[r], bc.y, acc);
      }
      dt_sum += dt;
      if (phase == 1) return;                        // only the state is wanted
      acc = sum_of_8_lanes(acc);
      if (live && sub == 0)
        out[(int64_t)(t0 + i) * c.ld_out + ch] = from_float<T>((acc + Dc * xv) * silu_f(zs[i * 8 + cl]));
    };
    // four tokens at a time, written out: their reads from LDS, exponentials and sums are in flight
    // together and only the state ties them (the lane sums keep the compiler from unrolling a loop
    // whose length it does not know)
    int i = 0;
    for (; i + 4 <= count; i += 4) {
#pragma unroll
      for (int u = 0; u < 4; ++u) token(i + u);
    }
    for (; i < count; ++i) token(i);
  }
  if (phase == 1) {
    if (live) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int n = sub + 8 * r;
        if (n < c.state) mine[(int64_t)ch * c.state + n] = S[r];
      }
      if (sub == 0) mine[(int64_t)c.channels * c.state + ch] = dt_sum;
    }
    return;
  }
  if (live && phase == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = sub + 8 * r;
      if (n < c.state) held[n] = S[r];
    }
  }
  // the columns behind the last channel, which the next product reads as zeros
  if (blockIdx.x == 0)
    for (int t = first; t < last; ++t)
      for (int col = c.channels + lane; col < c.out_cols; col += 64) out[(int64_t)t * c.ld_out + col] = from_float<T>(0.f);
}

// C_k = exp(A * sum of dt of span k) * C_(k-1) + E_k along every sequence, in place; C_(-1), the state the
// sequence came with, is kept in front of its spans, and the last C goes into the slot.
__global__ void __launch_bounds__(256) selective_carry_kernel(SelectiveScanCall c) {
  const int seq = blockIdx.y;
  const int64_t index = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, size = (int64_t)c.channels * c.state;
  if (index >= size) return;
  const int count = c.seq_off[seq + 1] - c.seq_off[seq];
  const int spans = (count + c.span - 1) / c.span;
  const int64_t per_span = size + c.channels;
  float* block = c.carry + span_block(c.seq_off, seq, c.span, 0) * per_span;
  float* slot = c.S + (int64_t)c.slots[seq] * c.state_stride;
  float state = slot[index];
  (block - per_span)[index] = state;
  const float A = -expf(c.A_log[index]);
  const int ch = (int)(index / c.state);
  for (int k = 0; k < spans; ++k, block += per_span) {
    state = expf(A * block[size + ch]) * state + block[index];
    block[index] = state;
  }
  slot[index] = state;
}

template <typename T, int R>
static void launch_selective_scan_r(hipStream_t stream, const SelectiveScanCall& c) {
  const int per_token = 2 * 8 * R + 24;
  dim3 block(64);
  const int span = span_tokens(c.span, c.max_count, c.carry, (int64_t)((c.channels + 7) / 8) * c.n_seqs, 2);
  if (span > 0) {
    SelectiveScanCall cut = c;
    cut.span = span;
    const int chunk = scan_chunk(per_token, span);
    const int spans = (c.max_count + span - 1) / span;
    dim3 grid((c.channels + 7) / 8, c.n_seqs, spans);
    const size_t lds = (size_t)chunk * per_token * sizeof(float);
    hipLaunchKernelGGL((selective_scan_kernel<T, R>), grid, block, lds, stream, cut, chunk, 1);
    hipLaunchKernelGGL(selective_carry_kernel, dim3((c.channels * c.state + 255) / 256, c.n_seqs), dim3(256), 0, stream, cut);
    hipLaunchKernelGGL((selective_scan_kernel<T, R>), grid, block, lds, stream, cut, chunk, 3);
    return;
  }
  const int chunk = scan_chunk(per_token, c.tokens);
  dim3 grid((c.channels + 7) / 8, c.n_seqs);
  hipLaunchKernelGGL((selective_scan_kernel<T, R>), grid, block, (size_t)chunk * per_token * sizeof(float), stream, c, chunk, 0);
}

template <typename T>
static int launch_selective_scan(hipStream_t stream, const SelectiveScanCall& c) {
  const int per = (c.state + 7) / 8;
  if (per <= 1) launch_selective_scan_r<T, 1>(stream, c);
  else if (per <= 2) launch_selective_scan_r<T, 2>(stream, c);
  else if (per <= 4) launch_selective_scan_r<T, 4>(stream, c);
  else if (per <= 8) launch_selective_scan_r<T, 8>(stream, c);
  else if (per <= 16) launch_selective_scan_r<T, 16>(stream, c);
  else launch_selective_scan_r<T, 32>(stream, c);
  return bt_check_launch("selective_scan");
}

BT_EXPORT int bt_selective_scan_call(void* stream, const SelectiveScanCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->channels <= 0 || c->state <= 0 || c->state > 256 || c->n_seqs <= 0)
    BT_REFUSE("selective_scan: %d channels with %d state elements (1..256), %d sequences", c->channels, c->state, c->n_seqs);
  if (!c->x || !c->z || !c->dt || !c->B || !c->C || !c->A_log || !c->D || !c->out || !c->S || !c->seq_off || !c->slots)
    BT_REFUSE("selective_scan: missing operand");
  if (c->ld_x < c->channels || c->ld_z < c->channels || c->ld_dt < c->channels || c->ld_bc < c->state ||
      c->out_cols < c->channels || c->ld_out < c->out_cols || c->state_stride < (int64_t)c->channels * c->state)
    BT_REFUSE("selective_scan: rows or state too short for %d channels of %d", c->channels, c->state);
  return c->out_dtype == 0 ? launch_selective_scan<float>((hipStream_t)stream, *c)
                           : launch_selective_scan<bf16_t>((hipStream_t)stream, *c);
}

// ---------------------------------------------------------------------------------------------
// Scan with one decay per head.  Per head h (its group g = h / (heads / groups)), token after token:
//   dt = softplus(dt_raw_h + dt_bias_h);   a = exp(-exp(A_log_h) * dt)
//   S_h[n][p] <- a * S_h[n][p] + dt * B_g[n] * x_h[p];   y_h[p] = sum_n S_h[n][p] * C_g[n] + D_h * x_h[p]
// One wave per (4 channels p of a head, sequence): sixteen lanes share a channel, lane j of them owns
// the state elements j, j + 16, ... in registers.
struct HeadScanCall {
  int tokens, n_seqs, heads, vdim, state, groups;
  const float* x;         // [tokens][ld]: head h at columns h * vdim (after convolution and silu)
  const float* B;         // [tokens][ld]: group g at columns g * state
  const float* C;
  int64_t ld;
  const float* dt_raw;    // [tokens][ld_dt]: one per head, before bias and softplus
  int64_t ld_dt;
  const float* dt_bias;   // [heads]
  const float* A_log;     // [heads]
  const float* D;         // [heads]
  float* y;               // [tokens][ld_y] float32: head h at columns h * vdim
  int64_t ld_y;
  float* S;               // slot s: [heads][vdim / 4 rounded up][state][4] at S + s * state_stride
  int64_t state_stride;
  const int* seq_off;
  const int* slots;
  // spans, as in SelectiveScanCall: a block of the carry holds a state (in the slot's layout) and, behind
  // it, one number a head: the sum over the span of the logarithms of its decays
  int span;
  int max_count;
  float* carry;
};

// The state of a slot is laid out for this kernel's lanes: [heads][tiles of 4 channels][state][4], so
// that a wave's load of one register's worth of state (16 state elements by 4 channels) is 256
// contiguous bytes.  Nobody else reads it; a new sequence's state is all zeros in any layout.
// A work-group is four waves, each with four channels of the same head: they share the run of B and C in
// LDS (every wave bringing a quarter of it in) and have one SIMD each.
#define HS_WAVES 4

template <int R, int PHASE>
__global__ void __launch_bounds__(64 * HS_WAVES) head_scan_kernel(HeadScanCall c, int chunk, int spans, int tiles) {
  extern __shared__ float lds[];
  constexpr int NP = 16 * R;
  float2* BC = reinterpret_cast<float2*>(lds);                              // [chunk][NP] pairs (B, C): one 8-byte read for both
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, sub = lane & 15, pl = lane >> 4;
  // [waves][chunk][4]: a token and channel's dt * x, D * x, decay, log decay
  float4* tok = reinterpret_cast<float4*>(lds + (size_t)chunk * NP * 2) + (size_t)wave * chunk * 4;
  const int tile = min((int)blockIdx.x * HS_WAVES + wave, tiles - 1), head = blockIdx.y;
  const bool works = (int)blockIdx.x * HS_WAVES + wave < tiles;          // (a wave without a tile only helps to bring B and C in)
  const int seq = blockIdx.z / spans, part = blockIdx.z % spans;
  const int p = tile * 4 + pl;
  const bool live = works && p < c.vdim;
  const int group = head / (c.heads / c.groups);
  int first = c.seq_off[seq], last = c.seq_off[seq + 1];
  const int seq_last = last;
  const int64_t state_size = (int64_t)c.heads * tiles * c.state * 4, per_span = state_size + c.heads;
  const int64_t in_state = ((int64_t)head * tiles + tile) * c.state * 4 + pl;
  float* mine = nullptr;                             // this span's block of the carry
  if (PHASE) {
    first += part * c.span;
    if (first >= seq_last) return;                   // (the whole work-group: it is one span's)
    last = min(first + c.span, seq_last);
    mine = c.carry + span_block(c.seq_off, seq, c.span, part) * per_span;
  }
  float* held = c.S + (int64_t)c.slots[seq] * c.state_stride + in_state;
  const float* start = PHASE == 3 ? mine - per_span + in_state : held;
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int n = sub + 16 * r;
    S[r] = (n < c.state && PHASE != 1) ? start[(int64_t)n * 4] : 0.f;
  }
  float log_decay = 0.f;
  const float rate = -expf(c.A_log[head]), bias = c.dt_bias[head], Dh = c.D[head];
  const float* Bg = c.B + group * c.state;
  const float* Cg = c.C + group * c.state;
  float* ycol = c.y + head * c.vdim + (live ? p : 0);
  for (int t0 = first; t0 < last; t0 += chunk) {
    const int count = min(chunk, last - t0);
    __syncthreads();
    fill_pairs<NP, 64 * HS_WAVES>(BC, Bg, Cg, (int)c.ld, t0, count, c.state, (int)threadIdx.x);
    for (int e = lane; e < count * 4; e += 64) {
      const int i = e >> 2, q = tile * 4 + (e & 3);
      const float xv = q < c.vdim ? c.x[(int64_t)(t0 + i) * c.ld + head * c.vdim + q] : 0.f;
      const float step = softplus_f(c.dt_raw[(int64_t)(t0 + i) * c.ld_dt + head] + bias);
      tok[e] = make_float4(step * xv, Dh * xv, expf(rate * step), rate * step);
    }
    __syncthreads();
    if (!works) continue;
    // one token: the state moves on; the channel's output (in every lane of its sixteen) is returned
    auto token = [&](int i) -> float {
      const float4 in = tok[i * 4 + pl];
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const float2 bc = BC[i * NP + sub + 16 * r];
        S[r] = fmaf(in.z, S[r], in.x * bc.x);
        acc = fmaf(S[r], bc.y, acc);
      }
      if (PHASE == 1) {
        log_decay += in.w;
        return 0.f;                                  // only the state is wanted
      }
      return sum_of_16_lanes(acc) + in.y;
    };
    // Sixteen tokens at a time, written out: their reads from LDS and sums are in flight together and
    // only the state ties them (the lane sums keep the compiler from unrolling a loop whose length it
    // does not know); lane j of a channel's sixteen keeps the j-th of them, and one store writes all.
    int i = 0;
    for (; i + 16 <= count; i += 16) {
      float kept = 0.f;
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const float y = token(i + u);
        kept = sub == u ? y : kept;
      }
      if (PHASE != 1 && live) ycol[(int64_t)(t0 + i + sub) * c.ld_y] = kept;
    }
    for (; i < count; ++i) {
      const float y = token(i);
      if (PHASE != 1 && live && sub == 0) ycol[(int64_t)(t0 + i) * c.ld_y] = y;
    }
  }
  if (!works) return;
  if (PHASE == 1) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = sub + 16 * r;
      if (n < c.state) mine[in_state + (int64_t)n * 4] = S[r];
    }
    if (tile == 0 && lane == 0) mine[state_size + head] = log_decay;
    return;
  }
  if (PHASE == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = sub + 16 * r;
      if (n < c.state) held[(int64_t)n * 4] = S[r];
    }
  }
}

// C_k = exp(sum of the span's log decays) * C_(k-1) + E_k along every sequence, in place (see selective_carry_kernel).
__global__ void __launch_bounds__(256) head_carry_kernel(HeadScanCall c, int tiles) {
  const int seq = blockIdx.y;
  const int64_t per_head = (int64_t)tiles * c.state * 4, size = per_head * c.heads;
  const int64_t index = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= size) return;
  const int count = c.seq_off[seq + 1] - c.seq_off[seq];
  const int spans = (count + c.span - 1) / c.span;
  const int64_t per_span = size + c.heads;
  float* block = c.carry + span_block(c.seq_off, seq, c.span, 0) * per_span;
  float* slot = c.S + (int64_t)c.slots[seq] * c.state_stride;
  float state = slot[index];
  (block - per_span)[index] = state;
  const int head = (int)(index / per_head);
  for (int k = 0; k < spans; ++k, block += per_span) {
    state = expf(block[size + head]) * state + block[index];
    block[index] = state;
  }
  slot[index] = state;
}

template <int R>
static void launch_head_scan_r(hipStream_t stream, const HeadScanCall& c) {
  const int per_token = 2 * 16 * R + 16 * HS_WAVES;
  const int tiles = (c.vdim + 3) / 4, groups = (tiles + HS_WAVES - 1) / HS_WAVES;
  dim3 block(64 * HS_WAVES);
  const int span = span_tokens(c.span, c.max_count, c.carry, (int64_t)tiles * c.heads * c.n_seqs, 1);
  if (span > 0) {
    HeadScanCall cut = c;
    cut.span = span;
    const int chunk = scan_chunk(per_token, span);
    const int spans = (c.max_count + span - 1) / span;
    dim3 grid(groups, c.heads, c.n_seqs * spans);
    const size_t lds = (size_t)chunk * per_token * sizeof(float);
    hipLaunchKernelGGL((head_scan_kernel<R, 1>), grid, block, lds, stream, cut, chunk, spans, tiles);
    const int64_t size = (int64_t)c.heads * tiles * c.state * 4;
    hipLaunchKernelGGL(head_carry_kernel, dim3((unsigned)((size + 255) / 256), c.n_seqs), dim3(256), 0, stream, cut, tiles);
    hipLaunchKernelGGL((head_scan_kernel<R, 3>), grid, block, lds, stream, cut, chunk, spans, tiles);
    return;
  }
  const int chunk = scan_chunk(per_token, c.tokens);
  dim3 grid(groups, c.heads, c.n_seqs);
  hipLaunchKernelGGL((head_scan_kernel<R, 0>), grid, block, (size_t)chunk * per_token * sizeof(float), stream, c, chunk, 1, tiles);
}

BT_EXPORT int bt_head_scan_call(void* stream, const HeadScanCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->heads <= 0 || c->vdim <= 0 || c->state <= 0 || c->state > 256 || c->groups <= 0 || c->heads % c->groups != 0 || c->n_seqs <= 0)
    BT_REFUSE("head_scan: %d heads of %d in %d groups with %d state elements (1..256)", c->heads, c->vdim, c->groups, c->state);
  if (!c->x || !c->B || !c->C || !c->dt_raw || !c->dt_bias || !c->A_log || !c->D || !c->y || !c->S || !c->seq_off || !c->slots)
    BT_REFUSE("head_scan: missing operand");
  if (c->ld_dt < c->heads || c->ld_y < (int64_t)c->heads * c->vdim ||
      c->state_stride < (int64_t)c->heads * c->state * ((c->vdim + 3) / 4 * 4))
    BT_REFUSE("head_scan: rows or state too short for %d heads of %d", c->heads, c->vdim);
  if ((int64_t)c->tokens * c->ld >= (int64_t)1 << 31) BT_REFUSE("head_scan: the rows of B and C are addressed with 32 bits");
  hipStream_t s = (hipStream_t)stream;
  const int per = (c->state + 15) / 16;
  if (per <= 1) launch_head_scan_r<1>(s, *c);
  else if (per <= 2) launch_head_scan_r<2>(s, *c);
  else if (per <= 4) launch_head_scan_r<4>(s, *c);
  else if (per <= 8) launch_head_scan_r<8>(s, *c);
  else launch_head_scan_r<16>(s, *c);
  return bt_check_launch("head_scan");
}

// ---------------------------------------------------------------------------------------------
// v = y * silu(z); out = v / sqrt(mean(v^2) + eps) * weight, the mean over each of `parts` equal
// parts of the row on its own.
struct GatedNormCall {
  int out_dtype;
  int tokens, channels, parts;
  int out_cols;           // columns of out written: the channels, then zeros
  float eps;
  const float* y;         // [tokens][ld_y]
  int64_t ld_y;
  const float* z;         // [tokens][ld_z] gate, pre-activation
  int64_t ld_z;
  const float* weight;    // [channels]
  void* out;              // [tokens][ld_out]
  int64_t ld_out;
};

template <typename T>
__global__ void __launch_bounds__(256) gated_norm_kernel(GatedNormCall c) {
  extern __shared__ float row_buf[];
  __shared__ float scratch[32];
  const int t = blockIdx.x, part = blockIdx.y;
  const int n = c.channels / c.parts, base = part * n;
  float partial = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = c.y[(int64_t)t * c.ld_y + base + i] * silu_f(c.z[(int64_t)t * c.ld_z + base + i]);
    row_buf[i] = v;
    partial += v * v;
  }
  const float rstd = 1.0f / sqrtf(block_sum(partial, scratch) / (float)n + c.eps);
  T* out = static_cast<T*>(c.out) + (int64_t)t * c.ld_out;
  for (int i = threadIdx.x; i < n; i += blockDim.x) out[base + i] = from_float<T>(row_buf[i] * rstd * c.weight[base + i]);
  if (part == 0)
    for (int col = c.channels + threadIdx.x; col < c.out_cols; col += blockDim.x) out[col] = from_float<T>(0.f);
}

BT_EXPORT int bt_gated_norm_call(void* stream, const GatedNormCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->channels <= 0 || c->parts <= 0 || c->channels % c->parts != 0 || c->channels / c->parts > 15360)
    BT_REFUSE("gated_norm: %d channels in %d equal parts (each up to 15360)", c->channels, c->parts);
  if (!c->y || !c->z || !c->weight || !c->out || c->ld_y < c->channels || c->ld_z < c->channels ||
      c->out_cols < c->channels || c->ld_out < c->out_cols)
    BT_REFUSE("gated_norm: missing operand or rows too short");
  dim3 grid(c->tokens, c->parts), block(256);
  size_t lds = (size_t)(c->channels / c->parts) * sizeof(float);
  if (c->out_dtype == 0)
    hipLaunchKernelGGL(gated_norm_kernel<float>, grid, block, lds, (hipStream_t)stream, *c);
  else
    hipLaunchKernelGGL(gated_norm_kernel<bf16_t>, grid, block, lds, (hipStream_t)stream, *c);
  return bt_check_launch("gated_norm");
}
