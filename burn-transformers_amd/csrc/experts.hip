// Kernels of the routed feed-forward (a mixture of gated experts).
//   * route: per token the router's logits (32-bit, from 32-bit router weights), their softmax over
//     all experts, the choice of `top` experts by score + correction, restricted to the best `keep`
//     of `groups` equal groups of neighbouring experts (a group's score is its best corrected
//     score), and the chosen experts' softmax scores divided by their sum.  The result is a dense
//     row of weights per token, zero where an expert was not chosen.  Optionally the sigmoid gate
//     of an expert that every token uses (one number per token).
//   * gated activation: hidden = weight * silu(gate) * up for every expert side by side (and the
//     always-on expert with its sigmoid gate as weight), so that ONE product with the experts' down
//     matrices laid side by side gives the weighted sum of their outputs; experts whose output is
//     their input ("identity experts", the last router outputs) leave weight * h as 32-bit rows.
// A router may differ in three ways (`score`, `group_rank`, `normalize`): scores that are the
// logits' sigmoids instead of their softmax, a group's score that is the sum of its `group_rank` best
// instead of its best, and weights that are the chosen experts' scores as they are instead of over
// their sum.  The experts' activation (`act`) is silu(g) * u, or with a `limit`:
// g' = min(g, limit), u' = clamp(u, -limit, limit), g' * sigmoid(alpha * g') * (u' + 1).
// Ties between equal scores go to the lower index.
#include "host.h"

#define ROUTE_THREADS 1024
#define ROUTE_MAX_EXPERTS 1024

struct RouteCall {
  int dtype;                // element type of `h`: 0 float32, 1 bfloat16
  int tokens, width;
  int experts;              // router outputs: experts with tensors and identity experts together
  int top;
  int groups, keep;         // groups <= 1: every expert can be chosen
  const void* h;            // [tokens][ldh]
  int64_t ldh;
  const float* W;           // [experts][width] float32
  const float* correction;  // [experts] or null: added to the scores for the choice only
  const float* gate_w;      // [width] float32 or null
  float* weights;           // [tokens][experts]
  float* gate;              // [tokens]: sigmoid(gate_w . h), or null
  int score;                // 0: softmax over all experts; 1: each logit's sigmoid
  int group_rank;           // a group's score is the sum of its so many best (corrected) scores; 0 or 1: its best
  int normalize;            // 1: the chosen experts' scores over their sum; 0: the scores as they are
};

// The best (value, index) of a wave; among equal values the lowest index.  Every lane gets it.
__device__ __forceinline__ void wave_best(float& value, int& index) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float other = __shfl_xor(value, o, 64);
    const int other_index = __shfl_xor(index, o, 64);
    if (other > value || (other == value && other_index < index)) { value = other; index = other_index; }
  }
}

// One work-group of sixteen waves per token.  Logits: a wave takes whole outputs (two at a time, the
// outputs dealt round the waves), its lanes the columns, sixteen a turn; nothing of a turn's loads stands
// behind a branch of its own, so all of them are in flight together, every wave's at once: the
// logits cost one round trip to memory and a wave reduction, and no sum crosses waves.  (Columns
// dealt to the threads and sixteen outputs' sums met through LDS, batch after batch, took 6 us a batch
// of sixteen outputs: a decode step has few tokens, and a kernel's time is the chain of its waits.)
// Everything after the logits is the first wave's alone, the experts dealt to its lanes, maxima and
// choices as wave reductions: no barrier, no serial scan.
#define ROUTE_OUTPUTS 2         // outputs whose sums a wave carries at once
#define ROUTE_COLUMNS 16        // columns of a lane and turn

template <typename T>
__global__ void __launch_bounds__(ROUTE_THREADS) route_kernel(RouteCall c) {
  __shared__ float score[ROUTE_MAX_EXPERTS];      // logits, then softmax scores
  __shared__ float choice[ROUTE_MAX_EXPERTS];     // scores with the correction; +inf once taken, -inf where shut out
  __shared__ float gate_sum;
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const T* h = static_cast<const T*>(c.h) + (int64_t)t * c.ldh;
  const int outputs = c.experts + (c.gate_w ? 1 : 0);
  const int waves = blockDim.x >> 6;              // sixteen in steps of few tokens, four where tokens fill the chip anyway
  // the corrections of this lane's first experts are asked for now, with the first loads
  float early_correction[4] = {0.f, 0.f, 0.f, 0.f};
  if (wave == 0 && c.correction)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (lane + 64 * j < c.experts) early_correction[j] = c.correction[lane + 64 * j];
  for (int first = wave; first < outputs; first += waves * ROUTE_OUTPUTS) {
    float sums[ROUTE_OUTPUTS];
    const float* rows[ROUTE_OUTPUTS];               // an output beyond the last reads the last one's row and is dropped
#pragma unroll
    for (int j = 0; j < ROUTE_OUTPUTS; ++j) {
      sums[j] = 0.f;
      const int e = first + waves * j < outputs ? first + waves * j : outputs - 1;
      rows[j] = e < c.experts ? c.W + (int64_t)e * c.width : c.gate_w;
    }
    for (int col0 = lane; col0 < c.width; col0 += 64 * ROUTE_COLUMNS) {
      int cc[ROUTE_COLUMNS];
      float xs[ROUTE_COLUMNS];
#pragma unroll
      for (int u = 0; u < ROUTE_COLUMNS; ++u) {
        const int col = col0 + 64 * u;
        cc[u] = col < c.width ? col : 0;
        xs[u] = to_float(h[cc[u]]);
      }
      float ws[ROUTE_OUTPUTS][ROUTE_COLUMNS];
#pragma unroll
      for (int j = 0; j < ROUTE_OUTPUTS; ++j)
#pragma unroll
        for (int u = 0; u < ROUTE_COLUMNS; ++u) ws[j][u] = rows[j][cc[u]];
#pragma unroll
      for (int u = 0; u < ROUTE_COLUMNS; ++u) xs[u] = col0 + 64 * u < c.width ? xs[u] : 0.f;
#pragma unroll
      for (int j = 0; j < ROUTE_OUTPUTS; ++j)
#pragma unroll
        for (int u = 0; u < ROUTE_COLUMNS; ++u) sums[j] = fmaf(ws[j][u], xs[u], sums[j]);
    }
#pragma unroll
    for (int j = 0; j < ROUTE_OUTPUTS; ++j) {
      const float sum = wave_sum(sums[j]);
      const int e = first + waves * j;
      if (lane == 0 && e < outputs) {
        if (e < c.experts) score[e] = sum;
        else gate_sum = sum;                         // (stored at the end: nothing waits for a store meanwhile)
      }
    }
  }
  __syncthreads();
  if (wave != 0) return;
  float top_logit = -INFINITY;
  for (int e = lane; e < c.experts; e += 64) top_logit = fmaxf(top_logit, score[e]);
  top_logit = wave_max(top_logit);
  float total = 0.f;
  for (int e = lane; e < c.experts; e += 64) total += expf(score[e] - top_logit);
  total = wave_sum(total);
  float* weights = c.weights + (int64_t)t * c.experts;
  for (int e = lane, j = 0; e < c.experts; e += 64, ++j) {     // a lane keeps to its own experts: no other lane reads them yet
    const float s = c.score == 1 ? 1.0f / (1.0f + expf(-score[e])) : expf(score[e] - top_logit) / total;
    score[e] = s;
    choice[e] = s + (c.correction ? (j < 4 ? early_correction[j < 4 ? j : 0] : c.correction[e]) : 0.f);
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if (c.groups > 1) {
    // a group's score is its best corrected score; the best `keep` groups stay open, the experts of
    // the others are shut out (minus infinity, since corrected scores may be negative).  Lane g
    // holds group g (at most 64 groups).
    const int per = c.experts / c.groups;
    float group_score = -INFINITY;
    if (lane < c.groups) {
      if (c.group_rank <= 1) {
        for (int i = 0; i < per; ++i) group_score = fmaxf(group_score, choice[lane * per + i]);
      } else {
        // the sum of the group's `group_rank` best: best after best, each below the one before it or
        // an equal one at a higher index
        float last = INFINITY;
        int last_index = -1;
        group_score = 0.f;
        for (int r = 0; r < c.group_rank && r < per; ++r) {
          float best = -INFINITY;
          int best_index = -1;
          for (int i = 0; i < per; ++i) {
            const float v = choice[lane * per + i];
            const bool left = v < last || (v == last && i > last_index);
            if (left && (best_index < 0 || v > best)) { best = v; best_index = i; }
          }
          group_score += best;
          last = best;
          last_index = best_index;
        }
      }
    }
    bool open = false;
    for (int kept = 0; kept < c.keep; ++kept) {
      float value = (lane < c.groups && !open) ? group_score : -INFINITY;
      int index = (lane < c.groups && !open) ? lane : 0x7fffffff;
      // (a group whose score is minus infinity itself still ranks before no group at all)
      unsigned long long candidates = __builtin_amdgcn_ballot_w64(lane < c.groups && !open);
      wave_best(value, index);
      if (index == 0x7fffffff) index = __builtin_ctzll(candidates);
      if (lane == index) open = true;
    }
    if (lane < c.groups && !open)
      for (int i = 0; i < per; ++i) choice[lane * per + i] = -INFINITY;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  float sum = 0.f;
  for (int k = 0; k < c.top; ++k) {
    float value = -INFINITY;
    int index = 0x7fffffff;
    for (int e = lane; e < c.experts; e += 64) {
      const float v = choice[e];
      if (v > value && v != INFINITY) { value = v; index = e; }     // (ascending e: the lowest index among equals; +inf: taken)
    }
    wave_best(value, index);
    if (index == 0x7fffffff) break;                // (nothing left to choose: refused on the host)
    if (lane == (index & 63)) choice[index] = INFINITY;            // taken: its owner marks it
    sum += score[index];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  // the one store of a lane's experts: the chosen ones' scores over their sum, zero elsewhere
  const float inverse = c.normalize ? 1.0f / (sum + 1e-20f) : 1.0f;
  for (int e = lane; e < c.experts; e += 64) weights[e] = choice[e] == INFINITY ? score[e] * inverse : 0.f;
  if (c.gate_w && lane == 0) c.gate[t] = 1.0f / (1.0f + expf(-gate_sum));
}

BT_EXPORT int bt_route_call(void* stream, const RouteCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->experts <= 0 || c->experts > ROUTE_MAX_EXPERTS) BT_REFUSE("route: %d experts outside 1..%d", c->experts, ROUTE_MAX_EXPERTS);
  if (c->top <= 0 || c->top > c->experts || c->top > 64) BT_REFUSE("route: %d of %d experts a token (at most 64)", c->top, c->experts);
  if (c->groups > 1) {
    if (c->groups > 64 || c->experts % c->groups != 0 || c->keep <= 0 || c->keep > c->groups)
      BT_REFUSE("route: %d groups (at most 64) must divide %d experts, and 1..groups of them stay open, not %d", c->groups, c->experts, c->keep);
    if (c->keep * (c->experts / c->groups) < c->top)
      BT_REFUSE("route: %d open groups of %d experts cannot give %d experts", c->keep, c->experts / c->groups, c->top);
  }
  if (c->width <= 0) BT_REFUSE("route: width %d must be positive", c->width);
  if ((c->score != 0 && c->score != 1) || c->group_rank < 0 || (c->normalize != 0 && c->normalize != 1))
    BT_REFUSE("route: score %d, group_rank %d, normalize %d: not a router this kernel knows", c->score, c->group_rank, c->normalize);
  if (!c->h || !c->W || !c->weights || (c->gate_w && !c->gate)) BT_REFUSE("route: missing operand");
  // (measured at 2,048 tokens of width 2,048: 32 us with sixteen waves a token, 18 with four)
  dim3 grid(c->tokens), block(c->tokens <= 256 ? ROUTE_THREADS : 256);
  if (c->dtype == 0)
    hipLaunchKernelGGL(route_kernel<float>, grid, block, 0, (hipStream_t)stream, *c);
  else
    hipLaunchKernelGGL(route_kernel<bf16_t>, grid, block, 0, (hipStream_t)stream, *c);
  return bt_check_launch("route");
}

struct GatedExpertsCall {
  int dtype;                // element type of `gu`, `hidden` and `h`
  int tokens;
  int experts;              // experts with tensors, each `ff` wide
  int ff;
  int shared_ff;            // width of the expert every token uses; 0: none
  int identity;             // identity experts: router outputs experts .. experts + identity - 1
  int hidden_cols;          // columns of `hidden` written: experts * ff + shared_ff, then zeros
  int width;
  const void* gu;           // [tokens][ld_gu]: per expert its gate rows (ff) then its up rows (ff); then the shared expert's
  int64_t ld_gu;
  const float* weights;     // [tokens][experts + identity]
  const float* gate;        // [tokens]: the shared expert's weight, or null
  void* hidden;             // [tokens][ld_hidden]
  int64_t ld_hidden;
  const void* h;            // [tokens][ldh]: the experts' input (read for identity experts only)
  int64_t ldh;
  float* identity_out;      // [tokens][width] float32: (sum of the identity experts' weights) * h; or null
  int act;                  // 0: silu(g) * u; 1: min(g, limit) * sigmoid(alpha * min(g, limit)) * (clamp(u, -limit, limit) + 1);
                            // 2, 3: units WITHOUT a gate, gelu(u) in its exact (erf) form and silu(u): `gu` then holds per
                            // expert its ff up rows only, the shared expert's behind them
  float limit;
  float alpha;
};

__device__ __forceinline__ float plain_unit(const GatedExpertsCall& c, float u) {
  return c.act == 2 ? 0.5f * u * (1.0f + erff(u * 0.70710678118654752f)) : u / (1.0f + expf(-u));
}

__device__ __forceinline__ float gated_unit(const GatedExpertsCall& c, float g, float u) {
  if (c.act == 1) {
    g = fminf(g, c.limit);
    u = fminf(fmaxf(u, -c.limit), c.limit);
    return g / (1.0f + expf(-c.alpha * g)) * (u + 1.0f);
  }
  return g / (1.0f + expf(-g)) * u;
}

template <typename T>
__global__ void __launch_bounds__(256) gated_experts_kernel(GatedExpertsCall c) {
  const int t = blockIdx.x;
  const T* gu = static_cast<const T*>(c.gu) + (int64_t)t * c.ld_gu;
  T* hidden = static_cast<T*>(c.hidden) + (int64_t)t * c.ld_hidden;
  const float* weights = c.weights + (int64_t)t * (c.experts + c.identity);
  const int routed = c.experts * c.ff;
  const bool gated = c.act < 2;
  // a token's columns are dealt to the work-groups of its row of the grid (a decode step has few tokens)
  for (int col = blockIdx.y * blockDim.x + threadIdx.x; col < c.hidden_cols; col += gridDim.y * blockDim.x) {
    float out = 0.f;
    if (col < routed) {
      const int e = col / c.ff, i = col - e * c.ff;
      const float w = weights[e];
      if (w != 0.f && gated) {
        const float g = to_float(gu[(int64_t)e * 2 * c.ff + i]), u = to_float(gu[(int64_t)e * 2 * c.ff + c.ff + i]);
        out = w * gated_unit(c, g, u);
      } else if (w != 0.f) {
        out = w * plain_unit(c, to_float(gu[col]));
      }
    } else if (col < routed + c.shared_ff) {
      const int i = col - routed;
      const float share = c.gate ? c.gate[t] : 1.0f;
      if (gated) {
        const float g = to_float(gu[(int64_t)2 * routed + i]), u = to_float(gu[(int64_t)2 * routed + c.shared_ff + i]);
        out = share * gated_unit(c, g, u);
      } else {
        out = share * plain_unit(c, to_float(gu[col]));
      }
    }
    hidden[col] = from_float<T>(out);
  }
  if (c.identity_out) {
    float w = 0.f;
    for (int i = 0; i < c.identity; ++i) w += weights[c.experts + i];
    const T* h = static_cast<const T*>(c.h) + (int64_t)t * c.ldh;
    for (int col = blockIdx.y * blockDim.x + threadIdx.x; col < c.width; col += gridDim.y * blockDim.x)
      c.identity_out[(int64_t)t * c.width + col] = w != 0.f ? w * to_float(h[col]) : 0.f;
  }
}

BT_EXPORT int bt_gated_experts_call(void* stream, const GatedExpertsCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->experts < 0 || c->ff <= 0 || c->shared_ff < 0 || c->identity < 0)
    BT_REFUSE("gated_experts: %d experts of %d, a shared one of %d and %d identity experts", c->experts, c->ff, c->shared_ff, c->identity);
  const int64_t columns = (int64_t)c->experts * c->ff + c->shared_ff;
  if (c->act < 0 || c->act > 3) BT_REFUSE("gated_experts: unknown activation %d", c->act);
  if (c->hidden_cols < columns || c->ld_hidden < c->hidden_cols || c->ld_gu < (c->act < 2 ? 2 : 1) * columns)
    BT_REFUSE("gated_experts: the rows do not hold the experts");
  if (!c->gu || (!c->weights && c->experts + c->identity > 0) || !c->hidden || (c->identity_out && (!c->h || c->width <= 0)))
    BT_REFUSE("gated_experts: missing operand");
  // about 1,024 columns a work-group, fewer work-groups a token where there are many tokens
  int per_token = (c->hidden_cols + 1023) / 1024;
  if (per_token > 64) per_token = 64;
  dim3 grid(c->tokens, per_token), block(256);
  if (c->dtype == 0)
    hipLaunchKernelGGL(gated_experts_kernel<float>, grid, block, 0, (hipStream_t)stream, *c);
  else
    hipLaunchKernelGGL(gated_experts_kernel<bf16_t>, grid, block, 0, (hipStream_t)stream, *c);
  return bt_check_launch("gated_experts");
}
