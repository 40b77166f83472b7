// Kernels of mixers that are linear attention with a matrix state per head (no softmax, no cache of
// keys): per head a state S [dim][vdim] in 32-bit that every token first lets decay per key channel
// and then writes a rank-one update into, token after token.
//   * keyed scan: per token and head, with a decay g [dim], a key k [dim], a value v [vdim], a query q [dim]:
//         S <- diag(g) S;   u = v                              (plain write)
//                           u = beta (v - S^T k)               (delta rule: what S already answers for k is taken off)
//         S <- S + k u^T;   o = S^T q                          (the read-out sees the token's own write)
//     How g, k and q come about is the kernel's `form`:
//       form 0 (gated delta rule): q and k are rows of their own (heads may share them), optionally made unit
//           vectors per head here, x / sqrt(sum x^2 + unit_eps), q times q_scale; g = exp(-exp(A_log[head]) * dt)
//           from step sizes dt per head and key channel, or one per head for all its key channels (`decay_span` 1);
//           with `dt_bias` the step sizes come raw and dt = softplus(raw + dt_bias); beta = sigmoid(beta logit of the head)
//       form 1 (forget gate that also decides what is written): f = lower + (1 - lower) * sigmoid(f_raw + f_bias)
//           per head and key channel; g = f, k = 1 - f, q = silu(q_raw); no beta
//   * head norm with a gate: every head's read-out over its root mean square over vdim, times a scale of
//     vdim entries that the heads share, times the sigmoid of a gate's logits where there are any
// A sequence's state lives in its slot's row of the cache's per-sequence state area; a step may bring any
// number of a sequence's tokens, which are walked in order from the state the last step left.
#include "host.h"
#include "scan.h"

struct KeyedScanCall {
  int tokens, n_seqs;
  int heads;              // heads of v, g, beta and of the state
  int kv_heads;           // heads of q and k (form 0); head h uses h / (heads / kv_heads)
  int dim, vdim;
  int form;               // 0: delta rule; 1: forget gate with complement keys
  int unit;               // form 0: 1 if q and k are made unit vectors per head here
  float unit_eps;
  float q_scale;          // form 0: factor on q (after the unit norm)
  const float* q;         // [tokens][ld_q]: form 0: head j at columns j * dim; form 1: raw, head h at h * dim
  int64_t ld_q;
  const float* k;         // [tokens][ld_k] (form 0)
  int64_t ld_k;
  const float* v;         // [tokens][ld_v]: head h at columns h * vdim
  int64_t ld_v;
  const float* g;         // [tokens][ld_g]: head h at columns h * dim: step sizes (form 0), gate logits (form 1);
  int64_t ld_g;           // with decay_span 1 head h at column h

  const float* beta;      // [tokens][ld_beta]: one logit a head (form 0)
  int64_t ld_beta;
  const float* A_log;     // [heads] (form 0)
  const float* g_bias;    // [heads * dim] (form 1), or null
  const float* lower;     // [heads * dim] (form 1)
  float* out;             // [tokens][ld_out] float32: head h at columns h * vdim
  int64_t ld_out;
  float* S;               // slot s: [heads][vdim / 4 rounded up][dim][4] at S + s * state_stride
  int64_t state_stride;
  const int* seq_off;     // [n_seqs + 1]
  const int* slots;       // [n_seqs]
  // form 1 only: long sequences are cut into spans of at least `span` tokens that are scanned side by side (see
  // "Spans" in scan.h; the forget gate's step is a diagonal decay and a write, which is linear in S; the delta
  // rule's is not diagonal and walks its sequences in order).  0: never; max_count is the most tokens a sequence
  // of the step brings, carry the room for the spans' states: (tokens / span + 2 n_seqs + 1) blocks of a slot's
  // state and heads * dim products of decays
  int span;
  int max_count;
  float* carry;
  int decay_span;         // form 0: 0 a step size per head and key channel, 1 one per head
  const float* dt_bias;   // form 0: null, or [heads * dim] ([heads] with decay_span 1): g holds raw sums, dt = softplus(g + dt_bias)
};

// One wave per (4 value channels of a head, sequence): sixteen lanes share a channel, each owns R key channels
// of its column of S in registers.  A work-group is four waves with four channels each of the same head: they
// share the run of decays, queries and keys in LDS.
// A run is up to 2048 / NP tokens (NP = 16 R key channels, padded), so that a thread stages KS_LOADS entries
// of it: every load of a run is issued before the first is used (a loop of single loads is waited for once
// per trip), and the NEXT run's loads are issued before this run's tokens are walked, so memory's latency
// hides behind the recurrence.
#define KS_WAVES 4
#define KS_THREADS (64 * KS_WAVES)
#define KS_LOADS 8

template <int R>
struct KsRun {
  static constexpr int NP = 16 * R;
  static constexpr int V = R < 4 ? R : 4;                          // floats a lane reads at a time
  static constexpr int MOST = 2048 / NP > 64 ? 64 : 2048 / NP;     // tokens of a run
  static constexpr int TOK_LOADS = (MOST * 4 + 63) / 64;           // (v, beta) pairs a lane stages
};

// Decays, queries and keys of a run lie in LDS as planes of [tokens][NP] floats (the forget gate's keys are
// 1 - decay and have no plane: every wave reads a token's whole row of every plane, and with several waves to a
// SIMD those reads are what bounds a token's time).  Lane j of the sixteen that share a value channel owns the
// key channels j + 16 r, r < R (so the lanes' loads of a register's worth of state are neighbours in memory); in
// a plane's row channel j + 16 r lies at (16 (r / V) + j) V + r % V, so that a lane reads V neighbouring floats
// at a time and neighbouring lanes read neighbouring vectors.
template <int R, int V>
__device__ __forceinline__ int ks_place(int sub, int r) { return (16 * (r / V) + sub) * V + r % V; }

template <int R, int V>
__device__ __forceinline__ void ks_read(const float* row, int sub, float* out) {
#pragma unroll
  for (int i = 0; i < R / V; ++i) {
    const float* at = row + (16 * i + sub) * V;
    if (V == 4) {
      const float4 x = *reinterpret_cast<const float4*>(at);
      out[4 * i] = x.x; out[4 * i + 1] = x.y; out[4 * i + 2] = x.z; out[4 * i + 3] = x.w;
    } else if (V == 2) {
      const float2 x = *reinterpret_cast<const float2*>(at);
      out[2 * i] = x.x; out[2 * i + 1] = x.y;
    } else {
      out[i] = at[0];
    }
  }
}

// phase 0: whole sequences, from and to the slot's state.  1: spans from zero, leaving their end states and the
// products of their decays, no read-outs.  3: spans from the carried states, writing read-outs, leaving no state.
template <int R, int FORM, int PHASE>
__global__ void __launch_bounds__(KS_THREADS) keyed_scan_kernel(KeyedScanCall c, int chunk, int tiles) {
  constexpr int phase = PHASE;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int NP = KsRun<R>::NP, V = KsRun<R>::V, TOK_LOADS = KsRun<R>::TOK_LOADS;
  constexpr int ROWS_A_TURN = KS_THREADS / NP;                                // tokens that the threads' entries of one turn span
  constexpr int PLANES = FORM == 0 ? 3 : 2;
  float* G = lds;                                                             // [chunk][NP] decays
  float* Q = lds + (size_t)chunk * NP;                                        // [chunk][NP] queries
  float* Kp = lds + (size_t)2 * chunk * NP;                                   // [chunk][NP] keys (delta rule)
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, sub = lane & 15, pl = lane >> 4;
  float2* tok = reinterpret_cast<float2*>(lds + (size_t)PLANES * chunk * NP) + (size_t)wave * chunk * 4;   // [waves][chunk][4]: v, beta
  // one decay a head: a run's decays are worked out once a token (thread i takes token i), not once a key channel
  float* dec = lds + (size_t)PLANES * chunk * NP + (size_t)KS_WAVES * chunk * 8;                          // [chunk]
  const bool per_head = FORM == 0 && c.decay_span == 1;
  const int tile = min((int)blockIdx.x * KS_WAVES + wave, tiles - 1), head = blockIdx.y;
  const int seq = blockIdx.z % c.n_seqs, part = blockIdx.z / c.n_seqs;
  const bool works = (int)blockIdx.x * KS_WAVES + wave < tiles;
  const int p = tile * 4 + pl;
  const bool live = works && p < c.vdim;
  const int shared = FORM == 0 ? head / (c.heads / c.kv_heads) : head;
  int first = c.seq_off[seq], last = c.seq_off[seq + 1];
  const int64_t in_slot = ((int64_t)head * tiles + tile) * c.dim * 4 + pl;        // where this lane's column of S starts
  float* held = c.S + (int64_t)c.slots[seq] * c.state_stride + in_slot;
  float* products = nullptr;                              // phase 1: where this span's products of decays go
  if (phase) {
    first += part * c.span;
    if (first >= last) return;                            // (the whole work-group: no barrier has been met)
    last = min(first + c.span, last);
    const int64_t state_floats = (int64_t)c.heads * tiles * c.dim * 4, per_span = state_floats + (int64_t)c.heads * c.dim;
    float* mine = c.carry + span_block(c.seq_off, seq, c.span, part) * per_span;
    held = (phase == 1 ? mine : mine - per_span) + in_slot;
    products = mine + state_floats + (int64_t)head * c.dim;
  }
  float S[R], P[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int n = sub + 16 * r;
    S[r] = n < c.dim && phase != 1 ? held[(int64_t)n * 4] : 0.f;
    P[r] = 1.0f;
  }
  const float rate = FORM == 0 ? -expf(c.A_log[head]) : 0.f;
  float* ocol = c.out + head * c.vdim + (live ? p : 0);
  // a thread's entries of a run are key channel `n` of the tokens row0, row0 + ROWS_A_TURN, ...
  const int n = threadIdx.x % NP, row0 = threadIdx.x / NP;
  const int place = ks_place<R, V>(n % 16, n / 16);       // where channel n lies in a plane's row
  const bool in_head = n < c.dim;
  const int nc = in_head ? n : 0;
  const int col_g = FORM == 0 && c.decay_span == 1 ? head : head * c.dim + nc, col_k = shared * c.dim + nc;
  float low = 0.f, bias = 0.f;
  if (FORM == 1) {
    low = c.lower[col_g];
    bias = c.g_bias ? c.g_bias[col_g] : 0.f;
  }
  const bool raw_steps = FORM == 0 && c.dt_bias != nullptr;
  if (raw_steps) bias = c.dt_bias[col_g];
  const int ch = tile * 4 + (lane & 3);                   // the value channel of a lane's (v, beta) pairs
  const int chc = ch < c.vdim ? ch : 0;
  float rg[KS_LOADS], rk[KS_LOADS], rq[KS_LOADS], rv[TOK_LOADS], rb[TOK_LOADS], rh = 0.f;
  // issues the loads of the run that starts at token t0 (rows beyond the run read its last token and are dropped)
  auto fetch = [&](int t0, int count) {
#pragma unroll
    for (int j = 0; j < KS_LOADS; ++j) {
      const int i = min(row0 + j * ROWS_A_TURN, count - 1);
      const int64_t t = t0 + i;
      rg[j] = per_head ? 0.f : c.g[t * c.ld_g + col_g];
      rq[j] = PHASE == 1 ? 0.f : c.q[t * c.ld_q + (FORM == 0 ? col_k : col_g)];
      rk[j] = FORM == 0 ? c.k[t * c.ld_k + col_k] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < TOK_LOADS; ++j) {
      const int i = min((lane >> 2) + 16 * j, count - 1);
      const int64_t t = t0 + i;
      rv[j] = c.v[t * c.ld_v + head * c.vdim + chc];
      rb[j] = FORM == 0 ? c.beta[t * c.ld_beta + head] : 0.f;
    }
    if (per_head) rh = c.g[(int64_t)(t0 + min((int)threadIdx.x, count - 1)) * c.ld_g + head];
  };
  if (first < last) fetch(first, min(chunk, last - first));
  for (int t0 = first; t0 < last; t0 += chunk) {
    const int count = min(chunk, last - t0);
    __syncthreads();                                       // the run before has been walked
    if (per_head) {
      if ((int)threadIdx.x < count) dec[threadIdx.x] = expf(rate * (raw_steps ? softplus_f(rh + bias) : rh));
      __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < KS_LOADS; ++j) {
      const int i = row0 + j * ROWS_A_TURN;
      if (i < count) {
        float decay = 0.f, query = 0.f;
        if (in_head) {
          if (FORM == 0) {
            decay = per_head ? dec[i] : expf(rate * (raw_steps ? softplus_f(rg[j] + bias) : rg[j]));
            query = rq[j];
          } else {
            decay = low + (1.0f - low) / (1.0f + expf(-(rg[j] + bias)));
            query = PHASE == 1 ? 0.f : silu_f(rq[j]);
          }
        }
        G[i * NP + place] = decay;
        if (PHASE != 1) Q[i * NP + place] = query;
        if (FORM == 0) Kp[i * NP + place] = in_head ? rk[j] : 0.f;
      }
    }
#pragma unroll
    for (int j = 0; j < TOK_LOADS; ++j) {
      const int i = (lane >> 2) + 16 * j;
      if (i < count)
        tok[i * 4 + (lane & 3)] = make_float2(ch < c.vdim ? rv[j] : 0.f, FORM == 0 ? 1.0f / (1.0f + expf(-rb[j])) : 1.0f);
    }
    __syncthreads();
    if (t0 + chunk < last) fetch(t0 + chunk, min(chunk, last - t0 - chunk));      // in flight while this run is walked
    if (FORM == 0 && c.unit) {          // q and k as unit vectors: sixteen lanes take a token
      for (int i = threadIdx.x >> 4; i < count; i += 4 * KS_WAVES) {
        float kk[R], qq[R], sk = 0.f, sq = 0.f;
        ks_read<R, V>(Kp + i * NP, sub, kk);
        ks_read<R, V>(Q + i * NP, sub, qq);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          sk = fmaf(kk[r], kk[r], sk);
          sq = fmaf(qq[r], qq[r], sq);
        }
        const float rk_ = 1.0f / sqrtf(sum_of_16_lanes(sk) + c.unit_eps);
        const float rq_ = c.q_scale / sqrtf(sum_of_16_lanes(sq) + c.unit_eps);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          Kp[i * NP + ks_place<R, V>(sub, r)] = kk[r] * rk_;
          Q[i * NP + ks_place<R, V>(sub, r)] = qq[r] * rq_;
        }
      }
      __syncthreads();
    }
    if (!works) continue;
    // a token's inputs are read from LDS while the token before it is worked on: a wave is alone on its SIMD,
    // so nothing else hides that latency
    float g[R], k[R], q[R];
    float2 vb = tok[pl];
    ks_read<R, V>(G, sub, g);
    if (PHASE != 1) ks_read<R, V>(Q, sub, q);
    if (FORM == 0) ks_read<R, V>(Kp, sub, k);
#pragma unroll 4
    for (int i = 0; i < count; ++i) {
      const int ahead = min(i + 1, count - 1);
      float g_next[R], k_next[R], q_next[R];
      const float2 vb_next = tok[ahead * 4 + pl];
      ks_read<R, V>(G + ahead * NP, sub, g_next);
      if (PHASE != 1) ks_read<R, V>(Q + ahead * NP, sub, q_next);
      if (FORM == 0) ks_read<R, V>(Kp + ahead * NP, sub, k_next);
      float u = vb.x;
      if (FORM == 0) {
        float answered = 0.f, answered_odd = 0.f;          // (two sums: half as long a chain of dependent adds)
#pragma unroll
        for (int r = 0; r < R; ++r) {
          S[r] *= g[r];
          if (r & 1) answered_odd = fmaf(S[r], k[r], answered_odd);
          else answered = fmaf(S[r], k[r], answered);
        }
        u = vb.y * (vb.x - sum_of_16_lanes(answered + answered_odd));
      } else {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          k[r] = 1.0f - g[r];
          S[r] *= g[r];
          if (PHASE == 1) P[r] *= g[r];
        }
      }
      if (PHASE == 1) {                                     // a span from zero leaves its state only: no read-out
#pragma unroll
        for (int r = 0; r < R; ++r) S[r] = fmaf(k[r], u, S[r]);
      } else {
        float acc = 0.f, acc_odd = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          S[r] = fmaf(k[r], u, S[r]);
          if (r & 1) acc_odd = fmaf(S[r], q[r], acc_odd);
          else acc = fmaf(S[r], q[r], acc);
        }
        const float o = sum_of_16_lanes(acc + acc_odd);
        if (live && sub == 0) ocol[(int64_t)(t0 + i) * c.ld_out] = o;
      }
      vb = vb_next;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        g[r] = g_next[r];
        if (PHASE != 1) q[r] = q_next[r];
        if (FORM == 0) k[r] = k_next[r];
      }
    }
  }
  if (!works || phase == 3) return;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int nn = sub + 16 * r;
    if (nn < c.dim) held[(int64_t)nn * 4] = S[r];
    if (nn < c.dim && phase == 1 && blockIdx.x == 0 && wave == 0 && pl == 0) products[nn] = P[r];
  }
}

// C_k = P_k C_(k-1) + E_k along every sequence, in place; C_(-1), the state the sequence came with, is kept in
// front of its spans, and the last C goes into the slot.
__global__ void __launch_bounds__(256) keyed_carry_kernel(KeyedScanCall c, int tiles) {
  const int seq = blockIdx.y;
  const int64_t index = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, size = (int64_t)c.heads * tiles * c.dim * 4;
  if (index >= size) return;
  const int count = c.seq_off[seq + 1] - c.seq_off[seq];
  const int spans = (count + c.span - 1) / c.span;
  const int64_t per_span = size + (int64_t)c.heads * c.dim;
  float* block = c.carry + span_block(c.seq_off, seq, c.span, 0) * per_span;
  float* slot = c.S + (int64_t)c.slots[seq] * c.state_stride;
  float state = slot[index];
  (block - per_span)[index] = state;
  const int64_t decay = size + (index / ((int64_t)4 * c.dim * tiles)) * c.dim + (index / 4) % c.dim;
  for (int k = 0; k < spans; ++k, block += per_span) {
    state = block[decay] * state + block[index];
    block[index] = state;
  }
  slot[index] = state;
}

template <int R>
static void launch_keyed_scan(hipStream_t stream, const KeyedScanCall& c) {
  const int per_token = (c.form == 0 ? 3 : 2) * 16 * R + 8 * KS_WAVES + 1;      // planes, (v, beta) pairs, a decay
  const int tiles = (c.vdim + 3) / 4, groups = (tiles + KS_WAVES - 1) / KS_WAVES;
  dim3 block(KS_THREADS);
  const int span = c.form == 1 ? span_tokens(c.span, c.max_count, c.carry, (int64_t)groups * KS_WAVES * c.heads * c.n_seqs, 1) : 0;
  if (span > 0 && (int64_t)c.n_seqs * ((c.max_count + span - 1) / span) <= 65535) {
    KeyedScanCall cut = c;
    cut.span = span;
    const int chunk = span < KsRun<R>::MOST ? span : KsRun<R>::MOST;
    const int spans = (c.max_count + span - 1) / span;
    dim3 grid(groups, c.heads, c.n_seqs * spans);
    const size_t lds = (size_t)chunk * per_token * sizeof(float);
    const int64_t state_floats = (int64_t)c.heads * tiles * c.dim * 4;
    hipLaunchKernelGGL((keyed_scan_kernel<R, 1, 1>), grid, block, lds, stream, cut, chunk, tiles);
    hipLaunchKernelGGL(keyed_carry_kernel, dim3((unsigned)((state_floats + 255) / 256), c.n_seqs), dim3(256), 0, stream, cut, tiles);
    hipLaunchKernelGGL((keyed_scan_kernel<R, 1, 3>), grid, block, lds, stream, cut, chunk, tiles);
    return;
  }
  const int chunk = c.tokens < KsRun<R>::MOST ? c.tokens : KsRun<R>::MOST;
  dim3 grid(groups, c.heads, c.n_seqs);
  const size_t lds = (size_t)chunk * per_token * sizeof(float);
  if (c.form == 0)
    hipLaunchKernelGGL((keyed_scan_kernel<R, 0, 0>), grid, block, lds, stream, c, chunk, tiles);
  else
    hipLaunchKernelGGL((keyed_scan_kernel<R, 1, 0>), grid, block, lds, stream, c, chunk, tiles);
}

BT_EXPORT int bt_keyed_scan_call(void* stream, const KeyedScanCall* c) {
  if (c->tokens <= 0 || c->n_seqs <= 0) return BT_OK;
  if (c->heads <= 0 || c->dim <= 0 || c->dim > 256 || c->vdim <= 0)
    BT_REFUSE("keyed_scan: %d heads with keys of %d (1..256) and values of %d", c->heads, c->dim, c->vdim);
  if (c->form != 0 && c->form != 1) BT_REFUSE("keyed_scan: unknown form %d", c->form);
  if (c->form == 0 && (c->kv_heads <= 0 || c->heads % c->kv_heads != 0))
    BT_REFUSE("keyed_scan: %d heads cannot share %d heads of queries and keys", c->heads, c->kv_heads);
  if (!c->q || !c->v || !c->g || !c->out || !c->S || !c->seq_off || !c->slots)
    BT_REFUSE("keyed_scan: missing operand");
  if (c->form == 0 && (!c->k || !c->beta || !c->A_log)) BT_REFUSE("keyed_scan: the delta rule lacks keys, beta or A_log");
  if (c->form == 1 && !c->lower) BT_REFUSE("keyed_scan: the forget gate lacks its lower bound");
  const int64_t qk = (int64_t)(c->form == 0 ? c->kv_heads : c->heads) * c->dim;
  if (c->decay_span != 0 && (c->decay_span != 1 || c->form != 0)) BT_REFUSE("keyed_scan: a decay per head goes with the delta rule");
  if (c->ld_q < qk || (c->form == 0 && c->ld_k < qk) || c->ld_g < (int64_t)c->heads * (c->decay_span == 1 ? 1 : c->dim) ||
      c->ld_v < (int64_t)c->heads * c->vdim || c->ld_out < (int64_t)c->heads * c->vdim ||
      (c->form == 0 && c->ld_beta < c->heads))
    BT_REFUSE("keyed_scan: rows too short for %d heads of %d and %d", c->heads, c->dim, c->vdim);
  if (c->state_stride < (int64_t)c->heads * ((c->vdim + 3) / 4) * c->dim * 4)
    BT_REFUSE("keyed_scan: a slot's state of %lld elements does not hold %d heads of %d x %d", (long long)c->state_stride,
              c->heads, c->dim, c->vdim);
  if (c->heads > 65535 || c->n_seqs > 65535) BT_REFUSE("keyed_scan: %d heads of %d sequences are too many", c->heads, c->n_seqs);
  hipStream_t s = (hipStream_t)stream;
  const int per = (c->dim + 15) / 16;
  if (per <= 1) launch_keyed_scan<1>(s, *c);
  else if (per <= 2) launch_keyed_scan<2>(s, *c);
  else if (per <= 4) launch_keyed_scan<4>(s, *c);
  else if (per <= 8) launch_keyed_scan<8>(s, *c);
  else launch_keyed_scan<16>(s, *c);
  return bt_check_launch("keyed_scan");
}

// out[t][h * vdim + i] = y / sqrt(mean_i(y^2) + eps) * weight[i] * sigmoid(gate[t][h * vdim + i]), y = the
// head's read-out; without `gate` no last factor.  Columns of `out` behind the heads are set to zero.
struct HeadNormGateCall {
  int out_dtype;          // 0 float32, 1 bfloat16
  int tokens, heads, vdim;
  int out_cols;           // columns of out written: heads * vdim, then zeros
  float eps;
  float mult;             // one more factor on the result
  const float* y;         // [tokens][ld_y]
  int64_t ld_y;
  const float* gate;      // [tokens][ld_gate] logits, or null
  int64_t ld_gate;
  const float* weight;    // [vdim]
  void* out;              // [tokens][ld_out]
  int64_t ld_out;
  int gate_act;           // what the gate's logits z become: 0 sigmoid(z), 1 silu(z) = z sigmoid(z)
};

template <typename T>
__global__ void __launch_bounds__(256) head_norm_gate_kernel(HeadNormGateCall c) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  T* out = static_cast<T*>(c.out) + (int64_t)t * c.ld_out;
  for (int head = blockIdx.y * 4 + wave; head < c.heads; head += gridDim.y * 4) {
    const float* y = c.y + (int64_t)t * c.ld_y + head * c.vdim;
    float squares = 0.f;
    for (int i = lane; i < c.vdim; i += 64) squares = fmaf(y[i], y[i], squares);
    const float scale = c.mult / sqrtf(wave_sum(squares) / (float)c.vdim + c.eps);
    for (int i = lane; i < c.vdim; i += 64) {
      float v = y[i] * scale * c.weight[i];
      if (c.gate) {
        const float z = c.gate[(int64_t)t * c.ld_gate + head * c.vdim + i];
        v *= (c.gate_act == 1 ? z : 1.0f) / (1.0f + expf(-z));
      }
      out[head * c.vdim + i] = from_float<T>(v);
    }
  }
  if (blockIdx.y == 0)
    for (int col = c.heads * c.vdim + threadIdx.x; col < c.out_cols; col += blockDim.x) out[col] = from_float<T>(0.f);
}

BT_EXPORT int bt_head_norm_gate_call(void* stream, const HeadNormGateCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->heads <= 0 || c->vdim <= 0) BT_REFUSE("head_norm_gate: %d heads of %d", c->heads, c->vdim);
  const int64_t columns = (int64_t)c->heads * c->vdim;
  if (!c->y || !c->weight || !c->out || c->ld_y < columns || c->out_cols < columns || c->ld_out < c->out_cols ||
      (c->gate && c->ld_gate < columns))
    BT_REFUSE("head_norm_gate: missing operand or rows too short");
  if (c->gate_act != 0 && c->gate_act != 1) BT_REFUSE("head_norm_gate: unknown activation %d of the gate", c->gate_act);
  int per_token = (c->heads + 3) / 4;
  if (per_token > 64) per_token = 64;
  dim3 grid(c->tokens, per_token), block(256);
  if (c->out_dtype == 0)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, grid, block, 0, (hipStream_t)stream, *c);
  else
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, grid, block, 0, (hipStream_t)stream, *c);
  return bt_check_launch("head_norm_gate");
}
