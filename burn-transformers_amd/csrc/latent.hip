// Kernels of the latent attention mixer (queries and keys/values through normalised low-rank
// latents; only the key/value latent is cached, and attention runs on it directly).
//   * latent norms: the two RMS norms behind the fused down-projection; the query latent goes to a
//     buffer for the next product, the key/value latent straight into the paged cache, where it is
//     the one shared "head" whose keys and values are the same vector.  With `rot_dim` > 0 the down-projection
//     has that many more rows behind the key/value latent: one key part that all heads share, not normalised,
//     turned by the token's position (channel 2 i with channel 2 i + 1, or i with i + rot_dim / 2), kept behind
//     the latent in the cached head's KEYS (its values have zeros there)
//   * query rotation: the absorbed queries (32-bit sums, a head's latent part and behind it its turned part)
//     into the attention kernels' type, the turned part rotated by the token's position
//   * head projection with gate: per head out = sigmoid(g) * (W_h . ctx_h), the value up-projection
//     applied AFTER the weighted sum over positions (it is linear, so it commutes with the sum)
// Statistics and sums are 32-bit.
#include "host.h"

struct LatentNormCall {
  int dtype;              // element type of `q_out` and of the cache: 0 float32, 1 bfloat16
  int tokens;
  int q_rank, q_cols;     // the query latent's length; columns of q_out written (latent, then zeros)
  int kv_rank;            // the key/value latent's length (the cache's head size may be larger: zeros)
  int kv_offset;          // its first column in `in`
  float eps;
  const float* in;        // [tokens][ld] float32: the fused down-projection
  int64_t ld;
  const float* q_gamma;   // [q_rank]
  const float* kv_gamma;  // [kv_rank]
  void* q_out;            // [tokens][ld_q]
  int64_t ld_q;
  const int* tok_seq;
  const int* tok_pos;
  KvView kv;              // one head of head_dim >= kv_rank + rot_dim
  int rot_dim;            // channels of the shared turned key part (even; 0: none), at in[kv_offset + kv_rank ..]
  int pairing;            // 0: channel i turns with channel i + rot_dim / 2; 1: channel 2 i with channel 2 i + 1
  float amplitude;        // factor on every sine and cosine
  const float* inv_freq;  // [rot_dim / 2]
};

template <typename T>
__global__ void __launch_bounds__(256) latent_norm_kernel(LatentNormCall c) {
  __shared__ float scratch[32];
  const int t = blockIdx.x;
  const bool query = blockIdx.y == 0;
  const int n = query ? c.q_rank : c.kv_rank;
  const float* row = c.in + (int64_t)t * c.ld + (query ? 0 : c.kv_offset);
  const float* gamma = query ? c.q_gamma : c.kv_gamma;
  float partial = 0.f;
  for (int col = threadIdx.x; col < n; col += blockDim.x) partial += row[col] * row[col];
  const float rstd = 1.0f / sqrtf(block_sum(partial, scratch) / (float)n + c.eps);
  if (query) {
    T* out = static_cast<T*>(c.q_out) + (int64_t)t * c.ld_q;
    for (int col = threadIdx.x; col < c.q_cols; col += blockDim.x)
      out[col] = from_float<T>(col < n ? row[col] * rstd * gamma[col] : 0.f);
  } else {
    const int seq = c.tok_seq[t], pos = c.tok_pos[t], hd = c.kv.head_dim;
    const int64_t base = kv_block_base(c.kv, seq, pos, 0);
    T* keys = static_cast<T*>(c.kv.keys) + base;
    T* values = static_cast<T*>(c.kv.values) + base;
    const int half = c.rot_dim >> 1;
    for (int col = threadIdx.x; col < hd; col += blockDim.x) {
      const T v = from_float<T>(col < n ? row[col] * rstd * gamma[col] : 0.f);
      if (col < n || col >= n + c.rot_dim) keys[key_offset(hd, pos, col)] = v;
      values[value_offset(hd, pos, col)] = v;
    }
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
      float sn, cs;
      sincosf((float)pos * c.inv_freq[i], &sn, &cs);
      sn *= c.amplitude;
      cs *= c.amplitude;
      const int first = c.pairing == 1 ? 2 * i : i, second = c.pairing == 1 ? 2 * i + 1 : i + half;
      const float u = row[n + first], w = row[n + second];
      keys[key_offset(hd, pos, n + first)] = from_float<T>(u * cs - w * sn);
      keys[key_offset(hd, pos, n + second)] = from_float<T>(w * cs + u * sn);
    }
  }
}

BT_EXPORT int bt_latent_norm_call(void* stream, const LatentNormCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->q_rank <= 0 || c->kv_rank <= 0) BT_REFUSE("latent_norm: ranks %d and %d must be positive", c->q_rank, c->kv_rank);
  if (c->rot_dim < 0 || c->rot_dim % 2 != 0 || (c->pairing != 0 && c->pairing != 1) || (c->rot_dim > 0 && !c->inv_freq))
    BT_REFUSE("latent_norm: a turned key part of %d channels (even, with frequencies), pairing %d (0 or 1)", c->rot_dim, c->pairing);
  if (c->kv.kv_heads != 1 || c->kv.head_dim < c->kv_rank + c->rot_dim)
    BT_REFUSE("latent_norm: the cache keeps %d heads of %d, expected one of at least %d", c->kv.kv_heads,
              c->kv.head_dim, c->kv_rank + c->rot_dim);
  if (c->q_cols < c->q_rank || c->ld_q < c->q_cols || c->ld < c->kv_offset + c->kv_rank + c->rot_dim || c->kv_offset < c->q_rank)
    BT_REFUSE("latent_norm: the rows do not hold the latents");
  if (!c->in || !c->q_gamma || !c->kv_gamma || !c->q_out || !c->tok_seq || !c->tok_pos || !c->kv.blocks ||
      !c->kv.keys || !c->kv.values)
    BT_REFUSE("latent_norm: missing operand");
  dim3 grid(c->tokens, 2), block(256);
  if (c->dtype == 0)
    hipLaunchKernelGGL(latent_norm_kernel<float>, grid, block, 0, (hipStream_t)stream, *c);
  else
    hipLaunchKernelGGL(latent_norm_kernel<bf16_t>, grid, block, 0, (hipStream_t)stream, *c);
  return bt_check_launch("latent_norm");
}

// q[t][h * pitch + j] = in[t][h * pitch + j], the channels [rot_at, rot_at + rot_dim) of every head turned by the
// token's position: pairs (2 i, 2 i + 1) or (i, i + rot_dim / 2) of that range, by the angle position * inv_freq[i].
struct LatentQueryCall {
  int dtype;              // element type of `out`: 0 float32, 1 bfloat16
  int tokens, heads;
  int pitch;              // channels of a head in `in` and `out`
  int rot_at, rot_dim;    // the turned range inside a head
  int pairing;
  float amplitude;
  const float* in;        // [tokens][ld_in] float32
  int64_t ld_in;
  void* out;              // [tokens][ld_out]
  int64_t ld_out;
  const float* inv_freq;  // [rot_dim / 2]
  const int* tok_pos;
};

template <typename T>
__global__ void __launch_bounds__(256) latent_query_kernel(LatentQueryCall c) {
  const int t = blockIdx.x, pos = c.tok_pos[t], half = c.rot_dim >> 1;
  const float* in = c.in + (int64_t)t * c.ld_in;
  T* out = static_cast<T*>(c.out) + (int64_t)t * c.ld_out;
  const int columns = c.heads * c.pitch;
  for (int col = blockIdx.y * blockDim.x + threadIdx.x; col < columns; col += gridDim.y * blockDim.x) {
    const int head = col / c.pitch, j = col - head * c.pitch - c.rot_at;
    float v = in[col];
    if (j >= 0 && j < c.rot_dim) {
      // channel j of the turned range: the first of its pair takes u cos - v sin, the second v cos + u sin
      const int i = c.pairing == 1 ? j >> 1 : (j < half ? j : j - half);
      const bool second = c.pairing == 1 ? (j & 1) : j >= half;
      const int mate = c.pairing == 1 ? (j ^ 1) : (second ? j - half : j + half);
      const float other = in[col - j + mate];
      float sn, cs;
      sincosf((float)pos * c.inv_freq[i], &sn, &cs);
      v = c.amplitude * (second ? v * cs + other * sn : v * cs - other * sn);
    }
    out[col] = from_float<T>(v);
  }
}

BT_EXPORT int bt_latent_query_call(void* stream, const LatentQueryCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->heads <= 0 || c->pitch <= 0 || c->rot_at < 0 || c->rot_dim < 0 || c->rot_dim % 2 != 0 || c->rot_at + c->rot_dim > c->pitch)
    BT_REFUSE("latent_query: %d heads of %d with a turned range of %d from %d", c->heads, c->pitch, c->rot_dim, c->rot_at);
  if (c->pairing != 0 && c->pairing != 1) BT_REFUSE("latent_query: pairing %d must be 0 or 1", c->pairing);
  const int64_t columns = (int64_t)c->heads * c->pitch;
  if (!c->in || !c->out || !c->tok_pos || (c->rot_dim > 0 && !c->inv_freq) || c->ld_in < columns || c->ld_out < columns)
    BT_REFUSE("latent_query: missing operand or rows too short");
  int per_token = (int)((columns + 1023) / 1024);
  if (per_token > 64) per_token = 64;
  dim3 grid(c->tokens, per_token), block(256);
  if (c->dtype == 0)
    hipLaunchKernelGGL(latent_query_kernel<float>, grid, block, 0, (hipStream_t)stream, *c);
  else
    hipLaunchKernelGGL(latent_query_kernel<bf16_t>, grid, block, 0, (hipStream_t)stream, *c);
  return bt_check_launch("latent_query");
}

// out[t][h * vdim + v] = sigmoid(gate[t][h * vdim + v]) * sum_r W[h * vdim + v][r] * ctx[t][h * ld_head + r]
// One work-group per (tile of HP_TOKENS tokens, head, run of up to HP_VCHUNK outputs); the rank is
// walked in steps of HP_RSTEP through LDS (the weights transposed, so that threads with consecutive
// outputs read consecutive words).
#define HP_TOKENS 16
#define HP_VCHUNK 128
#define HP_RSTEP 32
#define HP_PER_THREAD (HP_TOKENS * HP_VCHUNK / 256)

struct HeadProjectCall {
  int dtype;              // element type of ctx, W and out
  int tokens;
  int heads, vdim, rank;
  int head_pitch;         // elements between two heads' vectors in a row of ctx
  int out_cols;           // columns of out written: heads * vdim, then zeros
  const void* ctx;        // [tokens][ld_ctx]
  int64_t ld_ctx;
  const void* W;          // [heads * vdim][rank]
  const float* gate;      // [tokens][ld_gate] pre-activation, or null
  int64_t ld_gate;
  void* out;              // [tokens][ld_out]
  int64_t ld_out;
};

template <typename T>
__global__ void __launch_bounds__(256) head_project_kernel(HeadProjectCall c) {
  __shared__ float ws[HP_RSTEP][HP_VCHUNK + 1];
  __shared__ float cs[HP_TOKENS][HP_RSTEP + 1];
  const int t0 = blockIdx.x * HP_TOKENS, head = blockIdx.y, v0 = blockIdx.z * HP_VCHUNK;
  const int vc = min(HP_VCHUNK, c.vdim - v0);
  const T* ctx = static_cast<const T*>(c.ctx);
  const T* W = static_cast<const T*>(c.W) + ((int64_t)head * c.vdim + v0) * c.rank;
  float acc[HP_PER_THREAD];
#pragma unroll
  for (int k = 0; k < HP_PER_THREAD; ++k) acc[k] = 0.f;
  for (int r0 = 0; r0 < c.rank; r0 += HP_RSTEP) {
    for (int e = threadIdx.x; e < HP_VCHUNK * HP_RSTEP; e += 256) {
      const int v = e / HP_RSTEP, rr = e % HP_RSTEP;
      ws[rr][v] = (v < vc && r0 + rr < c.rank) ? to_float(W[(int64_t)v * c.rank + r0 + rr]) : 0.f;
    }
    for (int e = threadIdx.x; e < HP_TOKENS * HP_RSTEP; e += 256) {
      const int i = e / HP_RSTEP, rr = e % HP_RSTEP;
      cs[i][rr] = (t0 + i < c.tokens && r0 + rr < c.rank)
                      ? to_float(ctx[(int64_t)(t0 + i) * c.ld_ctx + (int64_t)head * c.head_pitch + r0 + rr]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < HP_PER_THREAD; ++k) {
      const int e = threadIdx.x + 256 * k;
      const int i = e / HP_VCHUNK, v = e % HP_VCHUNK;
      float sum = acc[k];
#pragma unroll
      for (int rr = 0; rr < HP_RSTEP; ++rr) sum = fmaf(cs[i][rr], ws[rr][v], sum);
      acc[k] = sum;
    }
    __syncthreads();
  }
  T* out = static_cast<T*>(c.out);
#pragma unroll
  for (int k = 0; k < HP_PER_THREAD; ++k) {
    const int e = threadIdx.x + 256 * k;
    const int i = e / HP_VCHUNK, v = e % HP_VCHUNK;
    if (t0 + i >= c.tokens || v >= vc) continue;
    const int col = head * c.vdim + v0 + v;
    float y = acc[k];
    if (c.gate) y *= 1.0f / (1.0f + expf(-c.gate[(int64_t)(t0 + i) * c.ld_gate + col]));
    out[(int64_t)(t0 + i) * c.ld_out + col] = from_float<T>(y);
  }
  // the columns behind the last head's, which the next product reads as zeros
  if (head == c.heads - 1 && blockIdx.z == gridDim.z - 1)
    for (int e = threadIdx.x; e < HP_TOKENS * (c.out_cols - c.heads * c.vdim); e += 256) {
      const int extra = c.out_cols - c.heads * c.vdim;
      const int i = e / extra, col = c.heads * c.vdim + e % extra;
      if (t0 + i < c.tokens) out[(int64_t)(t0 + i) * c.ld_out + col] = from_float<T>(0.f);
    }
}

// The same for steps of few tokens (decode): one work-group per (token, head, run of 64 outputs), four
// lanes share an output and split the rank, everything read straight from memory with all loads of
// a lane independent of each other.
#define HP_SMALL_TOKENS 32

template <typename T>
__global__ void __launch_bounds__(256) head_project_small_kernel(HeadProjectCall c) {
  const int t = blockIdx.x, head = blockIdx.y;
  const int v = blockIdx.z * 64 + (threadIdx.x >> 2), part = threadIdx.x & 3;
  const bool live = v < c.vdim;
  const int col = head * c.vdim + (live ? v : c.vdim - 1);
  const T* w = static_cast<const T*>(c.W) + (int64_t)col * c.rank;
  const T* ctx = static_cast<const T*>(c.ctx) + (int64_t)t * c.ld_ctx + (int64_t)head * c.head_pitch;
  float acc = 0.f;
  for (int r = part; r < c.rank; r += 4) acc = fmaf(to_float(w[r]), to_float(ctx[r]), acc);
  acc += __shfl_xor(acc, 2, 64);
  acc += __shfl_xor(acc, 1, 64);
  T* out = static_cast<T*>(c.out) + (int64_t)t * c.ld_out;
  if (live && part == 0) {
    if (c.gate) acc *= 1.0f / (1.0f + expf(-c.gate[(int64_t)t * c.ld_gate + col]));
    out[col] = from_float<T>(acc);
  }
  if (head == c.heads - 1 && blockIdx.z == gridDim.z - 1)
    for (int extra = c.heads * c.vdim + threadIdx.x; extra < c.out_cols; extra += 256) out[extra] = from_float<T>(0.f);
}

BT_EXPORT int bt_head_project_call(void* stream, const HeadProjectCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->heads <= 0 || c->vdim <= 0 || c->rank <= 0)
    BT_REFUSE("head_project: %d heads of %d from rank %d: all must be positive", c->heads, c->vdim, c->rank);
  if (c->head_pitch < c->rank || c->ld_ctx < (int64_t)c->heads * c->head_pitch ||
      c->out_cols < c->heads * c->vdim || c->ld_out < c->out_cols ||
      (c->gate && c->ld_gate < (int64_t)c->heads * c->vdim))
    BT_REFUSE("head_project: the rows do not hold %d heads", c->heads);
  if (!c->ctx || !c->W || !c->out) BT_REFUSE("head_project: missing operand");
  if (c->tokens <= HP_SMALL_TOKENS) {
    dim3 small(c->tokens, c->heads, (c->vdim + 63) / 64);
    if (c->dtype == 0)
      hipLaunchKernelGGL(head_project_small_kernel<float>, small, dim3(256), 0, (hipStream_t)stream, *c);
    else
      hipLaunchKernelGGL(head_project_small_kernel<bf16_t>, small, dim3(256), 0, (hipStream_t)stream, *c);
    return bt_check_launch("head_project");
  }
  dim3 grid((c->tokens + HP_TOKENS - 1) / HP_TOKENS, c->heads, (c->vdim + HP_VCHUNK - 1) / HP_VCHUNK), block(256);
  if (c->dtype == 0)
    hipLaunchKernelGGL(head_project_kernel<float>, grid, block, 0, (hipStream_t)stream, *c);
  else
    hipLaunchKernelGGL(head_project_kernel<bf16_t>, grid, block, 0, (hipStream_t)stream, *c);
  return bt_check_launch("head_project");
}
