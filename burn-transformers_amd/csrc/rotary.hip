// Kernels of attention mixers that turn queries and keys by their positions (rotary positions).
//   * head norms and rotation into the cache: behind a fused query/key/value projection that leaves
//     32-bit sums, every query and key head is divided by its root mean square (times a scale
//     shared by the heads), the first `rot_dims` channels of each head are turned by the token's
//     position, queries go to a buffer for the attention kernel and keys and values straight into
//     the paged cache at the token's position.  Queries/keys and values may have different head
//     sizes; the cache keeps heads of one size, and what lies behind a head's own channels is zero.
// Channel i < rot_dims / 2 is paired with channel i + rot_dims / 2 (`pairing` 0, the halves) or channel
// 2 i with channel 2 i + 1 (`pairing` 1, neighbours); the pair (u, v) at position p
// becomes (u cos a - v sin a, v cos a + u sin a), a = p * inv_freq[i], sine and cosine times `amplitude`
// (one where the frequencies are not rescaled; schedules that slow long waves let both grow a little).  With `norm_span` 1 the root mean
// square is taken over a token's WHOLE query (or key) projection, all heads at once, and the scale has
// an entry for every channel of the projection.  The frequencies come as a
// table, so any schedule of them (scaled, interpolated) is the caller's.  Norms, angles and the
// rotation are 32-bit.
#include "host.h"

struct HeadRotaryCall {
  int dtype;              // element type of `q_out` and of the cache: 0 float32, 1 bfloat16
  int tokens;
  int heads, kv_heads;
  int dim, vdim;          // a head's channels of queries and keys, and of values, in `in`
  int rot_dims;           // channels of each query and key head that are turned: even, at most dim; 0: none
  float eps;
  const float* in;        // [tokens][ld] float32: queries (heads * dim), keys (kv_heads * dim), values (kv_heads * vdim)
  int64_t ld;
  const float* q_gamma;   // [dim] ([heads * dim] with norm_span 1) or null: no norm of the queries
  const float* k_gamma;   // [dim] ([kv_heads * dim] with norm_span 1) or null
  const float* inv_freq;  // [rot_dims / 2]
  void* q_out;            // [tokens][ld_q]: head j at columns j * kv.head_dim
  int64_t ld_q;
  const int* tok_seq;
  const int* tok_pos;
  KvView kv;              // kv_heads heads of head_dim >= max(dim, vdim)
  int pairing;            // 0: channel i turns with channel i + rot_dims / 2; 1: channel 2 i with channel 2 i + 1
  int norm_span;          // 0: every head over its own root mean square; 1: the whole projection over one
  float amplitude;        // factor on every sine and cosine
};

#define HR_WAVES 4
#define HR_MAX_DIM 256

template <typename T>
__global__ void __launch_bounds__(HR_WAVES * 64) head_rotary_kernel(HeadRotaryCall c) {
  __shared__ float rows[HR_WAVES][HR_MAX_DIM];
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int unit = blockIdx.y * HR_WAVES + wave;           // a query head, then a key head, then a value head
  const int units = c.heads + 2 * c.kv_heads;
  const bool active = unit < units;
  const bool is_q = unit < c.heads, is_k = !is_q && unit < c.heads + c.kv_heads;
  const int head = is_q ? unit : (is_k ? unit - c.heads : unit - c.heads - c.kv_heads);
  const int n = (is_q || is_k) ? c.dim : c.vdim;
  const int hd = c.kv.head_dim;
  float* row = rows[wave];
  if (active) {
    const int64_t first = is_q ? (int64_t)head * c.dim
                               : (is_k ? (int64_t)c.heads * c.dim + (int64_t)head * c.dim
                                       : (int64_t)(c.heads + c.kv_heads) * c.dim + (int64_t)head * c.vdim);
    const float* src = c.in + (int64_t)t * c.ld + first;
    const float* gamma = is_q ? c.q_gamma : (is_k ? c.k_gamma : nullptr);
    float squares = 0.f;
    for (int col = lane; col < n; col += 64) {
      const float v = src[col];
      row[col] = v;
      squares += v * v;
    }
    if (gamma && c.norm_span == 1) {
      // every wave of a projection adds up the same squares in the same order: the heads agree exactly
      const int all = (is_q ? c.heads : c.kv_heads) * c.dim;
      const float* whole = c.in + (int64_t)t * c.ld + (is_q ? 0 : (int64_t)c.heads * c.dim);
      squares = 0.f;
      for (int col = lane; col < all; col += 64) squares = fmaf(whole[col], whole[col], squares);
      const float rstd = 1.0f / sqrtf(wave_sum(squares) / (float)all + c.eps);
      for (int col = lane; col < n; col += 64) row[col] = row[col] * rstd * gamma[head * c.dim + col];
    } else if (gamma) {
      const float rstd = 1.0f / sqrtf(wave_sum(squares) / (float)n + c.eps);
      for (int col = lane; col < n; col += 64) row[col] = row[col] * rstd * gamma[col];
    }
  }
  __syncthreads();
  if (!active) return;
  const int pos = c.tok_pos[t];
  const int half = c.rot_dims >> 1;
  const bool turned = (is_q || is_k) && half > 0;
  T* q_out = static_cast<T*>(c.q_out) + (int64_t)t * c.ld_q + (int64_t)head * hd;
  T* keys = nullptr;
  T* values = nullptr;
  if (!is_q) {
    const int64_t base = kv_block_base(c.kv, c.tok_seq[t], pos, head);
    keys = static_cast<T*>(c.kv.keys) + base;
    values = static_cast<T*>(c.kv.values) + base;
  }
  auto store = [&](int col, float v) {
    if (is_q)
      q_out[col] = from_float<T>(v);
    else if (is_k)
      keys[key_offset(hd, pos, col)] = from_float<T>(v);
    else
      values[value_offset(hd, pos, col)] = from_float<T>(v);
  };
  // a lane takes a pair of channels: the angle's sine and cosine are computed once for both
  if (turned)
    for (int i = lane; i < half; i += 64) {
      float sn, cs;
      sincosf((float)pos * c.inv_freq[i], &sn, &cs);
      sn *= c.amplitude;
      cs *= c.amplitude;
      const int first = c.pairing == 1 ? 2 * i : i, second = c.pairing == 1 ? 2 * i + 1 : i + half;
      const float u = row[first], v = row[second];
      store(first, u * cs - v * sn);
      store(second, v * cs + u * sn);
    }
  for (int col = (turned ? c.rot_dims : 0) + lane; col < hd; col += 64) store(col, col < n ? row[col] : 0.f);
}

BT_EXPORT int bt_head_rotary_call(void* stream, const HeadRotaryCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->heads <= 0 || c->kv_heads <= 0 || c->heads % c->kv_heads != 0)
    BT_REFUSE("head_rotary: %d query heads cannot share %d key/value heads", c->heads, c->kv_heads);
  if (c->dim <= 0 || c->vdim <= 0 || c->dim > HR_MAX_DIM || c->vdim > HR_MAX_DIM)
    BT_REFUSE("head_rotary: head sizes %d and %d outside 1..%d", c->dim, c->vdim, HR_MAX_DIM);
  if ((c->pairing != 0 && c->pairing != 1) || (c->norm_span != 0 && c->norm_span != 1))
    BT_REFUSE("head_rotary: pairing %d and norm_span %d must be 0 or 1", c->pairing, c->norm_span);
  if (c->rot_dims < 0 || c->rot_dims % 2 != 0 || c->rot_dims > c->dim)
    BT_REFUSE("head_rotary: %d turned channels must be even and at most the head size %d", c->rot_dims, c->dim);
  if (c->kv.kv_heads != c->kv_heads || c->kv.head_dim < c->dim || c->kv.head_dim < c->vdim || c->kv.head_dim > HR_MAX_DIM)
    BT_REFUSE("head_rotary: the cache keeps %d heads of %d, the mixer has %d of %d and %d", c->kv.kv_heads,
              c->kv.head_dim, c->kv_heads, c->dim, c->vdim);
  if (c->ld < (int64_t)(c->heads + c->kv_heads) * c->dim + (int64_t)c->kv_heads * c->vdim ||
      c->ld_q < (int64_t)c->heads * c->kv.head_dim)
    BT_REFUSE("head_rotary: the rows do not hold the heads");
  if (!c->in || !c->q_out || !c->tok_seq || !c->tok_pos || !c->kv.blocks || !c->kv.keys || !c->kv.values ||
      (c->rot_dims > 0 && !c->inv_freq))
    BT_REFUSE("head_rotary: missing operand");
  const int units = c->heads + 2 * c->kv_heads;
  dim3 grid(c->tokens, (units + HR_WAVES - 1) / HR_WAVES), block(HR_WAVES * 64);
  if (c->dtype == 0)
    hipLaunchKernelGGL(head_rotary_kernel<float>, grid, block, 0, (hipStream_t)stream, *c);
  else
    hipLaunchKernelGGL(head_rotary_kernel<bf16_t>, grid, block, 0, (hipStream_t)stream, *c);
  return bt_check_launch("head_rotary");
}
