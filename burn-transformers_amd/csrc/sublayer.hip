// Kernels for layers that normalise a sublayer's OUTPUT before it joins the residual stream, and
// for activations that are norms themselves.  All statistics and the residual sum are 32-bit.
//   * output norm: x[t] (+)= mult * N(v), v the sublayer's output (the sum of its partial sums and
//     its bias), N an RMS norm, v / sqrt(mean(v^2) + eps) * gamma, or a layer norm,
//     (v - mean) / sqrt(var + eps) * gamma + beta; and a copy of the new x in the products' type
//   * joined rows: [x | y] side by side in the products' type, the operand of a product that reads two streams
//   * PolyNorm: a N(z) + b N(z^2) + c N(z^3) + e, N(v) = v / sqrt(mean(v^2) + eps) over a row
#include "host.h"

struct OutputNormCall {
  int cast_dtype;        // element type of `cast`: 0 float32, 1 bfloat16
  int n_delta;           // partial sums of the sublayer's output; 0: the stream's own rows are normalised
  int tokens;
  int width;
  int accumulate;        // 1: x += mult * norm(v); 0: x = mult * norm(v)
  int cast_cols;         // columns of `cast` that are written: the new x, then zeros
  float eps;
  float mult;
  float* x;              // [tokens][width] float32 residual stream
  const float* delta;    // [n_delta][..][ldd]
  int64_t delta_stride;  // elements between two partial sums
  int64_t ldd;           // row pitch of a partial sum
  const float* bias;     // [width] or null: added to v
  const float* gamma;    // [width]
  void* cast;            // [tokens][ld_cast] or null
  int64_t ld_cast;
  int kind;              // 0: layer norm (mean taken off, `beta` added), 1: RMS norm
  const float* beta;     // [width] or null
  // The norm that reads the stream next, in the same pass over the row: next_out[t] = norm'(new x[t])
  // (what the next sublayer multiplies by).  next_out null: none.
  void* next_out;        // [tokens][next_ld] in the type `next_dtype`
  int64_t next_ld;
  int next_dtype;
  int next_kind;
  float next_eps;
  const float* next_gamma;
  const float* next_beta;   // or null
};

// y = N'(v) for one element, given the row's statistics
__device__ __forceinline__ float next_norm(const OutputNormCall& c, float v, float mean, float rstd, int col) {
  const float y = (v - mean) * rstd * c.next_gamma[col];
  return c.next_beta ? y + c.next_beta[col] : y;
}

template <typename T>
__global__ void __launch_bounds__(256) output_norm_kernel(OutputNormCall c) {
  extern __shared__ float row_buf[];
  __shared__ float scratch[32];
  const int t = blockIdx.x;
  float* xr = c.x + (int64_t)t * c.width;
  float partial = 0.f;
  for (int col = threadIdx.x; col < c.width; col += blockDim.x) {
    float v;
    if (c.n_delta == 0) {
      v = xr[col];
    } else {
      v = c.bias ? c.bias[col] : 0.f;
      for (int s = 0; s < c.n_delta; ++s) v += c.delta[s * c.delta_stride + (int64_t)t * c.ldd + col];
    }
    row_buf[col] = v;
    partial += v;
  }
  const float mean = c.kind == 0 ? block_sum(partial, scratch) / (float)c.width : 0.f;
  partial = 0.f;
  for (int col = threadIdx.x; col < c.width; col += blockDim.x) {
    const float d = row_buf[col] - mean;
    partial += d * d;
  }
  const float total = block_sum(partial, scratch);
  const float scale = c.mult / sqrtf(total / (float)c.width + c.eps);
  T* cast = static_cast<T*>(c.cast);
  for (int col = threadIdx.x; col < c.width; col += blockDim.x) {
    float y = (row_buf[col] - mean) * scale * c.gamma[col];
    if (c.beta) y += c.mult * c.beta[col];
    if (c.accumulate) y += xr[col];
    xr[col] = y;
    row_buf[col] = y;         // (a thread's own columns: read back below by the same thread)
    if (cast) cast[(int64_t)t * c.ld_cast + col] = from_float<T>(y);
  }
  if (cast)
    for (int col = c.width + threadIdx.x; col < c.cast_cols; col += blockDim.x)
      cast[(int64_t)t * c.ld_cast + col] = from_float<T>(0.f);
  if (c.next_out) {
    float sum = 0.f;
    if (c.next_kind == 0)
      for (int col = threadIdx.x; col < c.width; col += blockDim.x) sum += row_buf[col];
    const float next_mean = c.next_kind == 0 ? block_sum(sum, scratch) / (float)c.width : 0.f;
    sum = 0.f;
    for (int col = threadIdx.x; col < c.width; col += blockDim.x) sum += (row_buf[col] - next_mean) * (row_buf[col] - next_mean);
    const float next_rstd = 1.0f / sqrtf(block_sum(sum, scratch) / (float)c.width + c.next_eps);
    for (int col = threadIdx.x; col < c.width; col += blockDim.x) {
      const float y = next_norm(c, row_buf[col], next_mean, next_rstd, col);
      if (c.next_dtype == 0) static_cast<float*>(c.next_out)[(int64_t)t * c.next_ld + col] = y;
      else static_cast<bf16_t*>(c.next_out)[(int64_t)t * c.next_ld + col] = (bf16_t)y;
    }
  }
}

// The same for rows of up to 256 * KMAX columns: a thread's columns live in registers and every load
// of a thread (partial sums, bias, the stream, the scale) is issued before the first is used, so a
// row costs one round trip to memory.  A decode step has few rows: one row's latency is its time.
template <typename T, int KMAX>
__global__ void __launch_bounds__(256) output_norm_small_kernel(OutputNormCall c) {
  __shared__ float scratch[32];
  const int t = blockIdx.x;
  float* xr = c.x + (int64_t)t * c.width;
  // Every load of a thread is issued before the first is used and none stands behind a branch of its
  // own (columns beyond the row and partial sums beyond the last are read from a valid place and
  // dropped): loads behind branches, or in a loop of unknown length, are waited for one by one, and
  // a row then costs as many round trips to memory as it has of them (measured: 14 us for 16 of them).
  float v[KMAX], xv[KMAX], g[KMAX], b[KMAX];
  int cc[KMAX];
  bool in_row[KMAX];
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    const int col = threadIdx.x + 256 * k;
    in_row[k] = col < c.width;
    cc[k] = in_row[k] ? col : 0;
  }
  const float* beta = c.beta ? c.beta : c.gamma;           // (read in any case, used only where there is one)
  const float* bias = c.bias ? c.bias : c.gamma;
  const float* gamma2 = c.next_out ? c.next_gamma : c.gamma;
  const float* beta2 = c.next_out && c.next_beta ? c.next_beta : c.gamma;
  float g2[KMAX], b2[KMAX];
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    g2[k] = gamma2[cc[k]];
    b2[k] = beta2[cc[k]];
    g[k] = c.gamma[cc[k]];
    b[k] = beta[cc[k]];
    xv[k] = xr[cc[k]];
    v[k] = bias[cc[k]];
  }
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    b[k] = c.beta ? c.mult * b[k] : 0.f;
    v[k] = c.bias ? v[k] : 0.f;
  }
  if (c.n_delta == 0) {
#pragma unroll
    for (int k = 0; k < KMAX; ++k) { v[k] = xv[k]; xv[k] = 0.f; }
  } else {
    const float* row = c.delta + (int64_t)t * c.ldd;
    for (int s0 = 0; s0 < c.n_delta; s0 += 4) {            // four partial sums at a time, all their loads together
      float part[4][KMAX];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int sc = s0 + u < c.n_delta ? s0 + u : c.n_delta - 1;
#pragma unroll
        for (int k = 0; k < KMAX; ++k) part[u][k] = row[sc * c.delta_stride + cc[k]];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int k = 0; k < KMAX; ++k) v[k] += s0 + u < c.n_delta ? part[u][k] : 0.f;
    }
    if (!c.accumulate)
#pragma unroll
      for (int k = 0; k < KMAX; ++k) xv[k] = 0.f;
  }
#pragma unroll
  for (int k = 0; k < KMAX; ++k)
    if (!in_row[k]) v[k] = xv[k] = g[k] = b[k] = 0.f;
  float partial = 0.f;
  if (c.kind == 0) {          // a layer norm: the mean first, then the squared distances from it
#pragma unroll
    for (int k = 0; k < KMAX; ++k) partial += v[k];
    const float mean = block_sum(partial, scratch) / (float)c.width;
#pragma unroll
    for (int k = 0; k < KMAX; ++k) v[k] = threadIdx.x + 256 * k < c.width ? v[k] - mean : 0.f;
    partial = 0.f;
  }
#pragma unroll
  for (int k = 0; k < KMAX; ++k) partial += v[k] * v[k];
  const float scale = c.mult / sqrtf(block_sum(partial, scratch) / (float)c.width + c.eps);
  T* cast = static_cast<T*>(c.cast);
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    const int col = threadIdx.x + 256 * k;
    if (col < c.width) {
      const float y = v[k] * scale * g[k] + b[k] + xv[k];
      xr[col] = y;
      v[k] = y;
      if (cast) cast[(int64_t)t * c.ld_cast + col] = from_float<T>(y);
    } else {
      v[k] = 0.f;
    }
  }
  if (cast)
    for (int col = c.width + threadIdx.x; col < c.cast_cols; col += blockDim.x)
      cast[(int64_t)t * c.ld_cast + col] = from_float<T>(0.f);
  if (c.next_out) {           // the norm that reads the new row next, from the registers that hold it
    float next_mean = 0.f;
    if (c.next_kind == 0) {
      float sum = 0.f;
#pragma unroll
      for (int k = 0; k < KMAX; ++k) sum += v[k];
      next_mean = block_sum(sum, scratch) / (float)c.width;
    }
    float squares = 0.f;
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      const float d = threadIdx.x + 256 * k < c.width ? v[k] - next_mean : 0.f;
      squares += d * d;
    }
    const float next_rstd = 1.0f / sqrtf(block_sum(squares, scratch) / (float)c.width + c.next_eps);
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      const int col = threadIdx.x + 256 * k;
      if (col < c.width) {
        const float y = (v[k] - next_mean) * next_rstd * g2[k] + (c.next_beta ? b2[k] : 0.f);
        if (c.next_dtype == 0) static_cast<float*>(c.next_out)[(int64_t)t * c.next_ld + col] = y;
        else static_cast<bf16_t*>(c.next_out)[(int64_t)t * c.next_ld + col] = (bf16_t)y;
      }
    }
  }
}

template <typename T>
static void launch_output_norm(hipStream_t stream, const OutputNormCall& c) {
  dim3 grid(c.tokens), block(256);
  if (c.width <= 1024)
    hipLaunchKernelGGL((output_norm_small_kernel<T, 4>), grid, block, 0, stream, c);
  else if (c.width <= 2048)
    hipLaunchKernelGGL((output_norm_small_kernel<T, 8>), grid, block, 0, stream, c);
  else
    hipLaunchKernelGGL(output_norm_kernel<T>, grid, block, (size_t)c.width * sizeof(float), stream, c);
}

BT_EXPORT int bt_output_norm_call(void* stream, const OutputNormCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->width <= 0 || c->width > 15360) BT_REFUSE("output_norm: width %d outside 1..15360", c->width);
  if (!c->x || !c->gamma || (c->n_delta > 0 && !c->delta)) BT_REFUSE("output_norm: missing operand");
  if (c->n_delta == 0 && c->accumulate) BT_REFUSE("output_norm: the stream's own rows cannot be added to themselves");
  if (c->kind != 0 && c->kind != 1) BT_REFUSE("output_norm: unknown kind of norm %d", c->kind);
  if (c->next_out && (!c->next_gamma || c->next_ld < c->width || (c->next_kind != 0 && c->next_kind != 1)))
    BT_REFUSE("output_norm: the norm that follows lacks its scale, its kind or room for its rows");
  if (c->cast && (c->cast_cols < c->width || c->ld_cast < c->cast_cols))
    BT_REFUSE("output_norm: a copy of %d columns in rows of %lld does not hold width %d", c->cast_cols,
              (long long)c->ld_cast, c->width);
  if (c->cast_dtype == 0)
    launch_output_norm<float>((hipStream_t)stream, *c);
  else
    launch_output_norm<bf16_t>((hipStream_t)stream, *c);
  return bt_check_launch("output_norm");
}

// out[t] = [x[t] | y[t] | zeros] in the products' type: the operand of a product over two float32
// streams laid side by side (W [x; y] as one product).
struct JoinRowsCall {
  int out_dtype;         // 0 float32, 1 bfloat16
  int tokens;
  int width;             // columns of x and of y
  int out_cols;          // columns of out written: 2 * width, then zeros
  const float* x;        // [tokens][width]
  const float* y;        // [tokens][width]
  void* out;             // [tokens][ldo]
  int64_t ldo;
};

template <typename T>
__global__ void __launch_bounds__(256) join_rows_kernel(JoinRowsCall c) {
  const int t = blockIdx.x;
  T* out = static_cast<T*>(c.out) + (int64_t)t * c.ldo;
  for (int col = threadIdx.x; col < c.out_cols; col += blockDim.x) {
    float v = 0.f;
    if (col < c.width) v = c.x[(int64_t)t * c.width + col];
    else if (col < 2 * c.width) v = c.y[(int64_t)t * c.width + col - c.width];
    out[col] = from_float<T>(v);
  }
}

BT_EXPORT int bt_join_rows_call(void* stream, const JoinRowsCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->width <= 0 || c->out_cols < 2 * c->width || c->ldo < c->out_cols)
    BT_REFUSE("join_rows: rows of %lld columns (%d written) do not hold two of width %d", (long long)c->ldo, c->out_cols, c->width);
  if (!c->x || !c->y || !c->out) BT_REFUSE("join_rows: missing operand");
  if (c->out_dtype == 0)
    hipLaunchKernelGGL(join_rows_kernel<float>, dim3(c->tokens), dim3(256), 0, (hipStream_t)stream, *c);
  else
    hipLaunchKernelGGL(join_rows_kernel<bf16_t>, dim3(c->tokens), dim3(256), 0, (hipStream_t)stream, *c);
  return bt_check_launch("join_rows");
}

struct PolyNormCall {
  int out_dtype;          // 0 float32, 1 bfloat16
  int tokens;
  int columns;            // the row's length: statistics are means over these
  int out_cols;           // columns of `out` that are written: the result, then zeros
  float eps;
  const float* z;         // [tokens][ldz] float32
  int64_t ldz;
  const float* coefficients;  // a, b, c, e
  void* out;              // [tokens][ldo]
  int64_t ldo;
};

// Three block-wide sums with one meeting of the waves (blocks of up to 1024 threads).
__device__ __forceinline__ void block_sum3(float& a, float& b, float& d, float* scratch) {
  a = wave_sum(a);
  b = wave_sum(b);
  d = wave_sum(d);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = (blockDim.x + 63) >> 6;
  if (lane == 0) {
    scratch[wave * 3] = a;
    scratch[wave * 3 + 1] = b;
    scratch[wave * 3 + 2] = d;
  }
  __syncthreads();
  a = b = d = 0.f;
  for (int w = 0; w < waves; ++w) {
    a += scratch[w * 3];
    b += scratch[w * 3 + 1];
    d += scratch[w * 3 + 2];
  }
}

template <typename T>
__global__ void __launch_bounds__(256) poly_norm_kernel(PolyNormCall c) {
  extern __shared__ float row_buf[];
  __shared__ float scratch[48];
  const int t = blockIdx.x;
  const float* zr = c.z + (int64_t)t * c.ldz;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int col = threadIdx.x; col < c.columns; col += blockDim.x) {
    const float v = zr[col];
    row_buf[col] = v;
    const float v2 = v * v;
    s2 += v2;
    s4 += v2 * v2;
    s6 += v2 * v2 * v2;
  }
  block_sum3(s2, s4, s6, scratch);
  const float n = (float)c.columns;
  const float a = c.coefficients[0] / sqrtf(s2 / n + c.eps);
  const float b = c.coefficients[1] / sqrtf(s4 / n + c.eps);
  const float d = c.coefficients[2] / sqrtf(s6 / n + c.eps);
  const float e = c.coefficients[3];
  T* out = static_cast<T*>(c.out) + (int64_t)t * c.ldo;
  for (int col = threadIdx.x; col < c.columns; col += blockDim.x) {
    const float v = row_buf[col];
    out[col] = from_float<T>(a * v + b * (v * v) + d * (v * v * v) + e);
  }
  for (int col = c.columns + threadIdx.x; col < c.out_cols; col += blockDim.x) out[col] = from_float<T>(0.f);
}

BT_EXPORT int bt_poly_norm_call(void* stream, const PolyNormCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->columns <= 0 || c->columns > 15360) BT_REFUSE("poly_norm: %d columns outside 1..15360", c->columns);
  if (!c->z || !c->coefficients || !c->out) BT_REFUSE("poly_norm: missing operand");
  if (c->out_cols < c->columns || c->ldo < c->out_cols || c->ldz < c->columns)
    BT_REFUSE("poly_norm: rows of %lld and %lld elements do not hold %d (%d) columns", (long long)c->ldz,
              (long long)c->ldo, c->columns, c->out_cols);
  dim3 grid(c->tokens), block(256);
  size_t lds = (size_t)c->columns * sizeof(float);
  if (c->out_dtype == 0)
    hipLaunchKernelGGL(poly_norm_kernel<float>, grid, block, lds, (hipStream_t)stream, *c);
  else
    hipLaunchKernelGGL(poly_norm_kernel<bf16_t>, grid, block, lds, (hipStream_t)stream, *c);
  return bt_check_launch("poly_norm");
}

// RMS norm in equal consecutive parts of a row ("groups"), each over its own root mean square, the whole
// times `gamma`; of a sublayer's output on its way into the stream, or of rows of the stream itself.
//   output (n_delta > 0):  v = scale * (sum of delta + bias) + scale2 * (sum of delta2 + bias2), the second
//       term for layers whose sublayer is two parts side by side; v *= sigmoid(gate) where a gate's
//       logits come with it; x[t] (+)= mult * N(v), and `cast` receives the new x in the products' type.
//   rows (n_delta == 0):   cast[r] = N(x[rows[r]]) (every row in order without `rows`); x stays as it is.
struct GroupNormCall {
  int cast_dtype;         // element type of `cast`: 0 float32, 1 bfloat16
  int tokens;             // rows of this call
  int width;
  int groups;             // equal parts of a row, each with statistics of its own
  int n_delta, n_delta2;
  int accumulate;         // output: 1: x += mult * N(v); 0: x = mult * N(v)
  int cast_cols;          // columns of `cast` that are written: the result, then zeros
  float eps, mult;
  float scale, scale2;    // factors of the two terms
  float* x;               // [..][width] float32 residual stream
  const float* delta;     // [n_delta][..][ldd]
  int64_t delta_stride, ldd;
  const float* bias;      // [width] or null
  const float* delta2;    // [n_delta2][..][ldd2], or null
  int64_t delta2_stride, ldd2;
  const float* bias2;     // [width] or null
  const float* gate;      // [tokens][ld_gate] logits, or null
  int64_t ld_gate;
  const float* gamma;     // [width]
  void* cast;             // [tokens][ld_cast], or null
  int64_t ld_cast;
  const int* rows;        // rows mode: which rows of x, or null
};

template <typename T>
__global__ void __launch_bounds__(256) group_norm_kernel(GroupNormCall c) {
  extern __shared__ float row_buf[];          // [width], then [groups] reciprocal roots
  float* rstd = row_buf + c.width;
  const int t = blockIdx.x;
  const bool from_stream = c.n_delta == 0;
  const int source = from_stream && c.rows ? c.rows[t] : t;
  float* xr = c.x + (int64_t)source * c.width;
  for (int col = threadIdx.x; col < c.width; col += blockDim.x) {
    float v;
    if (from_stream) {
      v = xr[col];
    } else {
      v = c.bias ? c.bias[col] : 0.f;
      for (int s = 0; s < c.n_delta; ++s) v += c.delta[s * c.delta_stride + (int64_t)t * c.ldd + col];
      v *= c.scale;
      if (c.n_delta2 > 0) {
        float w = c.bias2 ? c.bias2[col] : 0.f;
        for (int s = 0; s < c.n_delta2; ++s) w += c.delta2[s * c.delta2_stride + (int64_t)t * c.ldd2 + col];
        v = fmaf(c.scale2, w, v);
      }
      if (c.gate) v *= 1.0f / (1.0f + expf(-c.gate[(int64_t)t * c.ld_gate + col]));
    }
    row_buf[col] = v;
  }
  __syncthreads();
  // a wave takes whole parts, so no sum crosses waves
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  const int per = c.width / c.groups;
  for (int g = wave; g < c.groups; g += waves) {
    float squares = 0.f;
    for (int i = lane; i < per; i += 64) squares = fmaf(row_buf[g * per + i], row_buf[g * per + i], squares);
    squares = wave_sum(squares);
    if (lane == 0) rstd[g] = 1.0f / sqrtf(squares / (float)per + c.eps);
  }
  __syncthreads();
  T* cast = static_cast<T*>(c.cast);
  for (int col = threadIdx.x; col < c.width; col += blockDim.x) {
    float y = row_buf[col] * rstd[col / per] * c.gamma[col];
    if (!from_stream) {
      y *= c.mult;
      if (c.accumulate) y += xr[col];
      xr[col] = y;
    }
    if (cast) cast[(int64_t)t * c.ld_cast + col] = from_float<T>(y);
  }
  if (cast)
    for (int col = c.width + threadIdx.x; col < c.cast_cols; col += blockDim.x)
      cast[(int64_t)t * c.ld_cast + col] = from_float<T>(0.f);
}

// The same for rows of up to 256 * KMAX columns: a thread's columns live in registers, and every load of a
// thread (partial sums of both terms, biases, the gate, the stream, the scale) is issued before the first is
// used and none stands behind a branch of its own, so a row costs one round trip to memory (a decode step has
// few rows: one row's latency is its time).  The parts' sums of squares meet in LDS, a wave a part.
template <typename T, int KMAX>
__global__ void __launch_bounds__(256) group_norm_small_kernel(GroupNormCall c) {
  extern __shared__ float row_buf[];          // [width], then [groups] reciprocal roots
  float* rstd = row_buf + c.width;
  const int t = blockIdx.x;
  const bool from_stream = c.n_delta == 0;
  const int source = from_stream && c.rows ? c.rows[t] : t;
  float* xr = c.x + (int64_t)source * c.width;
  float v[KMAX], w[KMAX], xv[KMAX], g[KMAX], gt[KMAX];
  int cc[KMAX];
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    const int col = threadIdx.x + 256 * k;
    cc[k] = col < c.width ? col : 0;
  }
  const float* bias = c.bias ? c.bias : c.gamma;           // (read in any case, used only where there is one)
  const float* bias2 = c.bias2 ? c.bias2 : c.gamma;
  const float* gate = c.gate ? c.gate + (int64_t)t * c.ld_gate : c.gamma;
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    g[k] = c.gamma[cc[k]];
    xv[k] = xr[cc[k]];
    v[k] = bias[cc[k]];
    w[k] = bias2[cc[k]];
    gt[k] = gate[cc[k]];
  }
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    v[k] = c.bias ? v[k] : 0.f;
    w[k] = c.bias2 ? w[k] : 0.f;
  }
  if (from_stream) {
#pragma unroll
    for (int k = 0; k < KMAX; ++k) v[k] = xv[k];
  } else {
    const float* row = c.delta + (int64_t)t * c.ldd;
    for (int s0 = 0; s0 < c.n_delta; s0 += 4) {            // four partial sums at a time, all their loads together
      float part[4][KMAX];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int sc = s0 + u < c.n_delta ? s0 + u : c.n_delta - 1;
#pragma unroll
        for (int k = 0; k < KMAX; ++k) part[u][k] = row[sc * c.delta_stride + cc[k]];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int k = 0; k < KMAX; ++k) v[k] += s0 + u < c.n_delta ? part[u][k] : 0.f;
    }
    const float* row2 = c.delta2 + (int64_t)t * c.ldd2;
    for (int s0 = 0; s0 < c.n_delta2; s0 += 4) {
      float part[4][KMAX];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int sc = s0 + u < c.n_delta2 ? s0 + u : c.n_delta2 - 1;
#pragma unroll
        for (int k = 0; k < KMAX; ++k) part[u][k] = row2[sc * c.delta2_stride + cc[k]];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int k = 0; k < KMAX; ++k) w[k] += s0 + u < c.n_delta2 ? part[u][k] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      v[k] *= c.scale;
      if (c.n_delta2 > 0) v[k] = fmaf(c.scale2, w[k], v[k]);
      if (c.gate) v[k] *= 1.0f / (1.0f + expf(-gt[k]));
    }
  }
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    const int col = threadIdx.x + 256 * k;
    if (col < c.width) row_buf[col] = v[k];
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  const int per = c.width / c.groups;
  for (int part = wave; part < c.groups; part += waves) {
    float squares = 0.f;
    for (int i = lane; i < per; i += 64) squares = fmaf(row_buf[part * per + i], row_buf[part * per + i], squares);
    squares = wave_sum(squares);
    if (lane == 0) rstd[part] = 1.0f / sqrtf(squares / (float)per + c.eps);
  }
  __syncthreads();
  T* cast = static_cast<T*>(c.cast);
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    const int col = threadIdx.x + 256 * k;
    if (col < c.width) {
      float y = v[k] * rstd[col / per] * g[k];
      if (!from_stream) {
        y *= c.mult;
        if (c.accumulate) y += xv[k];
        xr[col] = y;
      }
      if (cast) cast[(int64_t)t * c.ld_cast + col] = from_float<T>(y);
    }
  }
  if (cast)
    for (int col = c.width + threadIdx.x; col < c.cast_cols; col += blockDim.x)
      cast[(int64_t)t * c.ld_cast + col] = from_float<T>(0.f);
}

template <typename T>
static void launch_group_norm(hipStream_t stream, const GroupNormCall& c) {
  const size_t lds = (size_t)(c.width + c.groups) * sizeof(float);
  dim3 grid(c.tokens), block(256);
  if (c.width <= 1024)
    hipLaunchKernelGGL((group_norm_small_kernel<T, 4>), grid, block, lds, stream, c);
  else if (c.width <= 2048)
    hipLaunchKernelGGL((group_norm_small_kernel<T, 8>), grid, block, lds, stream, c);
  else
    hipLaunchKernelGGL(group_norm_kernel<T>, grid, block, lds, stream, c);
}

BT_EXPORT int bt_group_norm_call(void* stream, const GroupNormCall* c) {
  if (c->tokens <= 0) return BT_OK;
  if (c->width <= 0 || c->width > 15360) BT_REFUSE("group_norm: width %d outside 1..15360", c->width);
  if (c->groups <= 0 || c->groups > 512 || c->width % c->groups != 0)
    BT_REFUSE("group_norm: %d parts (1..512) must divide width %d", c->groups, c->width);
  if (!c->x || !c->gamma || (c->n_delta > 0 && !c->delta) || (c->n_delta2 > 0 && !c->delta2))
    BT_REFUSE("group_norm: missing operand");
  if (c->n_delta == 0 && (!c->cast || c->n_delta2 > 0 || c->gate))
    BT_REFUSE("group_norm: rows of the stream are normalised into `cast`, with one term and no gate");
  if (c->n_delta < 0 || c->n_delta2 < 0) BT_REFUSE("group_norm: negative counts of partial sums");
  if (c->cast && (c->cast_cols < c->width || c->ld_cast < c->cast_cols))
    BT_REFUSE("group_norm: a copy of %d columns in rows of %lld does not hold width %d", c->cast_cols,
              (long long)c->ld_cast, c->width);
  if (c->gate && c->ld_gate < c->width) BT_REFUSE("group_norm: the gate's rows are shorter than the width");
  if (c->cast_dtype == 0)
    launch_group_norm<float>((hipStream_t)stream, *c);
  else
    launch_group_norm<bf16_t>((hipStream_t)stream, *c);
  return bt_check_launch("group_norm");
}

// logits <- cap * tanh(logits / cap), in place, over float32 rows.
struct SoftCapCall {
  int rows;
  int columns;
  float cap;
  float* logits;          // [rows][ld]
  int64_t ld;
};

__global__ void __launch_bounds__(256) soft_cap_kernel(SoftCapCall c) {
  float* row = c.logits + (int64_t)blockIdx.x * c.ld;
  const float inverse = 1.0f / c.cap;
  for (int col = blockIdx.y * blockDim.x + threadIdx.x; col < c.columns; col += gridDim.y * blockDim.x)
    row[col] = c.cap * tanhf(row[col] * inverse);
}

BT_EXPORT int bt_soft_cap_call(void* stream, const SoftCapCall* c) {
  if (c->rows <= 0) return BT_OK;
  if (c->columns <= 0 || c->ld < c->columns || !c->logits) BT_REFUSE("soft_cap: missing operand or rows too short");
  if (!(c->cap > 0.f)) BT_REFUSE("soft_cap: the cap %g must be positive", (double)c->cap);
  int per_row = (c->columns + 2047) / 2048;
  if (per_row > 64) per_row = 64;
  hipLaunchKernelGGL(soft_cap_kernel, dim3(c->rows, per_row), dim3(256), 0, (hipStream_t)stream, *c);
  return bt_check_launch("soft_cap");
}
