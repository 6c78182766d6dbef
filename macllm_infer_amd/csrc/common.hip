// Embedding gather, residual add + RMSNorm, SwiGLU, logit scaling.
// The residual stream is float32; activations are float32 or bfloat16.
#include "common.h"

// ---------------------------------------------------------------- embedding
// h[t, :] = table[ids[t], :] * multiplier        (reference: src/decoder.rs:3194-3197)
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const T* __restrict__ table, float multiplier,
                             float* __restrict__ h, int d) {
  const long token = blockIdx.x;
  const T* row = table + (long)ids[token] * d;
  float* out = h + token * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) out[i] = to_float(row[i]) * multiplier;
}

extern "C" int mi_embed(const int* ids, const void* table, int table_dtype, float multiplier, float* h,
                        int T, int d, hipStream_t stream) {
  if (T <= 0 || d <= 0) return ERR_BAD_ARGUMENT;
  if (table_dtype == DT_F32)
    embed_kernel<float><<<T, 256, 0, stream>>>(ids, (const float*)table, multiplier, h, d);
  else if (table_dtype == DT_BF16)
    embed_kernel<bf16_t><<<T, 256, 0, stream>>>(ids, (const bf16_t*)table, multiplier, h, d);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- tokens fed from the device
// token_ids[dst[i]] = source[src[i]]: the tokens that the sampler left on the device for the step before go
// into this step's token ids without a round trip through the host (the host learns them one step late).
// The pairs travel in the launch's arguments, 64 a launch: no memory of their own.
#define FEED_PAIRS 64
struct FeedPairs {
  int dst[FEED_PAIRS];
  int src[FEED_PAIRS];
};

__global__ void feed_tokens_kernel(int* __restrict__ token_ids, const int* __restrict__ source, int count, FeedPairs pairs) {
  const int i = threadIdx.x;
  if (i < count) token_ids[pairs.dst[i]] = source[pairs.src[i]];
}

// dst, src: host arrays of `count` indices; every dst below tokens, every src below sources (checked here).
extern "C" int mi_feed_tokens(int* token_ids, int tokens, const int* source, int sources, const int* dst,
                              const int* src, int count, hipStream_t stream) {
  if (count < 0 || tokens <= 0 || sources <= 0 || !token_ids || !source || (count > 0 && (!dst || !src)))
    return ERR_BAD_ARGUMENT;
  for (int i = 0; i < count; ++i)
    if (dst[i] < 0 || dst[i] >= tokens || src[i] < 0 || src[i] >= sources) return ERR_BAD_ARGUMENT;
  for (int first = 0; first < count; first += FEED_PAIRS) {
    FeedPairs pairs = {};
    const int n = count - first < FEED_PAIRS ? count - first : FEED_PAIRS;
    for (int i = 0; i < n; ++i) {
      pairs.dst[i] = dst[first + i];
      pairs.src[i] = src[first + i];
    }
    feed_tokens_kernel<<<1, FEED_PAIRS, 0, stream>>>(token_ids, source, n, pairs);
    RETURN_IF_LAUNCH_FAILED();
  }
  return 0;
}

// ---------------------------------------------------------------- add + rmsnorm
// For each processed row r:  v = h[r] (+ factor0 * delta0[r]) (+ factor1 * delta1[r]);  if update: h[r] = v;
// out[i] = v / sqrt(mean(v^2) + eps) * weight.
// With `rows` the kernel processes h[rows[i]] and writes out[i] (h is not updated).
// The sum of squares is accumulated in float32 in an order fixed by (d, blockDim) alone,
// so a row's result does not depend on what else is in the batch.
template <typename TD, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta0,
                                   const TD* __restrict__ delta1, const float* __restrict__ weight, float eps,
                                   TO* __restrict__ out, const int* __restrict__ rows, int d, float factor0,
                                   float factor1) {
  extern __shared__ float row_values[];
  __shared__ float scratch[16];
  const long out_row = blockIdx.x;
  const long row = rows ? (long)rows[out_row] : out_row;
  float* hr = h + row * d;
  float sum_squares = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    float v = hr[i];
    if (delta0) v = fmaf(factor0, to_float(delta0[row * d + i]), v);
    if (delta1) v = fmaf(factor1, to_float(delta1[row * d + i]), v);
    if (!rows && (delta0 || delta1)) hr[i] = v;
    row_values[i] = v;
    sum_squares += v * v;
  }
  const float total = block_sum(sum_squares, scratch);
  const float denominator = sqrtf(total / (float)d + eps);
  if (out) {
    TO* o = out + out_row * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x)
      o[i] = from_float<TO>(row_values[i] / denominator * weight[i]);
  }
}

// The same with four consecutive elements a thread and every load of a row asked for before the
// first is used (d a multiple of 4, at most 256 * 4 * NORM_MAX_ROUNDS).  The order of the sum is
// again fixed by d alone.
#define NORM_MAX_ROUNDS 8
template <typename T> struct Vec4;
template <> struct Vec4<float> { typedef float type __attribute__((ext_vector_type(4))); };
template <> struct Vec4<bf16_t> { typedef __bf16 type __attribute__((ext_vector_type(4))); };

template <typename TD, typename TO, int ROUNDS>
__global__ void __launch_bounds__(256)
add_rmsnorm_vec_kernel(float* __restrict__ h, const TD* __restrict__ delta0, const TD* __restrict__ delta1,
                       const float* __restrict__ weight, float eps, TO* __restrict__ out,
                       const int* __restrict__ rows, int d, float factor0, float factor1) {
  typedef typename Vec4<float>::type f4;
  typedef typename Vec4<TD>::type d4;
  typedef typename Vec4<TO>::type o4;
  __shared__ float scratch[16];
  const long out_row = blockIdx.x;
  const long row = rows ? (long)rows[out_row] : out_row;
  float* hr = h + row * d;
  // every load first and none under a condition (a wait counts all loads before it): an absent delta
  // reads the row itself and is dropped, a column past the end reads the last one
  const TD* d0 = delta0 ? delta0 + row * d : reinterpret_cast<const TD*>(hr);
  const TD* d1 = delta1 ? delta1 + row * d : reinterpret_cast<const TD*>(hr);
  f4 v[ROUNDS], w[ROUNDS];
  d4 a[ROUNDS], b[ROUNDS];
  int at[ROUNDS];
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) at[r] = min(((int)threadIdx.x + r * 256) * 4, d - 4);
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) v[r] = *reinterpret_cast<const f4*>(hr + at[r]);
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) a[r] = *reinterpret_cast<const d4*>(d0 + at[r]);
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) b[r] = *reinterpret_cast<const d4*>(d1 + at[r]);
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) w[r] = *reinterpret_cast<const f4*>(weight + at[r]);
  float sum_squares = 0.f;
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const bool mine = ((int)threadIdx.x + r * 256) * 4 < d;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float value = v[r][j];
      if (delta0) value = fmaf(factor0, (float)a[r][j], value);        // a factor of one adds the delta as it is
      if (delta1) value = fmaf(factor1, (float)b[r][j], value);
      v[r][j] = value;
      if (mine) sum_squares += value * value;
    }
    if (mine && !rows && (delta0 || delta1)) *reinterpret_cast<f4*>(hr + at[r]) = v[r];
  }
  const float total = block_sum(sum_squares, scratch);
  const float denominator = sqrtf(total / (float)d + eps);
  if (out) {
    TO* o = out + out_row * d;
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
      if (((int)threadIdx.x + r * 256) * 4 < d) {
        o4 packed;
#pragma unroll
        for (int j = 0; j < 4; ++j) packed[j] = from_float<TO>(v[r][j] / denominator * w[r][j]);
        *reinterpret_cast<o4*>(o + at[r]) = packed;
      }
    }
  }
}

// ---------------------------------------------------------------- residual add of partial sums + RMSNorm
// The same as add_rmsnorm for a branch that arrives as S float32 slabs [S, T, d] (a product split
// over K): h[row] += sum over the slabs (in slab order), out = h / sqrt(mean(h^2) + eps) * w.
// One workgroup per row; a thread takes four columns at a time and asks for all its slabs at once.
#define PARTIALS_MOST 16
template <typename TO>
__global__ void __launch_bounds__(256)
add_partials_rmsnorm_kernel(float* __restrict__ h, const float* __restrict__ partial, int S, long slab,
                            const float* __restrict__ weight, float eps, TO* __restrict__ out,
                            const int* __restrict__ rows, int d) {
  typedef typename Vec4<float>::type f4;
  typedef typename Vec4<TO>::type o4;
  __shared__ float scratch[16];
  const long out_row = blockIdx.x;
  const long row = rows ? (long)rows[out_row] : out_row;
  float* hr = h + row * d;
  const float* pr = partial + row * d;
  float sum_squares = 0.f;
  for (int column = (int)threadIdx.x * 4; column < d; column += 256 * 4) {
    f4 value = *reinterpret_cast<const f4*>(hr + column);
    f4 parts[PARTIALS_MOST];
#pragma unroll
    for (int s = 0; s < PARTIALS_MOST; ++s) parts[s] = *reinterpret_cast<const f4*>(pr + (long)min(s, S - 1) * slab + column);
#pragma unroll
    for (int s = 0; s < PARTIALS_MOST; ++s)
      if (s < S) {
#pragma unroll
        for (int j = 0; j < 4; ++j) value[j] += parts[s][j];
      }
#pragma unroll
    for (int j = 0; j < 4; ++j) sum_squares += value[j] * value[j];
    *reinterpret_cast<f4*>(hr + column) = value;       // with `rows` the caller passes a copy's row: see the launcher
  }
  const float total = block_sum(sum_squares, scratch);
  const float denominator = sqrtf(total / (float)d + eps);
  if (out) {
    TO* o = out + out_row * d;
    for (int column = (int)threadIdx.x * 4; column < d; column += 256 * 4) {
      const f4 value = *reinterpret_cast<const f4*>(hr + column);
      const f4 w = *reinterpret_cast<const f4*>(weight + column);
      o4 packed;
#pragma unroll
      for (int j = 0; j < 4; ++j) packed[j] = from_float<TO>(value[j] / denominator * w[j]);
      *reinterpret_cast<o4*>(o + column) = packed;
    }
  }
}

// With `rows` (a gather: only those rows are normed) the stream itself must stay as it is, and a row may be
// asked for twice; the kernel above writes the sums back, so gathers are refused here and the caller adds
// the partial sums to the stream first (rows == nullptr, out == nullptr) and gathers with mi_add_rmsnorm.
extern "C" int mi_add_partials_rmsnorm(float* h, const float* partial, int S, const float* weight, float eps,
                                       void* out, int out_dtype, const int* rows, int n_rows, int T, int d,
                                       hipStream_t stream) {
  if (!h || !partial || !weight || S < 1 || n_rows <= 0 || T <= 0 || d <= 0) return ERR_BAD_ARGUMENT;
  if (rows) return ERR_BAD_ARGUMENT;
  if (S > PARTIALS_MOST || d % 4 != 0) return ERR_UNSUPPORTED_SIZE;
  const long slab = (long)T * d;
  if (out_dtype == DT_BF16)
    add_partials_rmsnorm_kernel<bf16_t><<<n_rows, 256, 0, stream>>>(h, partial, S, slab, weight, eps, (bf16_t*)out, rows, d);
  else if (out_dtype == DT_F32)
    add_partials_rmsnorm_kernel<float><<<n_rows, 256, 0, stream>>>(h, partial, S, slab, weight, eps, (float*)out, rows, d);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

extern "C" int mi_add_rmsnorm(float* h, const void* delta0, const void* delta1, int delta_dtype,
                              const float* weight, float eps, void* out, int out_dtype, const int* rows,
                              int n_rows, int d, float factor0, float factor1, hipStream_t stream) {
  if (n_rows <= 0 || d <= 0) return ERR_BAD_ARGUMENT;
  const bool vectors = d % 4 == 0 && d <= 256 * 4 * NORM_MAX_ROUNDS && ((uintptr_t)h % 16) == 0 &&
                       ((uintptr_t)delta0 % 16) == 0 && ((uintptr_t)delta1 % 16) == 0 &&
                       ((uintptr_t)out % 16) == 0 && ((uintptr_t)weight % 16) == 0;
  if (!vectors && (size_t)d * sizeof(float) > 64 * 1024) return ERR_UNSUPPORTED_SIZE;
  const size_t lds = (size_t)d * sizeof(float);
#define LAUNCH(TD, TO)                                                                                      \
  do {                                                                                                      \
    if (vectors && d <= 1024)                                                                               \
      add_rmsnorm_vec_kernel<TD, TO, 1><<<n_rows, 256, 0, stream>>>(h, (const TD*)delta0, (const TD*)delta1, \
                                                                    weight, eps, (TO*)out, rows, d, factor0, factor1); \
    else if (vectors && d <= 2048)                                                                          \
      add_rmsnorm_vec_kernel<TD, TO, 2><<<n_rows, 256, 0, stream>>>(h, (const TD*)delta0, (const TD*)delta1, \
                                                                    weight, eps, (TO*)out, rows, d, factor0, factor1); \
    else if (vectors && d <= 4096)                                                                          \
      add_rmsnorm_vec_kernel<TD, TO, 4><<<n_rows, 256, 0, stream>>>(h, (const TD*)delta0, (const TD*)delta1, \
                                                                    weight, eps, (TO*)out, rows, d, factor0, factor1); \
    else if (vectors)                                                                                       \
      add_rmsnorm_vec_kernel<TD, TO, NORM_MAX_ROUNDS><<<n_rows, 256, 0, stream>>>(                          \
          h, (const TD*)delta0, (const TD*)delta1, weight, eps, (TO*)out, rows, d, factor0, factor1);       \
    else                                                                                                    \
      add_rmsnorm_kernel<TD, TO><<<n_rows, 256, lds, stream>>>(h, (const TD*)delta0, (const TD*)delta1,     \
                                                               weight, eps, (TO*)out, rows, d, factor0, factor1); \
  } while (0)
  if (delta_dtype == DT_F32 && out_dtype == DT_F32) LAUNCH(float, float);
  else if (delta_dtype == DT_BF16 && out_dtype == DT_BF16) LAUNCH(bf16_t, bf16_t);
  else if (delta_dtype == DT_F32 && out_dtype == DT_BF16) LAUNCH(float, bf16_t);
  else if (delta_dtype == DT_BF16 && out_dtype == DT_F32) LAUNCH(bf16_t, float);
  else return ERR_BAD_ARGUMENT;
#undef LAUNCH
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- branches normed each on its own, then summed
// out[r] = sum over the branches b (in their order) of factor_b * x_b[r] / sqrt(mean(x_b[r]^2) + eps_b) * weight_b,
// float32: the outputs of a layer's mixers, each through an RMS norm of its own, before they join the stream.
// One workgroup a row; a branch's sum of squares is a float32 sum whose order the width alone fixes.
#define NORMED_SUM_MOST 4
struct NormedSumBranches {
  const void* rows[NORMED_SUM_MOST];
  const float* weight[NORMED_SUM_MOST];
  float factor[NORMED_SUM_MOST];
  float eps[NORMED_SUM_MOST];
  int is_bf16[NORMED_SUM_MOST];
  long ld[NORMED_SUM_MOST];
};

__global__ void __launch_bounds__(256)
normed_sum_kernel(NormedSumBranches branches, int count, float* __restrict__ out, int d) {
  __shared__ float scratch[16];
  const long row = blockIdx.x;
  float scale[NORMED_SUM_MOST];
  for (int b = 0; b < count; ++b) {
    float squares = 0.f;
    if (branches.is_bf16[b]) {
      const bf16_t* x = (const bf16_t*)branches.rows[b] + row * branches.ld[b];
      for (int i = threadIdx.x; i < d; i += blockDim.x) {
        const float v = to_float(x[i]);
        squares = fmaf(v, v, squares);
      }
    } else {
      const float* x = (const float*)branches.rows[b] + row * branches.ld[b];
      for (int i = threadIdx.x; i < d; i += blockDim.x) squares = fmaf(x[i], x[i], squares);
    }
    const float total = block_sum(squares, scratch);
    scale[b] = 1.0f / sqrtf(total / (float)d + branches.eps[b]);
  }
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    float sum = 0.f;
    for (int b = 0; b < count; ++b) {
      const float v = branches.is_bf16[b] ? to_float(((const bf16_t*)branches.rows[b])[row * branches.ld[b] + i])
                                          : ((const float*)branches.rows[b])[row * branches.ld[b] + i];
      sum = fmaf(branches.factor[b], v * scale[b] * branches.weight[b][i], sum);
    }
    out[row * d + i] = sum;
  }
}

// The same for rows of up to THREADS * ROUNDS numbers: a thread asks for all its elements of every branch at once and
// keeps them in registers, the branches' sums of squares cross the workgroup together (one barrier), and the row
// is read once.  A step of a few rows is a chain of waits, and this takes most of them out.
template <int ROUNDS, int THREADS>
__global__ void __launch_bounds__(THREADS)
normed_sum_rows_kernel(NormedSumBranches branches, int count, float* __restrict__ out, int d) {
  __shared__ float sums[THREADS / WAVE][NORMED_SUM_MOST];
  const long row = blockIdx.x;
  const int lane = threadIdx.x & (WAVE - 1);
  const int wave = threadIdx.x / WAVE;
  float values[NORMED_SUM_MOST][ROUNDS];
#pragma unroll
  for (int b = 0; b < NORMED_SUM_MOST; ++b) {
    const int from = b < count ? b : 0;           // an absent branch reads the first again and is dropped
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
      const int i = min((int)threadIdx.x + THREADS * r, d - 1);
      values[b][r] = branches.is_bf16[from] ? to_float(((const bf16_t*)branches.rows[from])[row * branches.ld[from] + i])
                                            : ((const float*)branches.rows[from])[row * branches.ld[from] + i];
    }
  }
  float squares[NORMED_SUM_MOST];
#pragma unroll
  for (int b = 0; b < NORMED_SUM_MOST; ++b) {
    squares[b] = 0.f;
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r)
      if ((int)threadIdx.x + THREADS * r < d) squares[b] = fmaf(values[b][r], values[b][r], squares[b]);
    squares[b] = wave_sum(squares[b]);
    if (lane == 0) sums[wave][b] = squares[b];
  }
  __syncthreads();
  float scale[NORMED_SUM_MOST];
#pragma unroll
  for (int b = 0; b < NORMED_SUM_MOST; ++b) {
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < THREADS / WAVE; ++w) total += sums[w][b];
    scale[b] = b < count ? branches.factor[b] / sqrtf(total / (float)d + branches.eps[b]) : 0.f;
  }
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const int i = (int)threadIdx.x + THREADS * r;
    if (i >= d) break;
    float sum = 0.f;
#pragma unroll
    for (int b = 0; b < NORMED_SUM_MOST; ++b)
      if (b < count) sum = fmaf(values[b][r] * scale[b], branches.weight[b][i], sum);
    out[row * d + i] = sum;
  }
}

extern "C" int mi_normed_sum(const void* const* rows, const int* dtypes, const long* lds, const float* const* weights,
                             const float* factors, const float* eps, int count, float* out, int T, int d,
                             hipStream_t stream) {
  if (!rows || !dtypes || !lds || !weights || !factors || !eps || !out || count <= 0 || T <= 0 || d <= 0)
    return ERR_BAD_ARGUMENT;
  if (count > NORMED_SUM_MOST) return ERR_UNSUPPORTED_SIZE;
  NormedSumBranches branches;
  for (int b = 0; b < NORMED_SUM_MOST; ++b) {
    const int from = b < count ? b : 0;
    if (!rows[from] || !weights[from] || lds[from] < d || !(eps[from] > 0.f)) return ERR_BAD_ARGUMENT;
    if (dtypes[from] != DT_F32 && dtypes[from] != DT_BF16) return ERR_BAD_ARGUMENT;
    branches.rows[b] = rows[from];
    branches.weight[b] = weights[from];
    branches.factor[b] = factors[from];
    branches.eps[b] = eps[from];
    branches.is_bf16[b] = dtypes[from] == DT_BF16;
    branches.ld[b] = lds[from];
  }
  if (d <= 256 * 4) normed_sum_rows_kernel<4, 256><<<T, 256, 0, stream>>>(branches, count, out, d);
  else if (d <= 1024 * 4) normed_sum_rows_kernel<4, 1024><<<T, 1024, 0, stream>>>(branches, count, out, d);
  else if (d <= 1024 * 8) normed_sum_rows_kernel<8, 1024><<<T, 1024, 0, stream>>>(branches, count, out, d);
  else normed_sum_kernel<<<T, 256, 0, stream>>>(branches, count, out, d);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- SwiGLU
// out[t, i] = SiLU(g[t, i]) * u[t, i]      (reference: src/decoder.rs:298-305)
// A row of the input holds [g | u] (tile = 0), or g and u interleaved in tiles:
// [g[0:tile] | u[0:tile] | g[tile:2 tile] | ...], the layout the fused decode kernel wants its
// weight rows in (tile = 8), so that one matrix serves both.
__device__ __forceinline__ long swiglu_gate_at(int i, int I, int tile) {
  return tile == 0 ? i : (long)(i / tile) * 2 * tile + i % tile;
}

// the gate's activation: 0 SiLU, 1 the tanh form of GELU, 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))
__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
// the same through the hardware's exponential: tanh(y) = 1 - 2 / (1 + e^(2y)); for results rounded to bfloat16 at once
__device__ __forceinline__ float gelu_tanh_bf16_f(float z) {
  const float y = 0.7978845608028654f * (z + 0.044715f * z * z * z);
  return z * (1.0f - __frcp_rn(1.0f + __expf(2.0f * y)));
}

template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, long ld, T* __restrict__ out, int I, int tile, long total,
                              int activation) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= total) return;
  const long t = index / I;
  const int i = (int)(index - t * I);
  const long at = swiglu_gate_at(i, I, tile);
  const float gate = to_float(gu[t * ld + at]);
  const float up = to_float(gu[t * ld + at + (tile == 0 ? I : tile)]);
  out[index] = from_float<T>((activation == 1 ? gelu_tanh_f(gate) : silu_f(gate)) * up);
}

// bfloat16, eight elements a thread (I, ld and the addresses multiples of 8 elements; tile 0 or 8)
typedef __bf16 common_bf16x8 __attribute__((ext_vector_type(8)));
__global__ void __launch_bounds__(256)
swiglu_vec_kernel(const bf16_t* __restrict__ gu, long ld, bf16_t* __restrict__ out, int I, int tile, long total,
                  int activation) {
  const long index = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (index >= total) return;
  const long t = index / I;
  const int i = (int)(index - t * I);
  const long at = tile == 0 ? i : 2L * i;
  const common_bf16x8 gate = *reinterpret_cast<const common_bf16x8*>(gu + t * ld + at);
  const common_bf16x8 up = *reinterpret_cast<const common_bf16x8*>(gu + t * ld + at + (tile == 0 ? I : 8));
  common_bf16x8 result;
#pragma unroll
  for (int j = 0; j < 8; ++j)
    result[j] = (bf16_t)((activation == 1 ? gelu_tanh_bf16_f((float)gate[j]) : silu_bf16_f((float)gate[j])) * (float)up[j]);
  *reinterpret_cast<common_bf16x8*>(out + index) = result;
}

extern "C" int mi_swiglu(const void* gu, int dtype, long ld, void* out, int T, int I, int tile, int activation,
                         hipStream_t stream) {
  if (T <= 0 || I <= 0 || ld < 2L * I || tile < 0 || (tile > 0 && I % tile != 0) || (activation != 0 && activation != 1))
    return ERR_BAD_ARGUMENT;
  const long total = (long)T * I;
  const int blocks = (int)((total + 255) / 256);
  if (dtype == DT_BF16 && I % 8 == 0 && ld % 8 == 0 && (tile == 0 || tile == 8) && ((uintptr_t)gu % 16) == 0 &&
      ((uintptr_t)out % 16) == 0) {
    const int vec_blocks = (int)((total / 8 + 255) / 256);
    swiglu_vec_kernel<<<vec_blocks, 256, 0, stream>>>((const bf16_t*)gu, ld, (bf16_t*)out, I, tile, total, activation);
  } else if (dtype == DT_F32)
    swiglu_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, ld, (float*)out, I, tile, total, activation);
  else if (dtype == DT_BF16)
    swiglu_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, ld, (bf16_t*)out, I, tile, total, activation);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- float32 rows into a matrix of activations
// out[t * ld + i] = (T)source[t * d + i]
template <typename T>
__global__ void cast_rows_kernel(const float* __restrict__ source, T* __restrict__ out, long ld, int d, long total) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= total) return;
  const long t = index / d;
  out[t * ld + (index - t * d)] = from_float<T>(source[index]);
}

extern "C" int mi_cast_rows(const float* source, void* out, int dtype, long ld, int T, int d, hipStream_t stream) {
  if (!source || !out || T <= 0 || d <= 0 || ld < d) return ERR_BAD_ARGUMENT;
  const long total = (long)T * d;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == DT_F32)
    cast_rows_kernel<float><<<blocks, 256, 0, stream>>>(source, (float*)out, ld, d, total);
  else if (dtype == DT_BF16)
    cast_rows_kernel<bf16_t><<<blocks, 256, 0, stream>>>(source, (bf16_t*)out, ld, d, total);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- logits to float32
// out[i] = (float)in[i] * multiplier              (reference: src/decoder.rs:3349-3357)
template <typename T>
__global__ void scale_to_f32_kernel(const T* __restrict__ in, float multiplier, float* __restrict__ out, long total) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index < total) out[index] = to_float(in[index]) * multiplier;
}

extern "C" int mi_scale_to_f32(const void* in, int dtype, float multiplier, float* out, long total,
                               hipStream_t stream) {
  if (total <= 0) return ERR_BAD_ARGUMENT;
  const int blocks = (int)((total + 255) / 256);
  if (dtype == DT_F32)
    scale_to_f32_kernel<float><<<blocks, 256, 0, stream>>>((const float*)in, multiplier, out, total);
  else if (dtype == DT_BF16)
    scale_to_f32_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)in, multiplier, out, total);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- a cap on the logits
// x <- cap * tanh(x / cap), in place on float32 (reference: src/decoder.rs:4791-4796, after the scaling of the
// logits, :3349-3355)
__global__ void tanh_softcap_kernel(float* __restrict__ x, float cap, float inverse, long total) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index < total) x[index] = cap * tanhf(x[index] * inverse);
}

extern "C" int mi_tanh_softcap(float* x, float cap, long total, hipStream_t stream) {
  if (total <= 0 || !x || !(cap > 0.f)) return ERR_BAD_ARGUMENT;
  const int blocks = (int)((total + 255) / 256);
  tanh_softcap_kernel<<<blocks, 256, 0, stream>>>(x, cap, 1.0f / cap, total);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- bias behind a library product
// out[m, n] = bf16(sums[m, n] + bias[n]): the float32 sums of a bfloat16 product get their float32 bias and are
// rounded once (reference: src/model_weights.rs:530-545 adds the bias to the product's result).
__global__ void add_bias_round_kernel(const float* __restrict__ sums, const float* __restrict__ bias,
                                      bf16_t* __restrict__ out, int N, long total) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index < total) out[index] = (bf16_t)(sums[index] + bias[index % N]);
}

extern "C" int mi_add_bias_round(const float* sums, const float* bias, void* out, int M, int N, hipStream_t stream) {
  if (M <= 0 || N <= 0 || !sums || !bias || !out) return ERR_BAD_ARGUMENT;
  const long total = (long)M * N;
  add_bias_round_kernel<<<(int)((total + 255) / 256), 256, 0, stream>>>(sums, bias, (bf16_t*)out, N, total);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- scaled residual add + rmsnorm
// add_rmsnorm for a branch that is multiplied, feature by feature, by a float32 vector where it joins the stream:
//   v = h[r] + scale * delta[r] (the product and the sum in float32);  if no `rows`: h[r] = v;
//   out[i] = v / sqrt(mean(v^2) + eps) * weight     (out may be null: the add alone).
// One workgroup a row; a thread keeps its elements of the row in registers (up to SCALED_MAX_ROUNDS * 256 columns)
// or, for wider rows, in LDS.  The sum of squares is added up in an order that d and the workgroup's size fix.
#define SCALED_MAX_ROUNDS 8
template <typename TD, typename TO, bool IN_LDS>
__global__ void __launch_bounds__(1024)
add_scaled_rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta, const float* __restrict__ scale,
                          const float* __restrict__ weight, float eps, TO* __restrict__ out,
                          const int* __restrict__ rows, int d) {
  extern __shared__ float wide_row[];
  __shared__ float scratch[16];
  const long out_row = blockIdx.x;
  const long row = rows ? (long)rows[out_row] : out_row;
  float* hr = h + row * d;
  const TD* dr = delta + row * d;
  float kept[SCALED_MAX_ROUNDS];
  float sum_squares = 0.f;
  if (IN_LDS) {
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
      const float v = fmaf(scale[i], to_float(dr[i]), hr[i]);
      if (!rows) hr[i] = v;
      wide_row[i] = v;
      sum_squares += v * v;
    }
  } else {
#pragma unroll
    for (int r = 0; r < SCALED_MAX_ROUNDS; ++r) {
      const int i = (int)threadIdx.x + r * (int)blockDim.x;
      const int at = min(i, d - 1);
      const float v = fmaf(scale[at], to_float(dr[at]), hr[at]);
      kept[r] = v;
      if (i < d) {
        if (!rows) hr[i] = v;
        sum_squares += v * v;
      }
    }
  }
  if (!out) return;
  const float total = block_sum(sum_squares, scratch);
  const float denominator = sqrtf(total / (float)d + eps);
  TO* o = out + out_row * d;
  if (IN_LDS) {
    for (int i = threadIdx.x; i < d; i += blockDim.x) o[i] = from_float<TO>(wide_row[i] / denominator * weight[i]);
  } else {
#pragma unroll
    for (int r = 0; r < SCALED_MAX_ROUNDS; ++r) {
      const int i = (int)threadIdx.x + r * (int)blockDim.x;
      if (i < d) o[i] = from_float<TO>(kept[r] / denominator * weight[i]);
    }
  }
}

extern "C" int mi_add_scaled_rmsnorm(float* h, const void* delta, int delta_dtype, const float* scale,
                                     const float* weight, float eps, void* out, int out_dtype, const int* rows,
                                     int n_rows, int d, hipStream_t stream) {
  if (!h || !delta || !scale || !weight || n_rows <= 0 || d <= 0) return ERR_BAD_ARGUMENT;
  // 256 threads a row; a wide row of a step of few rows 1,024, so that the step still has waves to hide its waits
  // (a prompt's thousands of rows fill the GPU as they are: 26 us against 19 for 2,048 rows of 3,072 with the wide ones)
  const int threads = (d > 2048 && n_rows <= 512) ? 1024 : 256;
  const bool in_lds = d > threads * SCALED_MAX_ROUNDS;
  if (in_lds && (size_t)d * sizeof(float) > 64 * 1024) return ERR_UNSUPPORTED_SIZE;
  const size_t lds = in_lds ? (size_t)d * sizeof(float) : 0;
#define LAUNCH(TD, TO)                                                                                              \
  do {                                                                                                              \
    if (in_lds)                                                                                                     \
      add_scaled_rmsnorm_kernel<TD, TO, true><<<n_rows, threads, lds, stream>>>(h, (const TD*)delta, scale, weight, eps, \
                                                                            (TO*)out, rows, d);                     \
    else                                                                                                            \
      add_scaled_rmsnorm_kernel<TD, TO, false><<<n_rows, threads, 0, stream>>>(h, (const TD*)delta, scale, weight, eps,  \
                                                                           (TO*)out, rows, d);                      \
  } while (0)
  if (delta_dtype == DT_F32 && out_dtype == DT_F32) LAUNCH(float, float);
  else if (delta_dtype == DT_BF16 && out_dtype == DT_BF16) LAUNCH(bf16_t, bf16_t);
  else if (delta_dtype == DT_F32 && out_dtype == DT_BF16) LAUNCH(float, bf16_t);
  else if (delta_dtype == DT_BF16 && out_dtype == DT_F32) LAUNCH(bf16_t, float);
  else return ERR_BAD_ARGUMENT;
#undef LAUNCH
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- PolyNorm
// out[t, i] = c0 * z / rms(z) + c1 * z^2 / rms(z^2) + c2 * z^3 / rms(z^3) + c3, with rms(x) = sqrt(mean over the
// row of x^2 + eps): the three sums of squares of a token's row (z^2, z^4, z^6) in float32, one pass; the row is
// read a second time (it is in cache) for the result.  One workgroup a row.
template <typename T>
__global__ void __launch_bounds__(1024)
polynorm_kernel(const T* __restrict__ z, long ld, const float* __restrict__ coefficients, float eps,
                T* __restrict__ out, long out_ld, int I) {
  __shared__ float scratch[16];
  const T* zr = z + (long)blockIdx.x * ld;
  float first = 0.f, second = 0.f, third = 0.f;
  for (int i = threadIdx.x; i < I; i += blockDim.x) {
    const float x = to_float(zr[i]);
    const float x2 = x * x;
    first += x2;
    second += x2 * x2;
    third += x2 * x2 * x2;
  }
  const float mean1 = block_sum(first, scratch) / (float)I;
  const float mean2 = block_sum(second, scratch) / (float)I;
  const float mean3 = block_sum(third, scratch) / (float)I;
  const float a = coefficients[0] / sqrtf(mean1 + eps);
  const float b = coefficients[1] / sqrtf(mean2 + eps);
  const float c = coefficients[2] / sqrtf(mean3 + eps);
  const float e = coefficients[3];
  T* o = out + (long)blockIdx.x * out_ld;
  for (int i = threadIdx.x; i < I; i += blockDim.x) {
    const float x = to_float(zr[i]);
    o[i] = from_float<T>(fmaf(x, fmaf(x, fmaf(x, c, b), a), e));
  }
}

extern "C" int mi_polynorm(const void* z, int dtype, long ld, const float* coefficients, float eps, void* out,
                           long out_ld, int T, int I, hipStream_t stream) {
  if (!z || !coefficients || !out || T <= 0 || I <= 0 || ld < I || out_ld < I) return ERR_BAD_ARGUMENT;
  const int threads = (I > 2048 && T <= 512) ? 1024 : 256;          // as add_scaled_rmsnorm: wide rows of few-row steps
  if (dtype == DT_F32)
    polynorm_kernel<float><<<T, threads, 0, stream>>>((const float*)z, ld, coefficients, eps, (float*)out, out_ld, I);
  else if (dtype == DT_BF16)
    polynorm_kernel<bf16_t><<<T, threads, 0, stream>>>((const bf16_t*)z, ld, coefficients, eps, (bf16_t*)out, out_ld, I);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- embedding with a hashed bigram row
// h[t, :] = table[ids[t], :] * multiplier + bigram[row, :], row = (token before * mul_prev + token * mul_cur) mod
// buckets, or `buckets` (the table's last row) for the token at position 0.  The token before a lane's first
// one is the request's state, previous[slot]; a second, tiny launch leaves the lane's last token there (a launch
// of its own: the rows of a lane are read by many workgroups).
template <typename T>
__global__ void embed_bigram_kernel(const int* __restrict__ ids, const T* __restrict__ table, float multiplier,
                                    const T* __restrict__ bigram, int buckets, long mul_prev, long mul_cur,
                                    const int* __restrict__ positions, const int* __restrict__ lane_of_token,
                                    const int* __restrict__ cu_seqlens, const int* __restrict__ slot_ids,
                                    const int* __restrict__ previous, float* __restrict__ h, int d) {
  const long token = blockIdx.x;
  const int id = ids[token];
  long row = buckets;
  if (positions[token] != 0) {
    const int lane = lane_of_token[token];
    const long before = token == cu_seqlens[lane] ? previous[slot_ids[lane]] : ids[token - 1];
    row = (before * mul_prev + (long)id * mul_cur) % buckets;
    if (row < 0) row += buckets;
  }
  const T* first = table + (long)id * d;
  const T* second = bigram + row * d;
  float* out = h + token * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) out[i] = fmaf(to_float(first[i]), multiplier, to_float(second[i]));
}

__global__ void keep_last_token_kernel(const int* __restrict__ ids, const int* __restrict__ cu_seqlens,
                                       const int* __restrict__ slot_ids, int* __restrict__ previous, int lanes) {
  const int lane = blockIdx.x * blockDim.x + threadIdx.x;
  if (lane >= lanes) return;
  const int end = cu_seqlens[lane + 1];
  if (end > cu_seqlens[lane]) previous[slot_ids[lane]] = ids[end - 1];
}

extern "C" int mi_embed_bigram(const int* ids, const void* table, int table_dtype, float multiplier, const void* bigram,
                               int buckets, long mul_prev, long mul_cur, const int* positions, const int* lane_of_token,
                               const int* cu_seqlens, const int* slot_ids, int* previous, float* h, int T, int d,
                               int lanes, hipStream_t stream) {
  if (T <= 0 || d <= 0 || lanes <= 0 || buckets <= 0 || !ids || !table || !bigram || !positions || !lane_of_token ||
      !cu_seqlens || !slot_ids || !previous || !h)
    return ERR_BAD_ARGUMENT;
  if (table_dtype == DT_F32)
    embed_bigram_kernel<float><<<T, 256, 0, stream>>>(ids, (const float*)table, multiplier, (const float*)bigram, buckets,
                                                      mul_prev, mul_cur, positions, lane_of_token, cu_seqlens, slot_ids,
                                                      previous, h, d);
  else if (table_dtype == DT_BF16)
    embed_bigram_kernel<bf16_t><<<T, 256, 0, stream>>>(ids, (const bf16_t*)table, multiplier, (const bf16_t*)bigram,
                                                       buckets, mul_prev, mul_cur, positions, lane_of_token, cu_seqlens,
                                                       slot_ids, previous, h, d);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  keep_last_token_kernel<<<(lanes + 255) / 256, 256, 0, stream>>>(ids, cu_seqlens, slot_ids, previous, lanes);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- h += factor * rows + vector
template <typename T>
__global__ void stream_add_kernel(float* __restrict__ h, const T* __restrict__ rows, float factor,
                                  const float* __restrict__ vector, long total, int d) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  float value = h[i];
  if (rows) value = fmaf(factor, to_float(rows[i]), value);
  if (vector) value += vector[i % d];
  h[i] = value;
}

extern "C" int mi_stream_add(float* h, const void* rows, int rows_dtype, float factor, const float* vector, int T, int d,
                             hipStream_t stream) {
  if (!h || T <= 0 || d <= 0) return ERR_BAD_ARGUMENT;
  const long total = (long)T * d;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (rows_dtype == DT_F32)
    stream_add_kernel<float><<<blocks, 256, 0, stream>>>(h, (const float*)rows, factor, vector, total, d);
  else if (rows_dtype == DT_BF16)
    stream_add_kernel<bf16_t><<<blocks, 256, 0, stream>>>(h, (const bf16_t*)rows, factor, vector, total, d);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- residual add + layer norm
// v = h + f0 b0 + f1 b1 + f2 b2 + vector (float32; written back to h unless rows are gathered);
// out = (v - mean) / sqrt(mean((v - mean)^2) + eps) * weight + bias.  The row is kept in LDS; the variance is
// taken from the deviations in a second pass over it.  One workgroup a row.
struct NormBranch {
  const void* rows;
  int dtype;
  float factor;
};

__device__ __forceinline__ float branch_value(const NormBranch& branch, long at) {
  if (!branch.rows) return 0.f;
  const float value = branch.dtype == DT_BF16 ? (float)((const bf16_t*)branch.rows)[at] : ((const float*)branch.rows)[at];
  return branch.factor * value;
}

template <typename TO>
__global__ void __launch_bounds__(1024)
add_layernorm_kernel(float* __restrict__ h, NormBranch b0, NormBranch b1, NormBranch b2, const float* __restrict__ vector,
                     const float* __restrict__ weight, const float* __restrict__ bias, float eps,
                     const float* __restrict__ branch_weight, const float* __restrict__ branch_bias, float branch_eps,
                     TO* __restrict__ out, const int* __restrict__ rows, int d) {
  extern __shared__ float wide_row[];
  __shared__ float scratch[16];
  const long out_row = blockIdx.x;
  const long row = rows ? (long)rows[out_row] : out_row;
  float sum = 0.f;
  if (branch_weight) {
    // the branches' sum goes through a layer norm of its own on its way into the stream: the sum is laid in LDS,
    // its mean and the variance of its deviations are taken as below, and the normed row is added to h
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
      const long at = row * d + i;
      float v = branch_value(b0, at);
      v += branch_value(b1, at);
      v += branch_value(b2, at);
      wide_row[i] = v;
      sum += v;
    }
    const float branch_mean = block_sum(sum, scratch) / (float)d;
    float branch_squares = 0.f;
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
      const float centred = wide_row[i] - branch_mean;
      branch_squares += centred * centred;
    }
    const float branch_denominator = sqrtf(block_sum(branch_squares, scratch) / (float)d + branch_eps);
    sum = 0.f;
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
      const long at = row * d + i;
      float v = h[at] + ((wide_row[i] - branch_mean) / branch_denominator * branch_weight[i] + branch_bias[i]);
      if (vector) v += vector[i];
      h[at] = v;
      wide_row[i] = v;
      sum += v;
    }
  } else {
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
      const long at = row * d + i;
      float v = h[at];
      v += branch_value(b0, at);
      v += branch_value(b1, at);
      v += branch_value(b2, at);
      if (vector) v += vector[i];
      if (!rows) h[at] = v;
      wide_row[i] = v;
      sum += v;
    }
  }
  if (!out) return;
  const float mean = block_sum(sum, scratch) / (float)d;
  float squares = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    const float centred = wide_row[i] - mean;
    squares += centred * centred;
  }
  const float variance = block_sum(squares, scratch) / (float)d;
  const float denominator = sqrtf(variance + eps);
  TO* o = out + out_row * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x)
    o[i] = from_float<TO>((wide_row[i] - mean) / denominator * weight[i] + bias[i]);
}

// The same for steps of few rows, whose time is the chain of waits: a thread keeps PER elements of the row in
// registers (element threadIdx.x + k * blockDim.x), and everything the later stages read from memory (the stream's
// row, the norms' weights and biases) is asked for at the start, beside the branches' rows.
template <typename TO, int PER>
__global__ void __launch_bounds__(1024)
add_layernorm_rows_kernel(float* __restrict__ h, NormBranch b0, NormBranch b1, NormBranch b2,
                          const float* __restrict__ vector, const float* __restrict__ weight,
                          const float* __restrict__ bias, float eps, const float* __restrict__ branch_weight,
                          const float* __restrict__ branch_bias, float branch_eps, TO* __restrict__ out,
                          const int* __restrict__ rows, int d) {
  __shared__ float scratch[16];
  const long out_row = blockIdx.x;
  const long row = rows ? (long)rows[out_row] : out_row;
  float branches[PER], stream[PER], bw[PER], bb[PER], w[PER], b[PER], v[PER];
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = threadIdx.x + k * blockDim.x;
    const bool live = i < d;
    const long at = row * d + i;
    branches[k] = 0.f;
    if (live) {
      branches[k] = branch_value(b0, at);
      branches[k] += branch_value(b1, at);
      branches[k] += branch_value(b2, at);
    }
    stream[k] = live ? h[at] : 0.f;
    bw[k] = (live && branch_weight) ? branch_weight[i] : 0.f;
    bb[k] = (live && branch_weight) ? branch_bias[i] : 0.f;
    w[k] = (live && out) ? weight[i] : 0.f;
    b[k] = (live && out) ? bias[i] : 0.f;
    v[k] = (live && vector) ? vector[i] : 0.f;
  }
  if (branch_weight) {
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < PER; ++k) sum += branches[k];
    const float branch_mean = block_sum(sum, scratch) / (float)d;
    float squares = 0.f;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const float centred = (int)(threadIdx.x + k * blockDim.x) < d ? branches[k] - branch_mean : 0.f;
      squares += centred * centred;
    }
    const float branch_denominator = sqrtf(block_sum(squares, scratch) / (float)d + branch_eps);
#pragma unroll
    for (int k = 0; k < PER; ++k) v[k] += stream[k] + ((branches[k] - branch_mean) / branch_denominator * bw[k] + bb[k]);
  } else {
#pragma unroll
    for (int k = 0; k < PER; ++k) v[k] += stream[k] + branches[k];
  }
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = threadIdx.x + k * blockDim.x;
    if (i >= d) v[k] = 0.f;
    else if (!rows) h[row * d + i] = v[k];
    sum += v[k];
  }
  if (!out) return;
  const float mean = block_sum(sum, scratch) / (float)d;
  float squares = 0.f;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const float centred = (int)(threadIdx.x + k * blockDim.x) < d ? v[k] - mean : 0.f;
    squares += centred * centred;
  }
  const float denominator = sqrtf(block_sum(squares, scratch) / (float)d + eps);
  TO* o = out + out_row * d;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = threadIdx.x + k * blockDim.x;
    if (i < d) o[i] = from_float<TO>((v[k] - mean) / denominator * w[k] + b[k]);
  }
}

template <typename TO>
static void launch_add_layernorm_rows(int per, int n_rows, int threads, hipStream_t stream, float* h, NormBranch b0,
                                      NormBranch b1, NormBranch b2, const float* vector, const float* weight,
                                      const float* bias, float eps, const float* branch_weight,
                                      const float* branch_bias, float branch_eps, TO* out, const int* rows, int d) {
#define ROWS_CASE(PER_)                                                                                          \
  if (per == PER_)                                                                                               \
    add_layernorm_rows_kernel<TO, PER_><<<n_rows, threads, 0, stream>>>(h, b0, b1, b2, vector, weight, bias, eps, \
                                                                        branch_weight, branch_bias, branch_eps,  \
                                                                        out, rows, d);
  ROWS_CASE(1) ROWS_CASE(2) ROWS_CASE(4) ROWS_CASE(8)
#undef ROWS_CASE
}

extern "C" int mi_add_layernorm(float* h, const void* rows0, int dtype0, float factor0, const void* rows1, int dtype1,
                                float factor1, const void* rows2, int dtype2, float factor2, const float* vector,
                                const float* weight, const float* bias, float eps, const float* branch_weight,
                                const float* branch_bias, float branch_eps, void* out, int out_dtype,
                                const int* rows, int n_rows, int d, hipStream_t stream) {
  if (!h || n_rows <= 0 || d <= 0) return ERR_BAD_ARGUMENT;
  if (out && (!weight || !bias)) return ERR_BAD_ARGUMENT;
  if (branch_weight && (!branch_bias || rows || !rows0)) return ERR_BAD_ARGUMENT;
  if ((size_t)d * sizeof(float) > 64 * 1024) return ERR_UNSUPPORTED_SIZE;
  const NormBranch b0 = {rows0, dtype0, factor0}, b1 = {rows1, dtype1, factor1}, b2 = {rows2, dtype2, factor2};
  if (n_rows <= 256 && d <= 8192 && (out_dtype == DT_F32 || out_dtype == DT_BF16)) {
    // few rows: the kernel that keeps a row in registers, as many threads as a row has elements where that fits
    const int per = d <= 1024 ? 1 : d <= 2048 ? 2 : d <= 4096 ? 4 : 8;
    const int row_threads = (((d + per - 1) / per + WAVE - 1) / WAVE) * WAVE;
    if (out_dtype == DT_F32)
      launch_add_layernorm_rows<float>(per, n_rows, row_threads, stream, h, b0, b1, b2, vector, weight, bias, eps,
                                       branch_weight, branch_bias, branch_eps, (float*)out, rows, d);
    else
      launch_add_layernorm_rows<bf16_t>(per, n_rows, row_threads, stream, h, b0, b1, b2, vector, weight, bias, eps,
                                        branch_weight, branch_bias, branch_eps, (bf16_t*)out, rows, d);
    RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  const int threads = (d > 2048 && n_rows <= 512) ? 1024 : 256;
  const size_t lds = (size_t)d * sizeof(float);
  if (out_dtype == DT_F32)
    add_layernorm_kernel<float><<<n_rows, threads, lds, stream>>>(h, b0, b1, b2, vector, weight, bias, eps, branch_weight,
                                                                  branch_bias, branch_eps, (float*)out, rows, d);
  else if (out_dtype == DT_BF16)
    add_layernorm_kernel<bf16_t><<<n_rows, threads, lds, stream>>>(h, b0, b1, b2, vector, weight, bias, eps, branch_weight,
                                                                   branch_bias, branch_eps, (bf16_t*)out, rows, d);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- clamped gated activation
// out[t, i] = g * sigmoid(alpha g) * (u + offset), g = min(gate, limit), u = clamp(up, -limit, limit); a row of
// gate_up holds [gate | up].
__device__ __forceinline__ float clamped_glu_f(float gate, float up, float limit, float alpha, float offset) {
  const float g = fminf(gate, limit);
  const float u = fminf(fmaxf(up, -limit), limit);
  return g / (1.0f + expf(-alpha * g)) * (u + offset);
}

template <typename T>
__global__ void clamped_glu_kernel(const T* __restrict__ gate_up, long ld, T* __restrict__ out, long out_ld, int I,
                                   long total, float limit, float alpha, float offset) {
  const long at = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (at >= total) return;
  const long t = at / I;
  const int i = (int)(at % I);
  const T* row = gate_up + t * ld;
  out[t * out_ld + i] = from_float<T>(clamped_glu_f(to_float(row[i]), to_float(row[I + i]), limit, alpha, offset));
}

extern "C" int mi_clamped_glu(const void* gate_up, int dtype, long ld, void* out, long out_ld, int T, int I, float limit,
                              float alpha, float offset, hipStream_t stream) {
  if (!gate_up || !out || T <= 0 || I <= 0 || ld < 2L * I || out_ld < I) return ERR_BAD_ARGUMENT;
  const long total = (long)T * I;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == DT_F32)
    clamped_glu_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gate_up, ld, (float*)out, out_ld, I, total, limit, alpha, offset);
  else if (dtype == DT_BF16)
    clamped_glu_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gate_up, ld, (bf16_t*)out, out_ld, I, total, limit, alpha, offset);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}
