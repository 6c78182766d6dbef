// Latent attention: the kernels around the attention proper.
//
//   latent_prepare   a token's down-projected row [query latent | key/value latent | key part to turn] -> the RMS
//                    norm of the query latent; the RMS norm of the key/value latent and the turned key part into
//                    the token's cache cell (K page: [latent | turned part], V page, transposed: the latent)
//   rotate_heads     a part of every head's row turned by position into another matrix
//   head_gemm        one product per head on the matrix cores (queries into the latent space, attended latents out)
//
// Norms, angles, sines and the turn itself are float32 whatever the activations are.
#include "mfma_tile.h"

// the pair (u, v) at angle a -> (u cos a - v sin a, v cos a + u sin a)
__device__ __forceinline__ void turn_pair(float u, float v, float angle, float& first, float& second) {
  float s, c;
  sincosf(angle, &s, &c);
  first = u * c - v * s;
  second = v * c + u * s;
}

// Element j of a row of `width` numbers after the turn of its first `rotary_dim`: pairs are (2i, 2i + 1)
// (interleaved) or (i, i + rotary_dim / 2).
template <typename T>
__device__ __forceinline__ float turned_element(const T* row, int j, int rotary_dim, int interleaved,
                                                const float* __restrict__ inv_freq, float position) {
  if (j >= rotary_dim) return to_float(row[j]);
  const int half = rotary_dim / 2;
  int pair, partner;
  bool is_first;
  if (interleaved) {
    pair = j / 2;
    is_first = (j & 1) == 0;
    partner = is_first ? j + 1 : j - 1;
  } else {
    pair = j < half ? j : j - half;
    is_first = j < half;
    partner = is_first ? j + half : j - half;
  }
  const float own = to_float(row[j]);
  const float other = to_float(row[partner]);
  float first, second;
  if (is_first) turn_pair(own, other, position * inv_freq[pair], first, second);
  else turn_pair(other, own, position * inv_freq[pair], first, second);
  return is_first ? first : second;
}

template <typename T>
__global__ void __launch_bounds__(256)
latent_prepare_kernel(const T* __restrict__ down, long ld, int q_rank, int kv_rank, int rope_dim,
                      const float* __restrict__ q_norm, const float* __restrict__ kv_norm, float eps,
                      const int* __restrict__ positions, const float* __restrict__ inv_freq, int rotary_dim,
                      int interleaved, const int* __restrict__ slot_mapping, T* __restrict__ k_cache,
                      T* __restrict__ v_cache, long page_stride, int page_size, T* __restrict__ q_latent, long q_ld) {
  __shared__ float scratch[16];
  const long token = blockIdx.x;
  const T* row = down + token * ld;
  float q_squares = 0.f, kv_squares = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) {
    const float v = to_float(row[i]);
    q_squares += v * v;
  }
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) {
    const float v = to_float(row[q_rank + i]);
    kv_squares += v * v;
  }
  const float q_denominator = sqrtf(block_sum(q_squares, scratch) / (float)q_rank + eps);
  const float kv_denominator = sqrtf(block_sum(kv_squares, scratch) / (float)kv_rank + eps);
  T* q_out = q_latent + token * q_ld;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x)
    q_out[i] = from_float<T>(to_float(row[i]) / q_denominator * q_norm[i]);
  if (!slot_mapping) return;
  const int cell = slot_mapping[token];
  const long page = cell / page_size;
  const int offset = cell % page_size;
  const int width = kv_rank + rope_dim;
  T* k_cell = k_cache + page * page_stride + (long)offset * width;
  T* v_cell = v_cache + page * page_stride + offset;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) {
    const T value = from_float<T>(to_float(row[q_rank + i]) / kv_denominator * kv_norm[i]);
    k_cell[i] = value;
    v_cell[(long)i * page_size] = value;
  }
  const float position = (float)positions[token];
  const T* part = row + q_rank + kv_rank;
  for (int j = threadIdx.x; j < rope_dim; j += blockDim.x)
    k_cell[kv_rank + j] = from_float<T>(turned_element(part, j, rotary_dim, interleaved, inv_freq, position));
}

extern "C" int mi_latent_prepare(const void* down, int dtype, long ld, int T, int q_rank, int kv_rank, int rope_dim,
                                 const float* q_norm, const float* kv_norm, float eps, const int* positions,
                                 const float* inv_freq, int rotary_dim, int interleaved, const int* slot_mapping,
                                 void* k_cache, void* v_cache, long page_stride, int page_size, void* q_latent, long q_ld,
                                 hipStream_t stream) {
  // q_rank 0: the row holds no query latent (queries projected directly); q_norm and q_latent are then not read
  if (!down || !kv_norm || !positions || T <= 0 || q_rank < 0 || (q_rank > 0 && (!q_norm || !q_latent)) || kv_rank <= 0 || rope_dim < 0 ||
      ld < q_rank + kv_rank + rope_dim || q_ld < q_rank || rotary_dim < 0 || rotary_dim > rope_dim || rotary_dim % 2 ||
      (rotary_dim > 0 && !inv_freq) || (slot_mapping && (!k_cache || !v_cache || page_size <= 0)))
    return ERR_BAD_ARGUMENT;
  if (dtype == DT_F32)
    latent_prepare_kernel<float><<<T, 256, 0, stream>>>((const float*)down, ld, q_rank, kv_rank, rope_dim, q_norm, kv_norm,
                                                        eps, positions, inv_freq, rotary_dim, interleaved, slot_mapping,
                                                        (float*)k_cache, (float*)v_cache, page_stride, page_size,
                                                        (float*)q_latent, q_ld);
  else if (dtype == DT_BF16)
    latent_prepare_kernel<bf16_t><<<T, 256, 0, stream>>>((const bf16_t*)down, ld, q_rank, kv_rank, rope_dim, q_norm,
                                                         kv_norm, eps, positions, inv_freq, rotary_dim, interleaved,
                                                         slot_mapping, (bf16_t*)k_cache, (bf16_t*)v_cache, page_stride,
                                                         page_size, (bf16_t*)q_latent, q_ld);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// out[t, out_col + h * out_head_stride + j] = turned x[t, col + h * head_stride + j], j < width
template <typename T>
__global__ void rotate_heads_kernel(const T* __restrict__ x, long ld, int col, int head_stride, int H, int width,
                                    const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                    int rotary_dim, int interleaved, T* __restrict__ out, long out_ld, int out_col,
                                    int out_head_stride) {
  const long token = blockIdx.x;
  const float position = (float)positions[token];
  for (int at = threadIdx.x; at < H * width; at += blockDim.x) {
    const int head = at / width;
    const int j = at % width;
    const T* row = x + token * ld + col + (long)head * head_stride;
    out[token * out_ld + out_col + (long)head * out_head_stride + j] =
        from_float<T>(turned_element(row, j, rotary_dim, interleaved, inv_freq, position));
  }
}

extern "C" int mi_rotate_heads(const void* x, int dtype, long ld, int col, int head_stride, int H, int width,
                               const int* positions, const float* inv_freq, int rotary_dim, int interleaved, void* out,
                               long out_ld, int out_col, int out_head_stride, int T, hipStream_t stream) {
  if (!x || !out || !positions || T <= 0 || H <= 0 || width <= 0 || rotary_dim < 0 || rotary_dim > width ||
      rotary_dim % 2 || (rotary_dim > 0 && !inv_freq) || col < 0 || out_col < 0)
    return ERR_BAD_ARGUMENT;
  const int threads = H * width >= 256 ? 256 : 64;
  if (dtype == DT_F32)
    rotate_heads_kernel<float><<<T, threads, 0, stream>>>((const float*)x, ld, col, head_stride, H, width, positions,
                                                          inv_freq, rotary_dim, interleaved, (float*)out, out_ld, out_col,
                                                          out_head_stride);
  else if (dtype == DT_BF16)
    rotate_heads_kernel<bf16_t><<<T, threads, 0, stream>>>((const bf16_t*)x, ld, col, head_stride, H, width, positions,
                                                           inv_freq, rotary_dim, interleaved, (bf16_t*)out, out_ld,
                                                           out_col, out_head_stride);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- one product per head
// out[m, out_col + h * out_head_stride + n] = sum_k x[m, x_col + h * x_head_stride + k] * W[h, n, k]
template <typename T, int MT, bool VEC>
__global__ void __launch_bounds__(TILE_THREADS)
head_gemm_kernel(const T* __restrict__ x, long ldx, int x_col, const T* __restrict__ W, int x_head_stride,
                 int out_head_stride, T* __restrict__ out, long ldo, int out_col, int M, int N, int K) {
  __shared__ float red[TILE_WAVES][256];
  const int tid = threadIdx.x;
  const int r = (tid & (WAVE - 1)) % 16;
  const int head = blockIdx.z;
  const long n0 = (long)blockIdx.x * 16;
  const long m0 = (long)blockIdx.y * 16 * MT;
  const T* w_row[1] = {W + ((long)head * N + min(n0 + r, (long)N - 1)) * K};
  const T* x_row[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
    x_row[mt] = x + min(m0 + 16 * mt + r, (long)M - 1) * ldx + x_col + (long)head * x_head_stride;
  tile_floatx4 acc[1][MT];
  tile_accumulate<T, MT, 1, VEC>(w_row, x_row, K, acc);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const float value = tile_reduce(acc[0][mt], red);
    const int l = tid % 64;
    const long n = n0 + 4 * (l / 16) + tid / 64;
    const long m = m0 + 16 * mt + (l % 16);
    if (n < N && m < M) out[m * ldo + out_col + (long)head * out_head_stride + n] = from_float<T>(value);
  }
}

template <typename T>
static int launch_head_gemm(const T* x, long ldx, int x_col, const T* W, int x_head_stride, int out_head_stride, T* out,
                            long ldo, int out_col, int M, int N, int K, int H, hipStream_t stream) {
  constexpr int PIECE = TileTraits<T>::PIECE;
  const bool vec = K % PIECE == 0 && ldx % PIECE == 0 && x_col % PIECE == 0 && x_head_stride % PIECE == 0 &&
                   ((unsigned long long)x % 16) == 0 && ((unsigned long long)W % 16) == 0;
  const int row_tiles = M <= 16 ? 1 : M <= 32 ? 2 : 4;
  const long blocks_y = ((long)M + 16 * row_tiles - 1) / (16 * row_tiles);
  if (blocks_y > 65535 || H > 65535) return ERR_UNSUPPORTED_SIZE;
  const dim3 grid((unsigned)((N + 15) / 16), (unsigned)blocks_y, (unsigned)H);
#define HEAD_LAUNCH(MT_)                                                                                              \
  do {                                                                                                                \
    if (vec)                                                                                                          \
      head_gemm_kernel<T, MT_, true><<<grid, TILE_THREADS, 0, stream>>>(x, ldx, x_col, W, x_head_stride,              \
                                                                        out_head_stride, out, ldo, out_col, M, N, K); \
    else                                                                                                              \
      head_gemm_kernel<T, MT_, false><<<grid, TILE_THREADS, 0, stream>>>(x, ldx, x_col, W, x_head_stride,             \
                                                                         out_head_stride, out, ldo, out_col, M, N, K); \
  } while (0)
  if (row_tiles == 1) HEAD_LAUNCH(1);
  else if (row_tiles == 2) HEAD_LAUNCH(2);
  else HEAD_LAUNCH(4);
#undef HEAD_LAUNCH
  return 0;
}

extern "C" int mi_head_gemm(const void* x, int dtype, long ldx, long x_col, const void* W, long x_head_stride,
                            long out_head_stride, void* out, long ldo, long out_col, int M, int N, int K, int H,
                            hipStream_t stream) {
  if (!x || !W || !out || M <= 0 || N <= 0 || K <= 0 || H <= 0 || x_col < 0 || out_col < 0 || x_head_stride < 0 ||
      out_head_stride < 0 || ldx < x_col + (H - 1) * x_head_stride + K || ldo < out_col + (H - 1) * out_head_stride + N)
    return ERR_BAD_ARGUMENT;
  int code;
  if (dtype == DT_F32)
    code = launch_head_gemm<float>((const float*)x, ldx, (int)x_col, (const float*)W, (int)x_head_stride,
                                   (int)out_head_stride, (float*)out, ldo, (int)out_col, M, N, K, H, stream);
  else if (dtype == DT_BF16)
    code = launch_head_gemm<bf16_t>((const bf16_t*)x, ldx, (int)x_col, (const bf16_t*)W, (int)x_head_stride,
                                    (int)out_head_stride, (bf16_t*)out, ldo, (int)out_col, M, N, K, H, stream);
  else
    return ERR_BAD_ARGUMENT;
  if (code) return code;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- prompt portions on the matrix cores
// Attention of a step's prompt portions over the cached rows [latent | turned part] (DK wide, one row a token for
// all heads; the values are the first DV of them, kept a second time transposed as the V pages), bfloat16.  The
// queries are already in the latent space.  A workgroup takes 16 consecutive tokens of one lane and NSET heads,
// which share every key and value fragment; its eight waves split the keys [0, last position] in runs of whole
// 32-key steps and merge through LDS, set by set (the scheme of the grouped-query prompt kernel, with every head in
// the one group).  Softmax in float32, in units of log2.
#include "attn_mfma.h"

#define LATENT_WAVES 8

template <int DK, int DV, int NSET, int STEPS>
__global__ void __launch_bounds__(LATENT_WAVES * WAVE)
latent_attention_kernel(const bf16_t* __restrict__ q, long q_ld, int H, const bf16_t* __restrict__ k_base,
                        const bf16_t* __restrict__ v_base, long page_stride, int page_size,
                        const int* __restrict__ block_tables, int max_pages, const int* __restrict__ tiles,
                        const int* __restrict__ cu_seqlens, const int* __restrict__ start_pos, float scale, int window,
                        bf16_t* __restrict__ out, long out_ld) {
  constexpr int ITEMS = 2 + 4 * (DV / 16);                    // m, l and the accumulator of one set
  __shared__ float part[LATENT_WAVES][ITEMS][WAVE];
  __shared__ int wave_pages[LATENT_WAVES][WAVE];
  // heavy tiles first; every other head pass the other way round
  const int block = (blockIdx.z & 1) ? blockIdx.x : gridDim.x - 1 - blockIdx.x;
  const int tile = block / 4;
  const int head0 = blockIdx.z * NSET;
  const int request = tiles[2 * tile];
  if (request < 0) return;                                    // a row of the table past the step's own runs
  const int lane = threadIdx.x & (WAVE - 1);
  const int wave = threadIdx.x / WAVE;
  const int qd = lane / 16;
  const int n = lane % 16;
  const int lane_end = cu_seqlens[request + 1];
  const int first_token = tiles[2 * tile + 1] + 16 * (block % 4);
  if (first_token >= lane_end) return;                        // the whole workgroup
  const int token = first_token + n;
  const bool has_query = token < lane_end;
  const int base_position = start_pos[request] - cu_seqlens[request];
  const int position = base_position + token;
  const int last_position = base_position + min(first_token + 15, lane_end - 1);
  const int first_position = base_position + first_token;
  const bool full_tile = first_token + 16 <= lane_end && head0 + NSET <= H;

  mfma_bf16x8 q_frag[NSET][DK / 32];
  int col_pos[NSET];
#pragma unroll
  for (int s = 0; s < NSET; ++s) {
    const bool valid = has_query && head0 + s < H;
    col_pos[s] = valid ? position : -1;
#pragma unroll
    for (int kk = 0; kk < DK / 32; ++kk) {
      if (valid) {
        q_frag[s][kk] = *reinterpret_cast<const mfma_bf16x8*>(q + (long)token * q_ld + (long)(head0 + s) * DK +
                                                               32 * kk + 8 * qd);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) q_frag[s][kk][j] = (bf16_t)0.f;
      }
    }
  }
  AttnAccumulator<DK, NSET, DV> acc;
  acc.clear();
  AttnCache cache;
  cache.k_base = k_base;
  cache.v_base = v_base;
  cache.page_stride = page_stride;
  cache.page_size = page_size;
  cache.kvh = 0;
  const int* cache_pages = block_tables + (long)request * max_pages;
  int key_lo = 0;
  if (window > 0 && first_position - window + 1 > 0) key_lo = ((first_position - window + 1) / 32) * 32;
  const int key_hi = last_position + 1;
  const int steps = (key_hi - key_lo + 31) / 32;
  const int steps_per_wave = (steps + LATENT_WAVES - 1) / LATENT_WAVES;
  const int my_lo = key_lo + 32 * steps_per_wave * wave;
  const int my_hi = min(key_hi, my_lo + 32 * steps_per_wave);
  // the page ids of the run go through LDS, 64 pages at a time (a wave's own corner of it: no barrier)
  for (int part_lo = my_lo; part_lo < my_hi;) {
    const int first_page = part_lo / page_size;
    const int part_hi = min(my_hi, (first_page + WAVE) * page_size);
    wave_pages[wave][lane] = cache_pages[min(first_page + lane, max_pages - 1)];
    cache.pages = wave_pages[wave];
    cache.base_page = first_page;
    attend_keys<DK, NSET, STEPS, false, false, DV>(acc, q_frag, col_pos, window, scale, part_lo, part_hi, cache,
                                                   full_tile ? first_position : -1, last_position);
    part_lo = part_hi;
  }

  // merge: set s is finished by wave s
#pragma unroll
  for (int s = 0; s < NSET; ++s) {
    __syncthreads();
    part[wave][0][lane] = acc.m[s];
    part[wave][1][lane] = acc.l[s];
#pragma unroll
    for (int dt = 0; dt < DV / 16; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) part[wave][2 + 4 * dt + i][lane] = acc.o[s][dt][i];
    __syncthreads();
    if (wave != s % LATENT_WAVES) continue;
    float m = -INFINITY;
#pragma unroll
    for (int w = 0; w < LATENT_WAVES; ++w) m = fmaxf(m, part[w][0][lane]);
    float factor[LATENT_WAVES];
    float l = 0.f;
#pragma unroll
    for (int w = 0; w < LATENT_WAVES; ++w) {
      const float m_w = part[w][0][lane];
      factor[w] = m_w == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_w - m);
      l += part[w][1][lane] * factor[w];
    }
    l += __shfl_xor(l, 16, WAVE);
    l += __shfl_xor(l, 32, WAVE);
    if (col_pos[s] < 0) continue;
    const float inverse = 1.f / l;
    bf16_t* o = out + (long)token * out_ld + (long)(head0 + s) * DV;
#pragma unroll
    for (int dt = 0; dt < DV / 16; ++dt) {
      mfma_bf16x4 packed;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float value = 0.f;
#pragma unroll
        for (int w = 0; w < LATENT_WAVES; ++w) value += part[w][2 + 4 * dt + i][lane] * factor[w];
        packed[i] = (bf16_t)(value * inverse);
      }
      *reinterpret_cast<mfma_bf16x4*>(o + 16 * dt + 4 * qd) = packed;
    }
  }
}

// The widths the kernel is built for: (latent, turned part).  most: how many heads share a fragment at most.
#define LATENT_SHAPES(CASE)                                                                                        \
  CASE(32, 32, 4, 4) CASE(64, 32, 4, 2) CASE(64, 64, 4, 2) CASE(96, 32, 2, 2) CASE(128, 32, 2, 1) CASE(128, 64, 2, 1) \
  CASE(192, 64, 1, 1)

extern "C" int mi_latent_attention_supported(int rank, int turned) {
#define SUPPORTED_CASE(RANK_, TURNED_, MOST_, STEPS_) \
  if (rank == RANK_ && turned == TURNED_) return 1;
  LATENT_SHAPES(SUPPORTED_CASE)
#undef SUPPORTED_CASE
  return 0;
}

template <int DK, int DV, int MOST, int STEPS>
static int launch_latent_attention(const bf16_t* q, long q_ld, int H, const bf16_t* k_base, const bf16_t* v_base,
                                   long page_stride, int page_size, const int* block_tables, int max_pages,
                                   const int* tiles, int n_tiles, const int* cu_seqlens, const int* start_pos, float scale,
                                   int window, bf16_t* out, long out_ld, hipStream_t stream) {
  const int passes = (H + MOST - 1) / MOST;
  const int per_pass = (H + passes - 1) / passes;
  const dim3 grid(4 * n_tiles, 1, passes);
#define LATENT_LAUNCH(NSET_)                                                                                       \
  latent_attention_kernel<DK, DV, NSET_, STEPS><<<grid, LATENT_WAVES * WAVE, 0, stream>>>(                         \
      q, q_ld, H, k_base, v_base, page_stride, page_size, block_tables, max_pages, tiles, cu_seqlens, start_pos, scale, \
      window, out, out_ld)
  if (MOST >= 4 && per_pass > 2) LATENT_LAUNCH(MOST >= 4 ? 4 : 1);
  else if (MOST >= 2 && per_pass > 1) LATENT_LAUNCH(MOST >= 2 ? 2 : 1);
  else LATENT_LAUNCH(1);
#undef LATENT_LAUNCH
  return 0;
}

// tiles: int32 [n_tiles, 2] = (lane, first token row) of runs of up to 64 tokens of one lane; the step's own keys
// must be in the cache already.  ERR_UNSUPPORTED_SIZE for widths the kernel is not built for.
extern "C" int mi_latent_attention(const void* q, long q_ld, int H, int rank, int turned, const void* k_base,
                                   const void* v_base, long page_stride, int page_size, const int* block_tables,
                                   int max_pages, const int* tiles, int n_tiles, const int* cu_seqlens,
                                   const int* start_pos, float scale, int window, void* out, long out_ld,
                                   hipStream_t stream) {
  if (!q || !k_base || !v_base || !block_tables || !tiles || !cu_seqlens || !start_pos || !out || n_tiles <= 0 || H <= 0 ||
      page_size <= 0 || max_pages <= 0)
    return ERR_BAD_ARGUMENT;
  if (page_size % 4 != 0 || q_ld % 8 != 0 || out_ld % 4 != 0 || ((unsigned long long)q % 16) != 0 ||
      ((unsigned long long)out % 8) != 0 || n_tiles > (1 << 28) || H > 65535 * 4)
    return ERR_UNSUPPORTED_SIZE;
#define LATENT_CASE(RANK_, TURNED_, MOST_, STEPS_)                                                                 \
  if (rank == RANK_ && turned == TURNED_) {                                                                        \
    launch_latent_attention<RANK_ + TURNED_, RANK_, MOST_, STEPS_>(                                                \
        (const bf16_t*)q, q_ld, H, (const bf16_t*)k_base, (const bf16_t*)v_base, page_stride, page_size, block_tables, \
        max_pages, tiles, n_tiles, cu_seqlens, start_pos, scale, window, (bf16_t*)out, out_ld, stream);            \
    RETURN_IF_LAUNCH_FAILED();                                                                                     \
    return 0;                                                                                                      \
  }
  LATENT_SHAPES(LATENT_CASE)
#undef LATENT_CASE
  return ERR_UNSUPPORTED_SIZE;
}

// ---------------------------------------------------------------- single decoded tokens, the context split
// For steps of single-token lanes in bfloat16: a wave takes one run of `split_keys` keys of one request and up to
// 16 heads, which are the columns of the matrix cores' products (all heads read the same cached rows, so a key or
// value fragment is fetched once for the sixteen); it leaves an unnormalized partial result with its maximum and
// normalizer (in units of log2), and a second kernel merges a token's runs in ascending order.  grid = (runs,
// tokens, sets of 16 heads), one wave a workgroup.
template <int DK, int DV, int STEPS>
__global__ void __launch_bounds__(WAVE)
latent_decode_kernel(const bf16_t* __restrict__ q, long q_ld, int H, const bf16_t* __restrict__ k_base,
                     const bf16_t* __restrict__ v_base, long page_stride, int page_size,
                     const int* __restrict__ block_tables, int max_pages, const int* __restrict__ lane_of_token,
                     const int* __restrict__ positions, float scale, int window, int split_keys, int splits,
                     float* __restrict__ partial_o, float* __restrict__ partial_ml) {
  const int split = blockIdx.x;
  const long token = blockIdx.y;
  const int head0 = blockIdx.z * 16;
  const int pos = positions[token];
  int first_key = 0;
  if (window > 0 && pos - window + 1 > 0) first_key = pos - window + 1;
  const int range_lo = (first_key / 32) * 32 + split * split_keys;
  if (range_lo > pos) return;                                 // the merge knows which runs hold keys
  const int range_hi = min(range_lo + split_keys, pos + 1);
  const int lane = threadIdx.x & (WAVE - 1);
  const int qd = lane / 16;
  const int n = lane % 16;
  const int head = head0 + n;
  const bool valid = head < H;
  mfma_bf16x8 q_frag[1][DK / 32];
  int col_pos[1] = {valid ? pos : -1};
#pragma unroll
  for (int kk = 0; kk < DK / 32; ++kk) {
    if (valid) {
      q_frag[0][kk] = *reinterpret_cast<const mfma_bf16x8*>(q + token * q_ld + (long)head * DK + 32 * kk + 8 * qd);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) q_frag[0][kk][j] = (bf16_t)0.f;
    }
  }
  AttnAccumulator<DK, 1, DV> acc;
  acc.clear();
  AttnCache cache;
  cache.k_base = k_base;
  cache.v_base = v_base;
  cache.page_stride = page_stride;
  cache.page_size = page_size;
  cache.kvh = 0;
  cache.pages = block_tables + (long)lane_of_token[token] * max_pages;
  cache.base_page = 0;
  attend_keys<DK, 1, STEPS, false, false, DV>(acc, q_frag, col_pos, window, scale, range_lo, range_hi, cache);
  const float l = attn_normalizer<DK, 1, DV>(acc, 0);
  if (!valid) return;
  const long at = (token * H + head) * splits + split;
  if (qd == 0) {
    partial_ml[2 * at] = acc.m[0];
    partial_ml[2 * at + 1] = l;
  }
#pragma unroll
  for (int dt = 0; dt < DV / 16; ++dt)
    *reinterpret_cast<mfma_floatx4*>(partial_o + at * DV + 16 * dt + 4 * qd) = acc.o[0][dt];
}

#define LATENT_MERGE_SPLITS 256

__global__ void latent_decode_merge_kernel(const float* __restrict__ partial_o, const float* __restrict__ partial_ml,
                                           const int* __restrict__ positions, int window, int split_keys, int splits,
                                           int H, int dv, bf16_t* __restrict__ out, long out_ld) {
  __shared__ float factor[LATENT_MERGE_SPLITS];      // exp2(maximum of the run - maximum), 0 for a run without keys
  __shared__ float scratch[16];
  const long token = blockIdx.x;
  const int head = blockIdx.y;
  const int pos = positions[token];
  int first_key = 0;
  if (window > 0 && pos - window + 1 > 0) first_key = pos - window + 1;
  const int used = min(splits, (pos - (first_key / 32) * 32) / split_keys + 1);
  const float* ml = partial_ml + (token * H + head) * splits * 2;
  const float* o = partial_o + (token * H + head) * (long)splits * dv;
  float maximum = -INFINITY;
  for (int s = threadIdx.x; s < used; s += blockDim.x) maximum = fmaxf(maximum, ml[2 * s]);
  maximum = wave_max(maximum);
  __syncthreads();
  if ((threadIdx.x & (WAVE - 1)) == 0) scratch[threadIdx.x / WAVE] = maximum;
  __syncthreads();
  for (int w = 0; w < (int)(blockDim.x + WAVE - 1) / WAVE; ++w) maximum = fmaxf(maximum, scratch[w]);
  float share = 0.f;
  for (int s = threadIdx.x; s < used; s += blockDim.x) {
    const float f = ml[2 * s] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ml[2 * s] - maximum);
    factor[s] = f;
    share += f * ml[2 * s + 1];
  }
  const float denominator = block_sum(share, scratch);           // (its barriers also publish the factors)
  for (int dim = threadIdx.x; dim < dv; dim += blockDim.x) {
    float sum = 0.f;
    for (int s = 0; s < used; ++s) sum = fmaf(factor[s], o[(long)s * dv + dim], sum);
    out[token * out_ld + (long)head * dv + dim] = (bf16_t)(sum / denominator);
  }
}

// partial_o: float32 [T, H, splits, rank]; partial_ml: float32 [T, H, splits, 2].  split_keys: a multiple of 32.
extern "C" int mi_latent_decode_attention(const void* q, long q_ld, int T, int H, int rank, int turned, const void* k_base,
                                          const void* v_base, long page_stride, int page_size, const int* block_tables,
                                          int max_pages, const int* lane_of_token, const int* positions, float scale,
                                          int window, int split_keys, int splits, float* partial_o, float* partial_ml,
                                          void* out, long out_ld, hipStream_t stream) {
  if (!q || !k_base || !v_base || !block_tables || !lane_of_token || !positions || !partial_o || !partial_ml || !out ||
      T <= 0 || H <= 0 || page_size <= 0 || max_pages <= 0 || splits <= 0 || split_keys <= 0)
    return ERR_BAD_ARGUMENT;
  if (page_size % 4 != 0 || q_ld % 8 != 0 || ((unsigned long long)q % 16) != 0 || split_keys % 32 != 0 || T > 65535 ||
      (H + 15) / 16 > 65535 || H > 65535 || splits > LATENT_MERGE_SPLITS)
    return ERR_UNSUPPORTED_SIZE;
  const dim3 grid(splits, T, (H + 15) / 16);
#define LATENT_DECODE_CASE(RANK_, TURNED_, MOST_, STEPS_)                                                          \
  if (rank == RANK_ && turned == TURNED_) {                                                                        \
    latent_decode_kernel<RANK_ + TURNED_, RANK_, (RANK_ + TURNED_ <= 128 ? 2 : 1)><<<grid, WAVE, 0, stream>>>(     \
        (const bf16_t*)q, q_ld, H, (const bf16_t*)k_base, (const bf16_t*)v_base, page_stride, page_size, block_tables, \
        max_pages, lane_of_token, positions, scale, window, split_keys, splits, partial_o, partial_ml);            \
    RETURN_IF_LAUNCH_FAILED();                                                                                     \
    latent_decode_merge_kernel<<<dim3(T, H), RANK_ <= 64 ? 64 : 128, 0, stream>>>(                                 \
        partial_o, partial_ml, positions, window, split_keys, splits, H, RANK_, (bf16_t*)out, out_ld);             \
    RETURN_IF_LAUNCH_FAILED();                                                                                     \
    return 0;                                                                                                      \
  }
  LATENT_SHAPES(LATENT_DECODE_CASE)
#undef LATENT_DECODE_CASE
  return ERR_UNSUPPORTED_SIZE;
}
