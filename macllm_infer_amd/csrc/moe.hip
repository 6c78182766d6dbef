// A feed-forward of many small experts of which a token uses a few.
//
//   moe_route        float32 router logits -> softmax, correction, the token's experts and their weights (one wave
//                    a token), and the sigmoid of the shared expert's gate logit; or (mode 1) logits + bias -> the
//                    largest ones and the softmax over those alone
//   moe_plan         the step's (token, choice) rows grouped by expert, every expert's rows starting a tile of 16
//                    places: built on the device by one workgroup, so that no count has to travel to the host and
//                    the launches that follow depend on the number of tokens alone
//   moe_expert_gemm  the grouped product on the matrix cores: a tile's rows (gathered from the tokens' rows, or
//                    the places themselves) with its expert's matrix; epilogue: plain, or the clamped gated
//                    activation of a gate tile and an up tile
//   moe_combine      a token's weighted sum over its choices, in their order, plus the gated shared expert
//
// A row of a tile is summed on its own (a column of the matrix cores' result), so a token's numbers do not depend
// on which other rows share its tile or on the place it was given.
#include "mfma_tile.h"

#define MOE_MAX_EXPERTS 1024
#define MOE_PER_LANE (MOE_MAX_EXPERTS / WAVE)

// ---------------------------------------------------------------- router
__global__ void __launch_bounds__(256)
moe_route_kernel(const float* __restrict__ logits, long ld, int T, int E, int top, const float* __restrict__ correction,
                 float scale, float eps, int mode, int* __restrict__ chosen, float* __restrict__ weights,
                 float* __restrict__ gate) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int token = blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  if (token >= T) return;
  const float* row = logits + (long)token * ld;
  float score[MOE_PER_LANE], choice[MOE_PER_LANE];
  const int held = (E + WAVE - 1) / WAVE;          // experts a lane holds: the loops below end there (the same in every lane)
  float most = -INFINITY;
#pragma unroll
  for (int j = 0; j < MOE_PER_LANE; ++j) {
    if (j >= held) break;
    const int e = lane + WAVE * j;
    score[j] = e < E ? row[e] : -INFINITY;
    most = fmaxf(most, score[j]);
  }
  if (mode == 0) {
    most = wave_max(most);
    float total = 0.f;
#pragma unroll
    for (int j = 0; j < MOE_PER_LANE; ++j) {
      if (j >= held) break;
      const int e = lane + WAVE * j;
      score[j] = e < E ? expf(score[j] - most) : 0.f;
      total += score[j];
    }
    total = wave_sum(total);
#pragma unroll
    for (int j = 0; j < MOE_PER_LANE; ++j) {
      if (j >= held) break;
      const int e = lane + WAVE * j;
      score[j] = score[j] / total;
      choice[j] = e < E ? score[j] + correction[e] : -INFINITY;
    }
  } else {
    // the logits with their bias are what is chosen by and what is weighted
#pragma unroll
    for (int j = 0; j < MOE_PER_LANE; ++j) {
      if (j >= held) break;
      const int e = lane + WAVE * j;
      score[j] = e < E ? score[j] + correction[e] : -INFINITY;
      choice[j] = score[j];
    }
  }
  float first_picked = 0.f;        // mode 1: the largest chosen logit, which is the first one picked
  float picked_sum = 0.f;
  float mine = 0.f;            // lane k keeps the score of the k-th choice
  int mine_id = 0;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY, best_score = 0.f;
    int best_id = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < MOE_PER_LANE; ++j) {
      if (j >= held) break;
      const int e = lane + WAVE * j;
      if (e < E && (choice[j] > best || (choice[j] == best && e < best_id))) {
        best = choice[j];
        best_id = e;
        best_score = score[j];
      }
    }
#pragma unroll
    for (int offset = WAVE / 2; offset > 0; offset >>= 1) {
      const float other = __shfl_xor(best, offset, WAVE);
      const int other_id = __shfl_xor(best_id, offset, WAVE);
      const float other_score = __shfl_xor(best_score, offset, WAVE);
      if (other > best || (other == best && other_id < best_id)) {
        best = other;
        best_id = other_id;
        best_score = other_score;
      }
    }
#pragma unroll
    for (int j = 0; j < MOE_PER_LANE; ++j)
      if (j < held && lane + WAVE * j == best_id) choice[j] = -INFINITY;
    if (mode != 0) {
      if (k == 0) first_picked = best_score;
      best_score = expf(best_score - first_picked);
    }
    picked_sum += best_score;
    if ((k & (WAVE - 1)) == lane) {
      // more choices than lanes: written as they come
      mine = best_score;
      mine_id = best_id;
    }
    if (top > WAVE && lane == 0) {
      chosen[(long)token * top + k] = best_id;
      weights[(long)token * top + k] = best_score;      // divided below
    }
  }
  const float denominator = picked_sum + eps;
  if (top <= WAVE) {
    if (lane < top) {
      chosen[(long)token * top + lane] = mine_id;
      weights[(long)token * top + lane] = mine / denominator * scale;
    }
  } else if (lane == 0) {
    for (int k = 0; k < top; ++k) weights[(long)token * top + k] = weights[(long)token * top + k] / denominator * scale;
  }
  if (gate && lane == 0) gate[token] = 1.0f / (1.0f + expf(-row[E]));
}

// mode 0: softmax over all experts, choice by score + correction, weights score / (sum of the chosen + eps) * scale.
// mode 1: choice by logit + correction (a bias), weights the softmax over the chosen (logit + correction) * scale.
extern "C" int mi_moe_route(const float* logits, long ld, int T, int E, int top, const float* correction, float scale,
                            float eps, int mode, int* chosen, float* weights, float* gate, hipStream_t stream) {
  if (!logits || !correction || !chosen || !weights || T <= 0 || E <= 0 || top <= 0 || top > E || ld < E + (gate ? 1 : 0))
    return ERR_BAD_ARGUMENT;
  if (E > MOE_MAX_EXPERTS) return ERR_UNSUPPORTED_SIZE;
  if (mode != 0 && mode != 1) return ERR_BAD_ARGUMENT;
  moe_route_kernel<<<(T + 3) / 4, 256, 0, stream>>>(logits, ld, T, E, top, correction, scale, eps, mode, chosen, weights, gate);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- rows grouped by expert
__global__ void __launch_bounds__(1024)
moe_plan_kernel(const int* __restrict__ chosen, int entries, int top, int E, int pad, int capacity,
                int* __restrict__ source, int* __restrict__ place, int* __restrict__ tile_expert, int* __restrict__ ranks) {
  __shared__ int counts[MOE_MAX_EXPERTS];
  __shared__ int offsets[MOE_MAX_EXPERTS];
  const int tid = threadIdx.x;
  const int threads = blockDim.x;
  for (int e = tid; e < E; e += threads) counts[e] = 0;
  for (int i = tid; i < capacity; i += threads) source[i] = -1;
  for (int t = tid; t < capacity / pad; t += threads) tile_expert[t] = -1;
  __syncthreads();
  for (int i = tid; i < entries; i += threads) ranks[i] = atomicAdd(&counts[chosen[i]], 1);
  __syncthreads();
  if (tid == 0) {
    int running = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = running;
      running += (counts[e] + pad - 1) / pad * pad;
    }
  }
  __syncthreads();
  for (int e = tid; e < E; e += threads) {
    const int first = offsets[e] / pad;
    const int tiles = (counts[e] + pad - 1) / pad;
    for (int t = 0; t < tiles; ++t) tile_expert[first + t] = e;
  }
  for (int i = tid; i < entries; i += threads) {
    const int at = offsets[chosen[i]] + ranks[i];
    source[at] = i / top;
    place[i] = at;
  }
}

extern "C" int mi_moe_plan(const int* chosen, int entries, int top, int E, int pad, int capacity, int* source, int* place,
                           int* tile_expert, int* ranks, hipStream_t stream) {
  if (!chosen || !source || !place || !tile_expert || !ranks || entries <= 0 || top <= 0 || E <= 0 || pad <= 0 ||
      capacity % pad != 0 || capacity < entries + E * (pad - 1))
    return ERR_BAD_ARGUMENT;
  if (E > MOE_MAX_EXPERTS) return ERR_UNSUPPORTED_SIZE;
  moe_plan_kernel<<<1, 1024, 0, stream>>>(chosen, entries, top, E, pad, capacity, source, place, tile_expert, ranks);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- the grouped product
// Tile t of 16 MT places belongs to expert tile_expert[t] (none: the workgroup leaves).  A workgroup owns the
// tile's rows and PAIRS tiles of 16 output features.  GLU: the expert's matrix is [2 I, K], gate rows then up
// rows; out[place, n] = act(gate tile, up tile), n < I.  Places without a row get zeros.  Steps of few rows take
// MT = 1 (every expert's matrix is read once, by as many workgroups as it has tiles of features); prompt portions,
// whose experts get dozens of rows each, MT = 4 and four tiles of features (the rows and the matrix come from the
// caches, 64 x 64 results a workgroup).
template <typename T, typename TO, bool VEC, bool GLU, int MT, int PAIRS>
__global__ void __launch_bounds__(TILE_THREADS)
moe_expert_gemm_kernel(const T* __restrict__ x, long ldx, int x_rows, const T* __restrict__ W, long expert_stride, long ldw,
                       int N, int K, const int* __restrict__ source, const int* __restrict__ tile_expert, int gather,
                       float limit, float alpha, float offset, int squared_relu, TO* __restrict__ out, long ldo) {
  __shared__ float red[TILE_WAVES][256];
  const int tile = blockIdx.y;
  const int expert = tile_expert[tile];
  if (expert < 0) return;
  const int tid = threadIdx.x;
  const int r = (tid & (WAVE - 1)) % 16;
  const int width = GLU ? N / 2 : N;
  const long n0 = (long)blockIdx.x * 16 * PAIRS;
  const T* matrix = W + (long)expert * expert_stride;
  constexpr int NT = GLU ? 2 * PAIRS : PAIRS;
  const T* w_row[NT];
  const T* x_row[MT];
#pragma unroll
  for (int p = 0; p < PAIRS; ++p) {
    const long n_row = min(n0 + 16 * p + r, (long)width - 1);
    w_row[p] = matrix + n_row * ldw;
    if (GLU) w_row[NT - PAIRS + p] = matrix + (width + n_row) * ldw;
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int place_in = (tile * MT + mt) * 16 + r;
    const long x_at = gather ? max(source[place_in], 0) : place_in;
    x_row[mt] = x + min(x_at, (long)x_rows - 1) * ldx;
  }
  tile_floatx4 acc[NT][MT];
  tile_accumulate<T, MT, NT, VEC>(w_row, x_row, K, acc);
  const int l = tid % 64;
#pragma unroll
  for (int p = 0; p < PAIRS; ++p)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float value = tile_reduce(acc[p][mt], red);
      if (GLU) {
        const float up = tile_reduce(acc[NT - PAIRS + p][mt], red);
        const float g = fminf(value, limit);
        const float u = fminf(fmaxf(up, -limit), limit);
        value = g / (1.0f + expf(-alpha * g)) * (u + offset);
      } else if (squared_relu) {
        value = fmaxf(value, 0.f);
        value *= value;
      }
      const long n = n0 + 16 * p + 4 * (l / 16) + tid / 64;
      const int place = (tile * MT + mt) * 16 + (l % 16);
      if (n < width) out[(long)place * ldo + n] = from_float<TO>(source[place] >= 0 ? value : 0.f);
    }
}

// Where piece `piece` (0..3) of row `row` of an LDS stage lies: a row is 64 bytes, and the pieces of rows 4 apart
// are swapped among themselves so that the sixteen rows a quarter of a wave reads at once fall into sixteen
// different groups of banks.
__device__ __forceinline__ int stage_slot(int row, int piece) { return row * 4 + (piece ^ ((row >> 2) & 3)); }

// The same product for prompt portions whose rows and matrices are whole 16-byte pieces: a workgroup owns a tile
// of 64 places and 128 rows of its expert's matrix (GLU: 64 gate rows and the 64 up rows that go with them, which
// make 64 outputs; else 128 outputs), walks K one chunk at a time through two LDS stages (the next chunk's pieces
// are asked for before the current one's products), and every wave owns all 64 places and a quarter of the
// features: no sum crosses a wave, a row's result is summed in k order by one lane's accumulator.
template <typename T, typename TO, bool GLU>
__global__ void __launch_bounds__(TILE_THREADS)
moe_expert_gemm_wide_kernel(const T* __restrict__ x, long ldx, int x_rows, const T* __restrict__ W, long expert_stride,
                            long ldw, int N, int K, const int* __restrict__ source, const int* __restrict__ tile_expert,
                            int gather, float limit, float alpha, float offset, int squared_relu, TO* __restrict__ out,
                            long ldo) {
  typedef typename TileTraits<T>::Piece Piece;
  constexpr int CHUNK = TileTraits<T>::CHUNK;
  constexpr int PIECE = TileTraits<T>::PIECE;
  constexpr int ROWS = 64, FEATURES = 128;
  __shared__ Piece stage[2][(ROWS + FEATURES) * 4];
  const int tile = blockIdx.y;
  const int expert = tile_expert[tile];
  if (expert < 0) return;
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;
  const int q = lane / 16;
  const int r = lane % 16;
  const int width = GLU ? N / 2 : N;
  const long n0 = (long)blockIdx.x * (GLU ? 64 : 128);
  const T* matrix = W + (long)expert * expert_stride;
  // what this thread brings into a stage: piece `part` of one row of x and of two rows of the matrix
  const int lrow = tid / 4;
  const int part = tid % 4;
  const int place_in = tile * ROWS + lrow;
  const long x_at = gather ? max(source[place_in], 0) : place_in;
  const T* x_from = x + min(x_at, (long)x_rows - 1) * ldx;
  const T* w_from[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int s = lrow + 64 * j;                                // row of the stage's matrix part
    long feature;
    if (GLU) feature = (j == 0 ? 0 : width) + min(n0 + lrow, (long)width - 1);
    else feature = min(n0 + s, (long)width - 1);
    w_from[j] = matrix + feature * ldw;
  }
  tile_floatx4 acc[2][4];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) acc[nt][mt] = tile_floatx4{0.f, 0.f, 0.f, 0.f};
  const int chunks = (K + CHUNK - 1) / CHUNK;
  Piece gx = tile_load<T, true>(x_from, PIECE * part, K);
  Piece gw0 = tile_load<T, true>(w_from[0], PIECE * part, K);
  Piece gw1 = tile_load<T, true>(w_from[1], PIECE * part, K);
  stage[0][stage_slot(lrow, part)] = gx;
  stage[0][stage_slot(ROWS + lrow, part)] = gw0;
  stage[0][stage_slot(ROWS + 64 + lrow, part)] = gw1;
  __syncthreads();
  for (int c = 0; c < chunks; ++c) {
    const int cur = c & 1;
    const int k_next = c + 1 < chunks ? (c + 1) * CHUNK + PIECE * part : K;      // past the end: zeros, never used
    gx = tile_load<T, true>(x_from, k_next, K);
    gw0 = tile_load<T, true>(w_from[0], k_next, K);
    gw1 = tile_load<T, true>(w_from[1], k_next, K);
    Piece a[2], b[4];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const int row = GLU ? 64 * nt + 16 * wave + r : 32 * wave + 16 * nt + r;
      a[nt] = stage[cur][stage_slot(ROWS + row, q)];
    }
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) b[mt] = stage[cur][stage_slot(16 * mt + r, q)];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) acc[nt][mt] = tile_mfma(a[nt], b[mt], acc[nt][mt]);
    stage[cur ^ 1][stage_slot(lrow, part)] = gx;
    stage[cur ^ 1][stage_slot(ROWS + lrow, part)] = gw0;
    stage[cur ^ 1][stage_slot(ROWS + 64 + lrow, part)] = gw1;
    __syncthreads();
  }
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
    const int place = tile * ROWS + 16 * mt + r;
    const bool live = source[place] >= 0;
    TO* row = out + (long)place * ldo;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (GLU) {
        const long n = n0 + 16 * wave + 4 * q + i;
        const float g = fminf(acc[0][mt][i], limit);
        const float u = fminf(fmaxf(acc[1][mt][i], -limit), limit);
        const float value = g / (1.0f + expf(-alpha * g)) * (u + offset);
        if (n < width) row[n] = from_float<TO>(live ? value : 0.f);
      } else {
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
          const long n = n0 + 32 * wave + 16 * nt + 4 * q + i;
          float value = acc[nt][mt][i];
          if (squared_relu) {
            value = fmaxf(value, 0.f);
            value *= value;
          }
          if (n < width) row[n] = from_float<TO>(live ? value : 0.f);
        }
      }
    }
  }
}

// The widest form, for prompt portions whose experts get hundreds of rows each: 128 places x 128 matrix rows a
// workgroup, every wave a quarter of it as 64 places x 64 matrix rows (GLU: 32 gate rows and their 32 up rows), so
// that eight fragments from LDS feed sixteen matrix instructions.
template <typename T, typename TO, bool GLU>
__global__ void __launch_bounds__(TILE_THREADS)
moe_expert_gemm_widest_kernel(const T* __restrict__ x, long ldx, int x_rows, const T* __restrict__ W, long expert_stride,
                              long ldw, int N, int K, const int* __restrict__ source, const int* __restrict__ tile_expert,
                              int gather, float limit, float alpha, float offset, int squared_relu, TO* __restrict__ out,
                              long ldo) {
  typedef typename TileTraits<T>::Piece Piece;
  constexpr int CHUNK = TileTraits<T>::CHUNK;
  constexpr int PIECE = TileTraits<T>::PIECE;
  constexpr int ROWS = 128, FEATURES = 128;
  __shared__ Piece stage[2][(ROWS + FEATURES) * 4];
  const int tile = blockIdx.y;
  const int expert = tile_expert[tile];
  if (expert < 0) return;
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;
  const int wm = wave / 2;                                     // which 64 places
  const int wn = wave % 2;                                     // which half of the features
  const int q = lane / 16;
  const int r = lane % 16;
  const int width = GLU ? N / 2 : N;
  const long n0 = (long)blockIdx.x * (GLU ? 64 : 128);
  const T* matrix = W + (long)expert * expert_stride;
  const int lrow = tid / 4;
  const int part = tid % 4;
  const T* x_from[2];
  const T* w_from[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int place_in = tile * ROWS + lrow + 64 * j;
    const long x_at = gather ? max(source[place_in], 0) : place_in;
    x_from[j] = x + min(x_at, (long)x_rows - 1) * ldx;
    long feature;
    if (GLU) feature = (j == 0 ? 0 : width) + min(n0 + lrow, (long)width - 1);
    else feature = min(n0 + lrow + 64 * j, (long)width - 1);
    w_from[j] = matrix + feature * ldw;
  }
  tile_floatx4 acc[4][4];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) acc[nt][mt] = tile_floatx4{0.f, 0.f, 0.f, 0.f};
  const int chunks = (K + CHUNK - 1) / CHUNK;
  Piece gx[2], gw[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    gx[j] = tile_load<T, true>(x_from[j], PIECE * part, K);
    gw[j] = tile_load<T, true>(w_from[j], PIECE * part, K);
    stage[0][stage_slot(lrow + 64 * j, part)] = gx[j];
    stage[0][stage_slot(ROWS + lrow + 64 * j, part)] = gw[j];
  }
  __syncthreads();
  for (int c = 0; c < chunks; ++c) {
    const int cur = c & 1;
    const int k_next = c + 1 < chunks ? (c + 1) * CHUNK + PIECE * part : K;      // past the end: zeros, never used
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      gx[j] = tile_load<T, true>(x_from[j], k_next, K);
      gw[j] = tile_load<T, true>(w_from[j], k_next, K);
    }
    Piece a[4], b[4];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      // GLU: nt 0, 1 are gate rows, nt 2, 3 the up rows of the same outputs (the stage's second 64 rows)
      const int row = GLU ? 64 * (nt / 2) + 32 * wn + 16 * (nt % 2) + r : 64 * wn + 16 * nt + r;
      a[nt] = stage[cur][stage_slot(ROWS + row, q)];
    }
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) b[mt] = stage[cur][stage_slot(64 * wm + 16 * mt + r, q)];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) acc[nt][mt] = tile_mfma(a[nt], b[mt], acc[nt][mt]);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      stage[cur ^ 1][stage_slot(lrow + 64 * j, part)] = gx[j];
      stage[cur ^ 1][stage_slot(ROWS + lrow + 64 * j, part)] = gw[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
    const int place = tile * ROWS + 64 * wm + 16 * mt + r;
    const bool live = source[place] >= 0;
    TO* row = out + (long)place * ldo;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (GLU) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const long n = n0 + 32 * wn + 16 * h + 4 * q + i;
          const float g = fminf(acc[h][mt][i], limit);
          const float u = fminf(fmaxf(acc[2 + h][mt][i], -limit), limit);
          const float value = g / (1.0f + expf(-alpha * g)) * (u + offset);
          if (n < width) row[n] = from_float<TO>(live ? value : 0.f);
        }
      } else {
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) {
          const long n = n0 + 64 * wn + 16 * nt + 4 * q + i;
          float value = acc[nt][mt][i];
          if (squared_relu) {
            value = fmaxf(value, 0.f);
            value *= value;
          }
          if (n < width) row[n] = from_float<TO>(live ? value : 0.f);
        }
      }
    }
  }
}

template <typename T, typename TO>
static void launch_expert_gemm(const T* x, long ldx, int x_rows, const T* W, long expert_stride, long ldw, int N, int K,
                               const int* source, const int* tile_expert, int tiles, int pad, int gather, int activation,
                               float limit, float alpha, float offset, TO* out, long ldo, hipStream_t stream) {
  const int glu = activation == 1;
  const int squared_relu = activation == 2;
  constexpr int PIECE = TileTraits<T>::PIECE;
  const bool vec = K % PIECE == 0 && ldx % PIECE == 0 && ldw % PIECE == 0 && expert_stride % PIECE == 0 &&
                   ((unsigned long long)x % 16) == 0 && ((unsigned long long)W % 16) == 0;
  const int width = glu ? N / 2 : N;
#define EXPERT_LAUNCH(VEC_, GLU_, MT_, PAIRS_)                                                                           moe_expert_gemm_kernel<T, TO, VEC_, GLU_, MT_, PAIRS_>                                                                    <<<dim3((unsigned)((width + 16 * PAIRS_ - 1) / (16 * PAIRS_)), (unsigned)tiles), TILE_THREADS, 0, stream>>>(               x, ldx, x_rows, W, expert_stride, ldw, N, K, source, tile_expert, gather, limit, alpha, offset, squared_relu, out, ldo)
#define EXPERT_SHAPE(MT_, PAIRS_GLU_, PAIRS_PLAIN_)                                                                      do {                                                                                                                    if (vec && glu) EXPERT_LAUNCH(true, true, MT_, PAIRS_GLU_);                                                            else if (vec) EXPERT_LAUNCH(true, false, MT_, PAIRS_PLAIN_);                                                           else if (glu) EXPERT_LAUNCH(false, true, MT_, PAIRS_GLU_);                                                             else EXPERT_LAUNCH(false, false, MT_, PAIRS_PLAIN_);                                                                 } while (0)
  if (pad == 128) {      // (only plans of rows and matrices in whole pieces are made so wide)
    const dim3 grid((unsigned)((width + (glu ? 64 : 128) - 1) / (glu ? 64 : 128)), (unsigned)tiles);
    if (glu)
      moe_expert_gemm_widest_kernel<T, TO, true><<<grid, TILE_THREADS, 0, stream>>>(
          x, ldx, x_rows, W, expert_stride, ldw, N, K, source, tile_expert, gather, limit, alpha, offset, squared_relu, out, ldo);
    else
      moe_expert_gemm_widest_kernel<T, TO, false><<<grid, TILE_THREADS, 0, stream>>>(
          x, ldx, x_rows, W, expert_stride, ldw, N, K, source, tile_expert, gather, limit, alpha, offset, squared_relu, out, ldo);
  } else if (pad == 64 && vec) {
    const dim3 grid((unsigned)((width + (glu ? 64 : 128) - 1) / (glu ? 64 : 128)), (unsigned)tiles);
    if (glu)
      moe_expert_gemm_wide_kernel<T, TO, true><<<grid, TILE_THREADS, 0, stream>>>(
          x, ldx, x_rows, W, expert_stride, ldw, N, K, source, tile_expert, gather, limit, alpha, offset, squared_relu, out, ldo);
    else
      moe_expert_gemm_wide_kernel<T, TO, false><<<grid, TILE_THREADS, 0, stream>>>(
          x, ldx, x_rows, W, expert_stride, ldw, N, K, source, tile_expert, gather, limit, alpha, offset, squared_relu, out, ldo);
  } else if (pad == 64) {
    EXPERT_SHAPE(4, 2, 4);
  } else {
    EXPERT_SHAPE(1, 1, 1);
  }
#undef EXPERT_SHAPE
#undef EXPERT_LAUNCH
}

extern "C" int mi_moe_expert_gemm(const void* x, int dtype, long ldx, int x_rows, const void* W, long expert_stride,
                                  long ldw, int N, int K, const int* source, const int* tile_expert, int tiles, int pad,
                                  int gather, int activation, float limit, float alpha, float offset, void* out,
                                  int out_dtype, long ldo, hipStream_t stream) {
  // activation: 0 none, 1 the clamped gated one (the matrix holds gate rows then up rows), 2 max(z, 0)^2
  const int glu = activation == 1;
  if (activation < 0 || activation > 2) return ERR_BAD_ARGUMENT;
  if (!x || !W || !source || !tile_expert || !out || x_rows <= 0 || N <= 0 || K <= 0 || tiles <= 0 || ldx < K || ldw < K ||
      (glu && N % 2) || ldo < (glu ? N / 2 : N))
    return ERR_BAD_ARGUMENT;
  if ((pad != 16 && pad != 64 && pad != 128) || tiles > 65535) return ERR_UNSUPPORTED_SIZE;
  if (pad == 128) {
    const long piece = dtype == DT_F32 ? 4 : 8;
    if (K % piece || ldx % piece || ldw % piece || expert_stride % piece || ((unsigned long long)x % 16) ||
        ((unsigned long long)W % 16))
      return ERR_UNSUPPORTED_SIZE;
  }
  if (dtype == DT_F32 && out_dtype == DT_F32)
    launch_expert_gemm<float, float>((const float*)x, ldx, x_rows, (const float*)W, expert_stride, ldw, N, K, source,
                                     tile_expert, tiles, pad, gather, activation, limit, alpha, offset, (float*)out, ldo, stream);
  else if (dtype == DT_BF16 && out_dtype == DT_BF16)
    launch_expert_gemm<bf16_t, bf16_t>((const bf16_t*)x, ldx, x_rows, (const bf16_t*)W, expert_stride, ldw, N, K, source,
                                       tile_expert, tiles, pad, gather, activation, limit, alpha, offset, (bf16_t*)out, ldo, stream);
  else if (dtype == DT_BF16 && out_dtype == DT_F32)
    launch_expert_gemm<bf16_t, float>((const bf16_t*)x, ldx, x_rows, (const bf16_t*)W, expert_stride, ldw, N, K, source,
                                      tile_expert, tiles, pad, gather, activation, limit, alpha, offset, (float*)out, ldo, stream);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- a token's weighted sum
template <typename TS>
__global__ void moe_combine_kernel(const float* __restrict__ down, long ld, const int* __restrict__ place,
                                   const float* __restrict__ weights, int top, const TS* __restrict__ shared, long shared_ld,
                                   const float* __restrict__ gate, float* __restrict__ out, int d) {
  const long token = blockIdx.x;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < d; i += gridDim.y * blockDim.x) {
    float total = 0.f;
    for (int k = 0; k < top; ++k)
      total = fmaf(weights[token * top + k], down[(long)place[token * top + k] * ld + i], total);
    if (shared) total = fmaf(gate[token], to_float(shared[token * shared_ld + i]), total);
    out[token * d + i] = total;
  }
}

extern "C" int mi_moe_combine(const float* down, long ld, const int* place, const float* weights, int top,
                              const void* shared, int shared_dtype, long shared_ld, const float* gate, float* out, int T,
                              int d, hipStream_t stream) {
  if (!down || !place || !weights || !out || T <= 0 || d <= 0 || top <= 0 || ld < d || (shared && (!gate || shared_ld < d)))
    return ERR_BAD_ARGUMENT;
  // a step of few tokens spreads a token's features over several workgroups
  const dim3 grid((unsigned)T, (unsigned)(T >= 256 ? 1 : min((d + 255) / 256, 16)));
  if (shared_dtype == DT_F32)
    moe_combine_kernel<float><<<grid, 256, 0, stream>>>(down, ld, place, weights, top, (const float*)shared, shared_ld, gate, out, d);
  else if (shared_dtype == DT_BF16)
    moe_combine_kernel<bf16_t><<<grid, 256, 0, stream>>>(down, ld, place, weights, top, (const bf16_t*)shared, shared_ld, gate, out, d);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}
