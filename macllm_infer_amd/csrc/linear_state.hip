// Mixers that carry a matrix-valued state per head: the scan of linear attention with a decay, in two forms,
// and what follows it.
//
//   retention        S <- decay[h] * S + k v^T                         o = S^T q
//   delta rule       S <- diag(w) S - (a * u)(u^T S) + k v^T           o = S^T r      (both products on the old S)
//   gated decay      S <- diag(w) S + k v^T                            o = S^T q      (w a gate of the token)
//
// with S [dk, dv] per head in float32, carried from token to token in the request's state slot.  What enters the
// recurrence is formed in float32 from the projection's rows inside the scan:
//   retention : q and k turned by position (half-split rotation of the first rotary_dim dims, angle =
//               (float)position * inv_freq[j]), then k * key_scale;
//   delta rule: u = k / sqrt(sum k^2 + key_eps), a = sigmoid(removal columns),
//               w = exp(-decay_floor * sigmoid(decay_logits + decay_bias));
//   gated decay: w = sigmoid(decay_logits + decay_bias)^gate_power = exp(gate_power * log sigmoid(.)) per head and
//               key channel, q * query_scale.
//
// The state is stored transposed, [slot][head][dv][dk]: a column of S (all key channels of one value channel)
// evolves on its own,
//   s_j <- w * s_j - (a * u) (u . s_j) + k v_j,    o_j = s_j . q,
// so a column is the unit of work: R neighbouring lanes own one column, each LS_PER_LANE-or-fewer consecutive key
// channels of it in registers, and the two dot products are added over the R lanes with shuffles.  A workgroup
// takes (lane of the step, head, a run of columns) and walks the lane's tokens in order; the per-token vectors
// (q, k, and for the delta rule w, u, a*u) are laid in LDS for a stage of tokens at a time by the waves of the
// workgroup, one token a wave at a time, and read from there by every column.  R and the order of every sum depend
// on dk alone.
//
// Long portions run in three passes over chunks of the lanes (a table of (lane, first row, tokens, index in the
// lane) that the step carries), so that the tokens of one prompt are worked on side by side:
//   local   every chunk but a lane's last, from an empty state: the state B the chunk's own tokens leave, and for
//           the delta rule the chunk's transition P = A_last ... A_first (A_t = diag(w_t) - (a_t u_t) u_t^T), whose
//           column i is what the same recurrence without keys makes of the unit vector e_i: dk more columns; for
//           the gated decay the transition is diagonal, the product of the chunk's w, which is what the recurrence
//           without keys makes of the vector of ones: one more column;
//   carry   per lane, chunk after chunk: S_start(c + 1) = P_c S_start(c) + B_c (retention: P_c = decay^tokens),
//           beginning with the request's state; every chunk's starting state is kept;
//   scan    every chunk from its starting state: the outputs, and behind a lane's last chunk the state of the request.
// All of it in float32: the passes add the same products in another order.
#include "common.h"
#include <cstdint>

#define LS_MAX_PER_LANE 16          // key channels of a column that one lane keeps
#define LS_THREADS 256
#define LS_PASS_THREADS 1024        // a workgroup of the passes over chunks: its many waves hide each other's waits
#define LS_PASS_LANES 16            // lanes a column there, when the head is wide enough (4 key channels a lane or more)
#define LS_STAGE_MOST 16            // tokens of a stage
#define LS_STAGE_BYTES (48 * 1024)

struct ScanArgs {
  const void* u;                    // the projection's rows [T, ld]
  long ld;
  int q_col, k_col, v_col, removal_col;
  int H, dk, dv;
  float* state;                     // [slots, H, dv, dk]
  const int* cu_seqlens;            // [lanes + 1]
  const int* slot_ids;              // [lanes]
  float* out;                       // [T, out_ld] float32, head h at columns h*dv
  long out_ld;
  const float* head_decay;          // retention: [H]
  float key_scale;
  const int* positions;             // [T]
  const float* inv_freq;            // [rotary_dim / 2] or null
  int rotary_dim;
  const float* decay_logits;        // delta rule: float32 [T, logits_ld], head h at columns h*dk
  long logits_ld;
  const float* decay_bias;          // [H * dk]
  float decay_floor, key_eps;
  float gate_power, query_scale;    // gated decay: the gate's exponent; what q is multiplied by (every kind)
  int R, per_lane, columns, stage;  // lanes a column, key channels a lane, columns a workgroup, tokens a stage
  const int* chunks;                // passes over chunks: [chunks, 4] = (lane, first row, tokens, index in the lane)
  const int* lane_chunks;           // [lanes, 2] = (first chunk, chunks)
  float* local;                     // [chunks, H, dv (+ dk), dk]: what the local pass leaves
  float* start;                     // [chunks, H, dv, dk]: every chunk's starting state
  int whole_fours;                  // dk a multiple of 4 and the state tables 16-byte aligned: states move 4 floats a load
};

#define LS_RETENTION 0              // the kinds of recurrence
#define LS_DELTA 1
#define LS_GATED 2

#define LS_WHOLE 0                  // a lane from and into its request's state
#define LS_LOCAL 1                  // a chunk from an empty state (and the unit vectors): no outputs
#define LS_CHUNK 2                  // a chunk from its starting state

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
// log(sigmoid(x)) = min(x, 0) - log1p(exp(-|x|)): finite for any finite x
__device__ __forceinline__ float log_sigmoid_f(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// sum over the R neighbouring lanes of a column (R a power of two up to 64).  A constant R up to 16 stays inside a
// row of 16 lanes, where the data-parallel primitives exchange lanes without a trip through the LDS crossbar:
// neighbours in a quad, the quads' other pair, then the mirror image within 8 and within 16 lanes (every lane of
// a half holds the half's sum by then, so the mirror brings the other half's).
template <int CONTROL>
__device__ __forceinline__ float lanes_moved(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CONTROL, 0xf, 0xf, true));
}

template <int R_CONST>
__device__ __forceinline__ float column_sum(float v, int R) {
  if (R_CONST > 0) {
    if (R_CONST >= 2) v += lanes_moved<0xB1>(v);       // quad_perm [1, 0, 3, 2]
    if (R_CONST >= 4) v += lanes_moved<0x4E>(v);       // quad_perm [2, 3, 0, 1]
    if (R_CONST >= 8) v += lanes_moved<0x141>(v);      // row_half_mirror
    if (R_CONST >= 16) v += lanes_moved<0x140>(v);     // row_mirror
  } else {
    for (int offset = R >> 1; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, WAVE);
  }
  return v;
}

__device__ __forceinline__ float dot4(const float4 a, const float* s) {
  return fmaf(a.w, s[3], fmaf(a.z, s[2], fmaf(a.y, s[1], a.x * s[0])));
}

// R_CONST: the lanes of a column when the launch knows them at compile time (1 .. 16), 0: a.R.
// PL: key channels a lane; a lane keeps 16 / PL neighbouring columns (their states in 16 registers), so that the
// token's vectors come out of LDS once for all of them.  PL = 16: one column, a.per_lane (<= 16) channels of it.
template <typename T, int KIND, int MODE, int R_CONST, int PL>
__global__ void __launch_bounds__(MODE == LS_WHOLE ? LS_THREADS : LS_PASS_THREADS)
linear_state_scan_kernel(const ScanArgs a) {
  constexpr bool DELTA = KIND == LS_DELTA;
  constexpr bool GATED = KIND == LS_GATED;
  constexpr int CPL = LS_MAX_PER_LANE / PL;              // columns a lane
  extern __shared__ __align__(16) float stage_lds[];
  const int head = blockIdx.y;
  int lane_of_step, first_token, end_token;
  bool last_of_lane = true;
  if (MODE == LS_WHOLE) {
    lane_of_step = blockIdx.x;
    first_token = a.cu_seqlens[lane_of_step];
    end_token = a.cu_seqlens[lane_of_step + 1];
  } else {
    const int* row = a.chunks + 4 * blockIdx.x;
    lane_of_step = row[0];
    if (lane_of_step < 0) return;                          // a row past the step's own chunks
    first_token = row[1];
    end_token = first_token + row[2];
    last_of_lane = row[3] == a.lane_chunks[2 * lane_of_step + 1] - 1;
    if (MODE == LS_LOCAL && last_of_lane) return;          // nothing follows it
  }
  if (end_token <= first_token) return;
  const int tid = threadIdx.x;
  const int wave = tid / WAVE;
  const int lane = tid & (WAVE - 1);
  const int waves = blockDim.x / WAVE;
  const int R = R_CONST > 0 ? R_CONST : a.R;
  const int per_lane = PL < LS_MAX_PER_LANE ? PL : a.per_lane;   // a multiple of 4
  const int dk = a.dk, dv = a.dv;
  const int padded = R * per_lane;                       // a vector's length in LDS; channels past dk hold zeros
  const int vectors = DELTA ? 5 : GATED ? 3 : 2;
  const int token_floats = vectors * padded + ((a.columns + 3) & ~3);
  const int group = tid / R;                             // the lanes of one run of CPL columns
  const int sub = tid - group * R;
  const int column_in_group = group * CPL;               // the first of this lane's columns among the workgroup's
  const int column0 = blockIdx.z * a.columns + column_in_group;
  // the local pass of the delta rule carries dk more columns: the transition's, which start as the unit vectors;
  // that of the gated decay one more: the diagonal transition, which starts as ones
  const int total_columns = MODE == LS_LOCAL ? (DELTA ? dv + dk : GATED ? dv + 1 : dv) : dv;
  const bool in_group = column_in_group < a.columns;
  const int channel0 = sub * per_lane;
  const T* rows = (const T*)a.u;

  // the columns' share of the state
  float s[CPL][PL];
  const bool whole_fours = a.whole_fours != 0;
  const long state_head = ((long)a.slot_ids[lane_of_step] * a.H + head) * dv;
#pragma unroll
  for (int c = 0; c < CPL; ++c) {
    const int column = column0 + c;
    const bool mine = in_group && column_in_group + c < a.columns && column < total_columns;
    const float* from = a.state + (state_head + (mine && column < dv ? column : 0)) * dk;
    if (MODE == LS_CHUNK) from = a.start + (((long)blockIdx.x * a.H + head) * dv + (mine ? column : 0)) * dk;
    if (MODE != LS_LOCAL && whole_fours) {
      // dk a multiple of 4: a lane's run of channels is whole groups of four, 16 bytes a load
#pragma unroll
      for (int g = 0; g < PL / 4; ++g) {
        const int channel = channel0 + 4 * g;
        const bool held = mine && 4 * g < per_lane && channel < dk;
        const float4 four = held ? *reinterpret_cast<const float4*>(from + channel) : make_float4(0.f, 0.f, 0.f, 0.f);
        s[c][4 * g + 0] = four.x;
        s[c][4 * g + 1] = four.y;
        s[c][4 * g + 2] = four.z;
        s[c][4 * g + 3] = four.w;
      }
      continue;
    }
#pragma unroll
    for (int e = 0; e < PL; ++e) {
      const int channel = channel0 + e;
      const bool held = mine && e < per_lane && channel < dk;
      if (MODE == LS_LOCAL) s[c][e] = (held && (GATED ? column == dv : channel == column - dv)) ? 1.f : 0.f;
      else s[c][e] = held ? from[channel] : 0.f;
    }
  }
  const float decay = KIND == LS_RETENTION ? a.head_decay[head] : 0.f;
  const int half = a.rotary_dim / 2;

  for (int stage_first = first_token; stage_first < end_token; stage_first += a.stage) {
    const int count = min(a.stage, end_token - stage_first);
    __syncthreads();                                       // the stage before is read
    // ---- lay the stage's vectors in LDS: every thread an element (token, channel) at a time, so that the loads
    // of a whole stage are under way together
    for (int index = tid; index < count * padded; index += blockDim.x) {
      const int tt = index / padded;
      const int channel = index - tt * padded;
      const long token = stage_first + tt;
      const T* row = rows + token * a.ld;
      float* q_lds = stage_lds + tt * token_floats;
      float qx = 0.f, kx = 0.f, w = 0.f, removal = 0.f;
      if (channel < dk) {
        qx = to_float(row[a.q_col + head * dk + channel]);
        kx = to_float(row[a.k_col + head * dk + channel]);
        if (DELTA) {
          removal = sigmoid_f(to_float(row[a.removal_col + head * dk + channel]));
          w = expf(-a.decay_floor * sigmoid_f(a.decay_logits[token * a.logits_ld + head * dk + channel] +
                                              a.decay_bias[head * dk + channel]));
        } else {
          if (a.inv_freq && channel < a.rotary_dim) {
            const bool low = channel < half;
            const int pair = low ? channel + half : channel - half;
            const float angle = (float)a.positions[token] * a.inv_freq[low ? channel : channel - half];
            float sine, cosine;
            sincosf(angle, &sine, &cosine);
            const float q_pair = to_float(row[a.q_col + head * dk + pair]);
            const float k_pair = to_float(row[a.k_col + head * dk + pair]);
            // (x, y) -> (x cos - y sin, y cos + x sin): the low half is x, the high half y
            qx = low ? qx * cosine - q_pair * sine : qx * cosine + q_pair * sine;
            kx = low ? kx * cosine - k_pair * sine : kx * cosine + k_pair * sine;
          }
          kx *= a.key_scale;
          if (GATED)
            w = expf(a.gate_power * log_sigmoid_f(a.decay_logits[token * a.logits_ld + head * dk + channel] +
                                                  a.decay_bias[head * dk + channel]));
        }
        qx *= a.query_scale;
      }
      q_lds[channel] = qx;
      q_lds[padded + channel] = kx;
      if (GATED) q_lds[2 * padded + channel] = w;
      if (DELTA) {
        q_lds[2 * padded + channel] = w;
        q_lds[4 * padded + channel] = removal;             // times the unit key below
      }
    }
    // the values of this workgroup's columns
    for (int index = tid; index < count * a.columns; index += blockDim.x) {
      const int tt = index / a.columns;
      const int c = index - tt * a.columns;
      const int value_column = blockIdx.z * a.columns + c;
      stage_lds[tt * token_floats + vectors * padded + c] =
          value_column < dv ? to_float(rows[(long)(stage_first + tt) * a.ld + a.v_col + head * dv + value_column]) : 0.f;
    }
    if (DELTA) {
      __syncthreads();
      // the unit keys: a wave a token
      for (int tt = wave; tt < count; tt += waves) {
        float* k_lds = stage_lds + tt * token_floats + padded;
        float sum_squares = 0.f;
        for (int channel = lane; channel < padded; channel += WAVE) sum_squares = fmaf(k_lds[channel], k_lds[channel], sum_squares);
        const float length = sqrtf(wave_sum(sum_squares) + a.key_eps);
        for (int channel = lane; channel < padded; channel += WAVE) {
          const float unit = k_lds[channel] / length;
          k_lds[2 * padded + channel] = unit;
          k_lds[3 * padded + channel] *= unit;
        }
      }
    }
    __syncthreads();
    // ---- the tokens of the stage in order
    if (in_group) {
      for (int tt = 0; tt < count; ++tt) {
        const float* q_lds = stage_lds + tt * token_floats + channel0;
        const float* k_lds = q_lds + padded;
        const float* values = stage_lds + tt * token_floats + vectors * padded + column_in_group;
        float value[CPL];
#pragma unroll
        for (int c = 0; c < CPL; ++c) value[c] = values[CPL > 1 ? min(c, a.columns - 1 - column_in_group) : 0];
        if (DELTA) {
          const float* w_lds = k_lds + padded;
          const float* u_lds = w_lds + padded;
          const float* au_lds = u_lds + padded;
          float along[CPL];
#pragma unroll
          for (int c = 0; c < CPL; ++c) along[c] = 0.f;
          float part[CPL][PL / 4];
#pragma unroll
          for (int g = 0; g < PL / 4; ++g) {
            const bool live = 4 * g < per_lane;
            const float4 u4 = live ? *reinterpret_cast<const float4*>(u_lds + 4 * g) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int c = 0; c < CPL; ++c) part[c][g] = dot4(u4, s[c] + 4 * g);
          }
#pragma unroll
          for (int c = 0; c < CPL; ++c) {
            float sum = part[c][0];
#pragma unroll
            for (int g = 1; g < PL / 4; ++g) sum += part[c][g];
            along[c] = column_sum<R_CONST>(sum, R);
          }
#pragma unroll
          for (int g = 0; g < PL / 4; ++g)
            if (4 * g < per_lane) {
              const float4 k4 = *reinterpret_cast<const float4*>(k_lds + 4 * g);
              const float4 w4 = *reinterpret_cast<const float4*>(w_lds + 4 * g);
              const float4 au4 = *reinterpret_cast<const float4*>(au_lds + 4 * g);
#pragma unroll
              for (int c = 0; c < CPL; ++c) {
                s[c][4 * g + 0] = fmaf(k4.x, value[c], fmaf(-au4.x, along[c], w4.x * s[c][4 * g + 0]));
                s[c][4 * g + 1] = fmaf(k4.y, value[c], fmaf(-au4.y, along[c], w4.y * s[c][4 * g + 1]));
                s[c][4 * g + 2] = fmaf(k4.z, value[c], fmaf(-au4.z, along[c], w4.z * s[c][4 * g + 2]));
                s[c][4 * g + 3] = fmaf(k4.w, value[c], fmaf(-au4.w, along[c], w4.w * s[c][4 * g + 3]));
              }
            }
        } else if (GATED) {
          const float* w_lds = k_lds + padded;
#pragma unroll
          for (int g = 0; g < PL / 4; ++g)
            if (4 * g < per_lane) {
              const float4 k4 = *reinterpret_cast<const float4*>(k_lds + 4 * g);
              const float4 w4 = *reinterpret_cast<const float4*>(w_lds + 4 * g);
#pragma unroll
              for (int c = 0; c < CPL; ++c) {
                s[c][4 * g + 0] = fmaf(k4.x, value[c], w4.x * s[c][4 * g + 0]);
                s[c][4 * g + 1] = fmaf(k4.y, value[c], w4.y * s[c][4 * g + 1]);
                s[c][4 * g + 2] = fmaf(k4.z, value[c], w4.z * s[c][4 * g + 2]);
                s[c][4 * g + 3] = fmaf(k4.w, value[c], w4.w * s[c][4 * g + 3]);
              }
            }
        } else {
#pragma unroll
          for (int g = 0; g < PL / 4; ++g)
            if (4 * g < per_lane) {
              const float4 k4 = *reinterpret_cast<const float4*>(k_lds + 4 * g);
#pragma unroll
              for (int c = 0; c < CPL; ++c) {
                s[c][4 * g + 0] = fmaf(k4.x, value[c], decay * s[c][4 * g + 0]);
                s[c][4 * g + 1] = fmaf(k4.y, value[c], decay * s[c][4 * g + 1]);
                s[c][4 * g + 2] = fmaf(k4.z, value[c], decay * s[c][4 * g + 2]);
                s[c][4 * g + 3] = fmaf(k4.w, value[c], decay * s[c][4 * g + 3]);
              }
            }
        }
        if (MODE != LS_LOCAL) {
          float part[CPL][PL / 4];
#pragma unroll
          for (int g = 0; g < PL / 4; ++g) {
            const bool live = 4 * g < per_lane;
            const float4 q4 = live ? *reinterpret_cast<const float4*>(q_lds + 4 * g) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int c = 0; c < CPL; ++c) part[c][g] = dot4(q4, s[c] + 4 * g);
          }
#pragma unroll
          for (int c = 0; c < CPL; ++c) {
            float sum = part[c][0];
#pragma unroll
            for (int g = 1; g < PL / 4; ++g) sum += part[c][g];
            const float result = column_sum<R_CONST>(sum, R);
            const int column = column0 + c;
            if (sub == 0 && column_in_group + c < a.columns && column < dv)
              a.out[(long)(stage_first + tt) * a.out_ld + head * dv + column] = result;
          }
        }
      }
    }
  }
#pragma unroll
  for (int c = 0; c < CPL; ++c) {
    const int column = column0 + c;
    const bool mine = in_group && column_in_group + c < a.columns && column < total_columns;
    float* into = a.state + (state_head + (mine && column < dv ? column : 0)) * dk;
    if (MODE == LS_LOCAL) into = a.local + (((long)blockIdx.x * a.H + head) * total_columns + (mine ? column : 0)) * dk;
    if (mine && (MODE != LS_CHUNK || last_of_lane)) {
      if (whole_fours) {
#pragma unroll
        for (int g = 0; g < PL / 4; ++g) {
          const int channel = channel0 + 4 * g;
          if (4 * g < per_lane && channel < dk)
            *reinterpret_cast<float4*>(into + channel) =
                make_float4(s[c][4 * g + 0], s[c][4 * g + 1], s[c][4 * g + 2], s[c][4 * g + 3]);
        }
      } else {
#pragma unroll
        for (int e = 0; e < PL; ++e) {
          const int channel = channel0 + e;
          if (e < per_lane && channel < dk) into[channel] = s[c][e];
        }
      }
    }
  }
}

// ---------------------------------------------------------------- the carry from chunk to chunk
// One workgroup a (lane, head, run of LS_CARRY_COLUMNS value columns): the columns' states sit in LDS, a thread
// owns key channels m and computes, for its columns j, s_j[m] <- sum_i P[m, i] s_j[i] + B_j[m] chunk after chunk
// (P's column i is row dv + i of what the local pass left); every chunk's starting state goes to ``start``.
#define LS_CARRY_COLUMNS 4

template <int KIND>
__global__ void __launch_bounds__(LS_THREADS)
linear_state_carry_kernel(const ScanArgs a) {
  constexpr bool DELTA = KIND == LS_DELTA;
  constexpr bool GATED = KIND == LS_GATED;
  extern __shared__ __align__(16) float carry_lds[];       // [LS_CARRY_COLUMNS][dk]
  const int lane_of_step = blockIdx.x;
  const int head = blockIdx.y;
  const int first_chunk = a.lane_chunks[2 * lane_of_step];
  const int count = a.lane_chunks[2 * lane_of_step + 1];
  if (count <= 0) return;
  const int dk = a.dk, dv = a.dv;
  const int column0 = blockIdx.z * LS_CARRY_COLUMNS;
  const int total_columns = DELTA ? dv + dk : GATED ? dv + 1 : dv;
  const float* state = a.state + ((long)a.slot_ids[lane_of_step] * a.H + head) * dv * dk;
  for (int index = threadIdx.x; index < LS_CARRY_COLUMNS * dk; index += blockDim.x) {
    const int c = index / dk, m = index - c * dk;
    const float value = column0 + c < dv ? state[(long)(column0 + c) * dk + m] : 0.f;
    carry_lds[index] = value;
    if (column0 + c < dv) a.start[(((long)first_chunk * a.H + head) * dv + column0 + c) * dk + m] = value;
  }
  __syncthreads();
  const float decay = KIND == LS_RETENTION ? a.head_decay[head] : 0.f;
  for (int chunk = first_chunk; chunk < first_chunk + count - 1; ++chunk) {
    const float* local = a.local + ((long)chunk * a.H + head) * total_columns * dk;
    float* start = a.start + ((long)(chunk + 1) * a.H + head) * dv * dk;
    const float shrink = KIND == LS_RETENTION ? powf(decay, (float)a.chunks[4 * chunk + 2]) : 0.f;
    // more key channels than threads: rounds of blockDim.x channels (the new values wait in registers of the round)
    for (int m0 = 0; m0 < dk; m0 += blockDim.x) {
      const int m = m0 + threadIdx.x;
      float next[LS_CARRY_COLUMNS];
#pragma unroll
      for (int c = 0; c < LS_CARRY_COLUMNS; ++c) next[c] = 0.f;
      if (m < dk) {
        if (DELTA) {
          const float* transition = local + (long)dv * dk + m;       // P[m, i] at transition[i * dk]
          // 32 of the transition's elements are asked for before the first is used
          for (int i0 = 0; i0 < dk; i0 += 32) {
            float p[32];
#pragma unroll
            for (int j = 0; j < 32; ++j) p[j] = transition[(long)min(i0 + j, dk - 1) * dk];
#pragma unroll
            for (int j = 0; j < 32; ++j) {
              const int i = min(i0 + j, dk - 1);
              const float weight = i0 + j < dk ? p[j] : 0.f;
#pragma unroll
              for (int c = 0; c < LS_CARRY_COLUMNS; ++c) next[c] = fmaf(weight, carry_lds[c * dk + i], next[c]);
            }
          }
        } else {
          // retention: one number a chunk; gated decay: channel m's product of the chunk's gates
          const float through = GATED ? local[(long)dv * dk + m] : shrink;
#pragma unroll
          for (int c = 0; c < LS_CARRY_COLUMNS; ++c) next[c] = through * carry_lds[c * dk + m];
        }
#pragma unroll
        for (int c = 0; c < LS_CARRY_COLUMNS; ++c)
          if (column0 + c < dv) next[c] += local[(long)(column0 + c) * dk + m];
      }
      __syncthreads();                                      // the old state is read before any of it is replaced
      if (m < dk) {
#pragma unroll
        for (int c = 0; c < LS_CARRY_COLUMNS; ++c) {
          if (dk <= (int)blockDim.x) carry_lds[c * dk + m] = next[c];
          if (column0 + c < dv) start[(long)(column0 + c) * dk + m] = next[c];
        }
      }
    }
    __syncthreads();
    if (dk > (int)blockDim.x) {                             // several rounds: the new state comes back from memory
      for (int index = threadIdx.x; index < LS_CARRY_COLUMNS * dk; index += blockDim.x) {
        const int c = index / dk, m = index - c * dk;
        carry_lds[index] = column0 + c < dv ? start[(long)(column0 + c) * dk + m] : 0.f;
      }
      __syncthreads();
    }
  }
}

// How a head's state is dealt out: R lanes a column (the smallest power of two that leaves a lane at most
// LS_MAX_PER_LANE key channels), per_lane = ceil(dk / R) channels a lane, LS_THREADS / R columns a workgroup of a
// prompt portion (one wave's worth, 64 / R, for steps of single tokens, which want many small workgroups).
static int scan_args(ScanArgs& a, const void* u, long ld, int q_col, int k_col, int v_col, int removal_col, int H, int dk,
                     int dv, float* state, const int* cu_seqlens, const int* slot_ids, int lanes, float* out, long out_ld,
                     const float* head_decay, float key_scale, const int* positions, const float* inv_freq,
                     int rotary_dim, const float* decay_logits, long logits_ld, const float* decay_bias,
                     float decay_floor, float key_eps, float gate_power, float query_scale) {
  if (!u || !state || !cu_seqlens || !slot_ids || !out || lanes <= 0 || H <= 0 || dk <= 0 || dv <= 0)
    return ERR_BAD_ARGUMENT;
  const bool delta = removal_col >= 0;
  const bool gated = !delta && gate_power > 0.f;
  if ((delta || gated) && (!decay_logits || !decay_bias || logits_ld < (long)H * dk)) return ERR_BAD_ARGUMENT;
  if (!delta && !gated && !head_decay) return ERR_BAD_ARGUMENT;
  if (inv_freq && (!positions || rotary_dim <= 0 || rotary_dim > dk || (rotary_dim & 1))) return ERR_BAD_ARGUMENT;
  if (out_ld < (long)H * dv) return ERR_BAD_ARGUMENT;
  if (dk > LS_MAX_PER_LANE * WAVE || H > 65535 || lanes > 0x7fffffff) return ERR_UNSUPPORTED_SIZE;
  a.u = u; a.ld = ld; a.q_col = q_col; a.k_col = k_col; a.v_col = v_col; a.removal_col = removal_col;
  a.H = H; a.dk = dk; a.dv = dv; a.state = state; a.cu_seqlens = cu_seqlens; a.slot_ids = slot_ids;
  a.out = out; a.out_ld = out_ld; a.head_decay = head_decay; a.key_scale = key_scale; a.positions = positions;
  a.inv_freq = inv_freq; a.rotary_dim = inv_freq ? rotary_dim : 0; a.decay_logits = decay_logits;
  a.logits_ld = logits_ld; a.decay_bias = decay_bias; a.decay_floor = decay_floor; a.key_eps = key_eps;
  a.gate_power = gate_power; a.query_scale = query_scale;
  a.chunks = nullptr; a.lane_chunks = nullptr; a.local = nullptr; a.start = nullptr;
  a.whole_fours = (dk % 4 == 0 && (uintptr_t)state % 16 == 0) ? 1 : 0;
  int R = 1;
  while (R * LS_MAX_PER_LANE < dk) R *= 2;
  a.R = R;
  a.per_lane = (((dk + R - 1) / R + 3) / 4) * 4;           // whole groups of four channels: 16-byte reads from LDS
  return 0;
}

// columns a workgroup of ``threads`` threads takes of ``total_columns``, the tokens of a stage and its bytes in LDS
static int scan_shape(ScanArgs& a, int threads, int total_columns, int kind, int longest, size_t* lds, int* splits) {
  a.columns = threads / a.R;
  if (a.columns > total_columns) a.columns = total_columns;
  *splits = (total_columns + a.columns - 1) / a.columns;
  if (*splits > 65535) return ERR_UNSUPPORTED_SIZE;
  const int token_floats = (kind == LS_DELTA ? 5 : kind == LS_GATED ? 3 : 2) * a.R * a.per_lane + ((a.columns + 3) & ~3);
  int stage = LS_STAGE_BYTES / (token_floats * (int)sizeof(float));
  if (stage > LS_STAGE_MOST) stage = LS_STAGE_MOST;
  if (longest > 0 && stage > longest) stage = longest;
  if (stage < 1) return ERR_UNSUPPORTED_SIZE;
  a.stage = stage;
  *lds = (size_t)stage * token_floats * sizeof(float);
  return 0;
}

#define LS_LAUNCH_R(MODE_, R_, PL_, grid_, threads_, lds_)                                                         \
  do {                                                                                                            \
    if (dtype == DT_F32) {                                                                                        \
      if (kind == LS_DELTA) linear_state_scan_kernel<float, LS_DELTA, MODE_, R_, PL_><<<grid_, threads_, lds_, stream>>>(a); \
      else if (kind == LS_GATED) linear_state_scan_kernel<float, LS_GATED, MODE_, R_, PL_><<<grid_, threads_, lds_, stream>>>(a); \
      else linear_state_scan_kernel<float, LS_RETENTION, MODE_, R_, PL_><<<grid_, threads_, lds_, stream>>>(a);   \
    } else {                                                                                                      \
      if (kind == LS_DELTA) linear_state_scan_kernel<bf16_t, LS_DELTA, MODE_, R_, PL_><<<grid_, threads_, lds_, stream>>>(a); \
      else if (kind == LS_GATED) linear_state_scan_kernel<bf16_t, LS_GATED, MODE_, R_, PL_><<<grid_, threads_, lds_, stream>>>(a); \
      else linear_state_scan_kernel<bf16_t, LS_RETENTION, MODE_, R_, PL_><<<grid_, threads_, lds_, stream>>>(a);  \
    }                                                                                                             \
  } while (0)
// the walk from end to end: one column a lane, up to 16 channels of it
#define LS_LAUNCH_WHOLE(grid_, threads_, lds_)                                                                    \
  do {                                                                                                            \
    switch (a.R) {                                                                                                \
      case 1: LS_LAUNCH_R(LS_WHOLE, 1, 16, grid_, threads_, lds_); break;                                         \
      case 2: LS_LAUNCH_R(LS_WHOLE, 2, 16, grid_, threads_, lds_); break;                                         \
      case 4: LS_LAUNCH_R(LS_WHOLE, 4, 16, grid_, threads_, lds_); break;                                         \
      case 8: LS_LAUNCH_R(LS_WHOLE, 8, 16, grid_, threads_, lds_); break;                                         \
      default: LS_LAUNCH_R(LS_WHOLE, 0, 16, grid_, threads_, lds_); break;                                        \
    }                                                                                                             \
  } while (0)
// the passes over chunks: (lanes a column, channels a lane) as pass_shape chose them
#define LS_LAUNCH_PASS(MODE_, grid_, threads_, lds_)                                                              \
  do {                                                                                                            \
    if (a.per_lane == 4 && a.R == 1) LS_LAUNCH_R(MODE_, 1, 4, grid_, threads_, lds_);                             \
    else if (a.per_lane == 4 && a.R == 2) LS_LAUNCH_R(MODE_, 2, 4, grid_, threads_, lds_);                        \
    else if (a.per_lane == 4 && a.R == 4) LS_LAUNCH_R(MODE_, 4, 4, grid_, threads_, lds_);                        \
    else if (a.per_lane == 4 && a.R == 8) LS_LAUNCH_R(MODE_, 8, 4, grid_, threads_, lds_);                        \
    else if (a.per_lane == 4 && a.R == 16) LS_LAUNCH_R(MODE_, 16, 4, grid_, threads_, lds_);                      \
    else if (a.per_lane == 8 && a.R == 16) LS_LAUNCH_R(MODE_, 16, 8, grid_, threads_, lds_);                      \
    else if (a.R == 16) LS_LAUNCH_R(MODE_, 16, 16, grid_, threads_, lds_);                                        \
    else LS_LAUNCH_R(MODE_, 0, 16, grid_, threads_, lds_);                                                        \
  } while (0)

extern "C" int mi_linear_state_scan(const void* u, int dtype, long ld, int q_col, int k_col, int v_col, int removal_col,
                                    int H, int dk, int dv, float* state, const int* cu_seqlens, const int* slot_ids,
                                    int lanes, float* out, long out_ld, int max_query_len, const float* head_decay,
                                    float key_scale, const int* positions, const float* inv_freq, int rotary_dim,
                                    const float* decay_logits, long logits_ld, const float* decay_bias,
                                    float decay_floor, float key_eps, float gate_power, float query_scale,
                                    hipStream_t stream) {
  if (dtype != DT_F32 && dtype != DT_BF16) return ERR_BAD_ARGUMENT;
  ScanArgs a;
  int code = scan_args(a, u, ld, q_col, k_col, v_col, removal_col, H, dk, dv, state, cu_seqlens, slot_ids, lanes, out,
                       out_ld, head_decay, key_scale, positions, inv_freq, rotary_dim, decay_logits, logits_ld,
                       decay_bias, decay_floor, key_eps, gate_power, query_scale);
  if (code) return code;
  const int kind = removal_col >= 0 ? LS_DELTA : gate_power > 0.f ? LS_GATED : LS_RETENTION;
  const int threads = max_query_len == 1 ? WAVE : LS_THREADS;
  size_t lds;
  int splits;
  code = scan_shape(a, threads, dv, kind, max_query_len, &lds, &splits);
  if (code) return code;
  const dim3 grid(lanes, H, splits);
  LS_LAUNCH_WHOLE(grid, threads, lds);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// floats of the two workspaces of the passes over ``chunks`` chunks
extern "C" long mi_linear_state_local_floats(int chunks, int H, int dk, int dv, int kind) {
  return (long)chunks * H * (kind == LS_DELTA ? dv + dk : kind == LS_GATED ? dv + 1 : dv) * dk;
}
extern "C" long mi_linear_state_start_floats(int chunks, int H, int dk, int dv) { return (long)chunks * H * dv * dk; }

// The same scan in three passes over the step's chunks (see the top of the file).  ``chunks`` int32 [num_chunks, 4],
// ``lane_chunks`` int32 [lanes, 2]; ``local`` and ``start``: float32 workspaces of the sizes above.
extern "C" int mi_linear_state_scan_chunked(const void* u, int dtype, long ld, int q_col, int k_col, int v_col,
                                            int removal_col, int H, int dk, int dv, float* state,
                                            const int* cu_seqlens, const int* slot_ids, int lanes, float* out,
                                            long out_ld, int chunk_tokens, const float* head_decay, float key_scale,
                                            const int* positions, const float* inv_freq, int rotary_dim,
                                            const float* decay_logits, long logits_ld, const float* decay_bias,
                                            float decay_floor, float key_eps, float gate_power, float query_scale,
                                            const int* chunks, const int* lane_chunks,
                                            int num_chunks, float* local, float* start, hipStream_t stream) {
  if (dtype != DT_F32 && dtype != DT_BF16) return ERR_BAD_ARGUMENT;
  if (!chunks || !lane_chunks || num_chunks <= 0 || !local || !start || chunk_tokens <= 0) return ERR_BAD_ARGUMENT;
  ScanArgs a;
  int code = scan_args(a, u, ld, q_col, k_col, v_col, removal_col, H, dk, dv, state, cu_seqlens, slot_ids, lanes, out,
                       out_ld, head_decay, key_scale, positions, inv_freq, rotary_dim, decay_logits, logits_ld,
                       decay_bias, decay_floor, key_eps, gate_power, query_scale);
  if (code) return code;
  a.chunks = chunks; a.lane_chunks = lane_chunks; a.local = local; a.start = start;
  if ((uintptr_t)local % 16 != 0 || (uintptr_t)start % 16 != 0) a.whole_fours = 0;
  const int kind = removal_col >= 0 ? LS_DELTA : gate_power > 0.f ? LS_GATED : LS_RETENTION;
  size_t lds;
  int splits;
  // the passes spread a column over more lanes than the walk from end to end: up to LS_PASS_LANES, four key
  // channels a lane or more, so that a token is a short chain of sums and a workgroup of LS_PASS_THREADS threads
  // still takes 64 columns with one copy of the stage's vectors
  // and a lane keeps 16 / (channels a lane) neighbouring columns, which share every read of the token's vectors
  int columns_a_lane = 1;
  {
    const int channels = dk <= 64 ? 4 : dk <= 128 ? 8 : LS_MAX_PER_LANE;
    int R = 1;
    while (R * channels < dk) R *= 2;
    a.R = R;
    a.per_lane = channels < LS_MAX_PER_LANE ? channels : (((dk + R - 1) / R + 3) / 4) * 4;
    columns_a_lane = LS_MAX_PER_LANE / channels;
  }
  // local: the chunks' own states (and transitions)
  code = scan_shape(a, LS_PASS_THREADS * columns_a_lane, kind == LS_DELTA ? dv + dk : kind == LS_GATED ? dv + 1 : dv, kind,
                    chunk_tokens, &lds, &splits);
  if (code) return code;
  // no more waves than the columns fill
  int threads = (((a.columns + columns_a_lane - 1) / columns_a_lane * a.R + WAVE - 1) / WAVE) * WAVE;
  if (threads < LS_THREADS) threads = LS_THREADS;
  LS_LAUNCH_PASS(LS_LOCAL, dim3(num_chunks, H, splits), threads, lds);
  RETURN_IF_LAUNCH_FAILED();
  // carry: every chunk's starting state
  const int carry_splits = (dv + LS_CARRY_COLUMNS - 1) / LS_CARRY_COLUMNS;
  if (carry_splits > 65535) return ERR_UNSUPPORTED_SIZE;
  int carry_threads = ((dk + WAVE - 1) / WAVE) * WAVE;
  if (carry_threads > LS_THREADS) carry_threads = LS_THREADS;
  const size_t carry_lds = (size_t)LS_CARRY_COLUMNS * dk * sizeof(float);
  if (kind == LS_DELTA) linear_state_carry_kernel<LS_DELTA><<<dim3(lanes, H, carry_splits), carry_threads, carry_lds, stream>>>(a);
  else if (kind == LS_GATED) linear_state_carry_kernel<LS_GATED><<<dim3(lanes, H, carry_splits), carry_threads, carry_lds, stream>>>(a);
  else linear_state_carry_kernel<LS_RETENTION><<<dim3(lanes, H, carry_splits), carry_threads, carry_lds, stream>>>(a);
  RETURN_IF_LAUNCH_FAILED();
  // scan: the outputs, and the requests' states behind their last chunks
  code = scan_shape(a, LS_PASS_THREADS * columns_a_lane, dv, kind, chunk_tokens, &lds, &splits);
  if (code) return code;
  threads = (((a.columns + columns_a_lane - 1) / columns_a_lane * a.R + WAVE - 1) / WAVE) * WAVE;
  if (threads < LS_THREADS) threads = LS_THREADS;
  LS_LAUNCH_PASS(LS_CHUNK, dim3(num_chunks, H, splits), threads, lds);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- head norm, weight and gate
// out[t, h, j] = raw[t, h, j] / sqrt(mean_j raw[t, h, :]^2 + eps) (* weight[h*dv + j]) * act(gate[t, h*dv + j]),
// act = SiLU (0) or the logistic sigmoid (1); statistics and products in float32.  One wave a (token, head).
template <typename T>
__global__ void __launch_bounds__(WAVE)
head_norm_gate_kernel(const float* __restrict__ raw, long raw_ld, const T* __restrict__ gate, long gate_ld,
                      const float* __restrict__ weight, int dv, float eps, int activation, T* __restrict__ out,
                      long out_ld) {
  const long token = blockIdx.x;
  const int head = blockIdx.y;
  const float* r = raw + token * raw_ld + (long)head * dv;
  float sum_squares = 0.f;
  for (int j = threadIdx.x; j < dv; j += WAVE) sum_squares += r[j] * r[j];
  const float denominator = sqrtf(wave_sum(sum_squares) / (float)dv + eps);
  const T* g = gate + token * gate_ld + (long)head * dv;
  T* o = out + token * out_ld + (long)head * dv;
  for (int j = threadIdx.x; j < dv; j += WAVE) {
    float value = r[j] / denominator;
    if (weight) value *= weight[head * dv + j];
    const float x = to_float(g[j]);
    value *= activation == 0 ? silu_f(x) : sigmoid_f(x);
    o[j] = from_float<T>(value);
  }
}

extern "C" int mi_head_norm_gate(const float* raw, long raw_ld, const void* gate, int dtype, long gate_ld,
                                 const float* weight, int H, int dv, float eps, int activation, void* out, long out_ld,
                                 int T, hipStream_t stream) {
  if (!raw || !gate || !out || T <= 0 || H <= 0 || dv <= 0 || H > 65535 || (activation != 0 && activation != 1))
    return ERR_BAD_ARGUMENT;
  const dim3 grid(T, H);
  if (dtype == DT_F32)
    head_norm_gate_kernel<float><<<grid, WAVE, 0, stream>>>(raw, raw_ld, (const float*)gate, gate_ld, weight, dv, eps,
                                                            activation, (float*)out, out_ld);
  else if (dtype == DT_BF16)
    head_norm_gate_kernel<bf16_t><<<grid, WAVE, 0, stream>>>(raw, raw_ld, (const bf16_t*)gate, gate_ld, weight, dv, eps,
                                                             activation, (bf16_t*)out, out_ld);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- tanh of a block of columns
template <typename T>
__global__ void tanh_rows_kernel(const T* __restrict__ x, long ld, T* __restrict__ out, long out_ld, int width, long total) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= total) return;
  const long t = index / width;
  const int i = (int)(index - t * width);
  out[t * out_ld + i] = from_float<T>(tanhf(to_float(x[t * ld + i])));
}

extern "C" int mi_tanh_rows(const void* x, int dtype, long ld, void* out, long out_ld, int T, int width,
                            hipStream_t stream) {
  if (!x || !out || T <= 0 || width <= 0 || ld < width || out_ld < width) return ERR_BAD_ARGUMENT;
  const long total = (long)T * width;
  const int blocks = (int)((total + 255) / 256);
  if (dtype == DT_F32)
    tanh_rows_kernel<float><<<blocks, 256, 0, stream>>>((const float*)x, ld, (float*)out, out_ld, width, total);
  else if (dtype == DT_BF16)
    tanh_rows_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)x, ld, (bf16_t*)out, out_ld, width, total);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}
