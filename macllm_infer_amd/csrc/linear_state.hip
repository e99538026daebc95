// Mixers that carry a matrix-valued state per head: the scan of linear attention with a decay, in two forms,
// and what follows it.
//
//   retention        S <- decay[h] * S + k v^T                         o = S^T q
//   delta rule       S <- diag(w) S - (a * u)(u^T S) + k v^T           o = S^T r      (both products on the old S)
//
// with S [dk, dv] per head in float32, carried from token to token in the request's state slot.  What enters the
// recurrence is formed in float32 from the projection's rows inside the scan:
//   retention : q and k turned by position (half-split rotation of the first rotary_dim dims, angle =
//               (float)position * inv_freq[j]), then k * key_scale;
//   delta rule: u = k / sqrt(sum k^2 + key_eps), a = sigmoid(removal columns),
//               w = exp(-decay_floor * sigmoid(decay_logits + decay_bias)).
//
// The state is stored transposed, [slot][head][dv][dk]: a column of S (all key channels of one value channel)
// evolves on its own,
//   s_j <- w * s_j - (a * u) (u . s_j) + k v_j,    o_j = s_j . q,
// so a column is the unit of work: R neighbouring lanes own one column, each LS_PER_LANE-or-fewer consecutive key
// channels of it in registers, and the two dot products are added over the R lanes with shuffles.  A workgroup
// takes (lane of the step, head, a run of columns) and walks the lane's tokens in order; the per-token vectors
// (q, k, and for the delta rule w, u, a*u) are laid in LDS for a stage of tokens at a time by the waves of the
// workgroup, one token a wave at a time, and read from there by every column.  R and the order of every sum depend
// on dk alone, so a token's result is the same bits however the step is cut and whatever else it holds.
#include "common.h"

#define LS_MAX_PER_LANE 16          // key channels of a column that one lane keeps
#define LS_THREADS 256
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
  int R, per_lane, columns, stage;  // lanes a column, key channels a lane, columns a workgroup, tokens a stage
};

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

// sum over the R neighbouring lanes of a column (R a power of two up to 64)
__device__ __forceinline__ float column_sum(float v, int R) {
  for (int offset = R >> 1; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, WAVE);
  return v;
}

template <typename T, bool DELTA>
__global__ void __launch_bounds__(LS_THREADS)
linear_state_scan_kernel(const ScanArgs a) {
  extern __shared__ __align__(16) float stage_lds[];
  const int lane_of_step = blockIdx.x;
  const int head = blockIdx.y;
  const int first_token = a.cu_seqlens[lane_of_step];
  const int end_token = a.cu_seqlens[lane_of_step + 1];
  if (end_token <= first_token) return;
  const int tid = threadIdx.x;
  const int wave = tid / WAVE;
  const int lane = tid & (WAVE - 1);
  const int waves = blockDim.x / WAVE;
  const int R = a.R, per_lane = a.per_lane;
  const int dk = a.dk, dv = a.dv;
  const int padded = R * per_lane;                       // a vector's length in LDS; channels past dk hold zeros
  const int vectors = DELTA ? 5 : 2;
  const int token_floats = vectors * padded + a.columns;
  const int column_in_group = tid / R;
  const int sub = tid - column_in_group * R;
  const int column = blockIdx.z * a.columns + column_in_group;
  const bool mine = column_in_group < a.columns && column < dv;
  const int channel0 = sub * per_lane;
  const T* rows = (const T*)a.u;

  // the column's share of the state
  float s[LS_MAX_PER_LANE];
  float* state_column = a.state + (((long)a.slot_ids[lane_of_step] * a.H + head) * dv + (mine ? column : 0)) * dk;
#pragma unroll
  for (int e = 0; e < LS_MAX_PER_LANE; ++e) {
    const int channel = channel0 + e;
    s[e] = (mine && e < per_lane && channel < dk) ? state_column[channel] : 0.f;
  }
  const float decay = DELTA ? 0.f : a.head_decay[head];
  const int half = a.rotary_dim / 2;

  for (int stage_first = first_token; stage_first < end_token; stage_first += a.stage) {
    const int count = min(a.stage, end_token - stage_first);
    __syncthreads();                                       // the stage before is read
    // ---- lay the stage's vectors in LDS: a wave a token
    for (int tt = wave; tt < count; tt += waves) {
      const long token = stage_first + tt;
      const T* row = rows + token * a.ld;
      float* q_lds = stage_lds + tt * token_floats;
      float* k_lds = q_lds + padded;
      float sum_squares = 0.f;
      float position = 0.f;
      if (!DELTA && a.inv_freq) position = (float)a.positions[token];
      for (int channel = lane; channel < padded; channel += WAVE) {
        float qx = 0.f, kx = 0.f;
        if (channel < dk) {
          qx = to_float(row[a.q_col + head * dk + channel]);
          kx = to_float(row[a.k_col + head * dk + channel]);
          if (!DELTA) {
            if (a.inv_freq && channel < a.rotary_dim) {
              const bool low = channel < half;
              const int pair = low ? channel + half : channel - half;
              const float angle = position * a.inv_freq[low ? channel : channel - half];
              const float sine = sinf(angle), cosine = cosf(angle);
              const float q_pair = to_float(row[a.q_col + head * dk + pair]);
              const float k_pair = to_float(row[a.k_col + head * dk + pair]);
              // (x, y) -> (x cos - y sin, y cos + x sin): the low half is x, the high half y
              qx = low ? qx * cosine - q_pair * sine : qx * cosine + q_pair * sine;
              kx = low ? kx * cosine - k_pair * sine : kx * cosine + k_pair * sine;
            }
            kx *= a.key_scale;
          }
        }
        q_lds[channel] = qx;
        k_lds[channel] = kx;
        sum_squares += kx * kx;
      }
      if (DELTA) {
        float* w_lds = k_lds + padded;
        float* u_lds = w_lds + padded;
        float* au_lds = u_lds + padded;
        const float length = sqrtf(wave_sum(sum_squares) + a.key_eps);
        const float* logits = a.decay_logits + token * a.logits_ld + head * dk;
        for (int channel = lane; channel < padded; channel += WAVE) {
          float w = 0.f, unit = 0.f, removed = 0.f;
          if (channel < dk) {
            unit = k_lds[channel] / length;
            removed = sigmoid_f(to_float(row[a.removal_col + head * dk + channel])) * unit;
            w = expf(-a.decay_floor * sigmoid_f(logits[channel] + a.decay_bias[head * dk + channel]));
          }
          w_lds[channel] = w;
          u_lds[channel] = unit;
          au_lds[channel] = removed;
        }
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
    __syncthreads();
    // ---- the tokens of the stage in order
    if (column_in_group < a.columns) {
      for (int tt = 0; tt < count; ++tt) {
        const float* q_lds = stage_lds + tt * token_floats + channel0;
        const float* k_lds = q_lds + padded;
        const float value = stage_lds[tt * token_floats + vectors * padded + column_in_group];
        float result = 0.f;
        if (DELTA) {
          const float* w_lds = k_lds + padded;
          const float* u_lds = w_lds + padded;
          const float* au_lds = u_lds + padded;
          float along = 0.f;
#pragma unroll
          for (int e = 0; e < LS_MAX_PER_LANE; ++e)
            if (e < per_lane) along = fmaf(u_lds[e], s[e], along);
          along = column_sum(along, R);
#pragma unroll
          for (int e = 0; e < LS_MAX_PER_LANE; ++e)
            if (e < per_lane) {
              s[e] = fmaf(k_lds[e], value, fmaf(-au_lds[e], along, w_lds[e] * s[e]));
              result = fmaf(s[e], q_lds[e], result);
            }
        } else {
#pragma unroll
          for (int e = 0; e < LS_MAX_PER_LANE; ++e)
            if (e < per_lane) {
              s[e] = fmaf(k_lds[e], value, decay * s[e]);
              result = fmaf(s[e], q_lds[e], result);
            }
        }
        result = column_sum(result, R);
        if (mine && sub == 0) a.out[(long)(stage_first + tt) * a.out_ld + head * dv + column] = result;
      }
    }
  }
  if (mine) {
#pragma unroll
    for (int e = 0; e < LS_MAX_PER_LANE; ++e) {
      const int channel = channel0 + e;
      if (e < per_lane && channel < dk) state_column[channel] = s[e];
    }
  }
}

// How a head's state is dealt out: R lanes a column (the smallest power of two that leaves a lane at most
// LS_MAX_PER_LANE key channels), per_lane = ceil(dk / R) channels a lane, LS_THREADS / R columns a workgroup of a
// prompt portion (one wave's worth, 64 / R, for steps of single tokens, which want many small workgroups).
extern "C" int mi_linear_state_scan(const void* u, int dtype, long ld, int q_col, int k_col, int v_col, int removal_col,
                                    int H, int dk, int dv, float* state, const int* cu_seqlens, const int* slot_ids,
                                    int lanes, float* out, long out_ld, int max_query_len, const float* head_decay,
                                    float key_scale, const int* positions, const float* inv_freq, int rotary_dim,
                                    const float* decay_logits, long logits_ld, const float* decay_bias,
                                    float decay_floor, float key_eps, hipStream_t stream) {
  if (!u || !state || !cu_seqlens || !slot_ids || !out || lanes <= 0 || H <= 0 || dk <= 0 || dv <= 0)
    return ERR_BAD_ARGUMENT;
  const bool delta = removal_col >= 0;
  if (delta && (!decay_logits || !decay_bias || logits_ld < (long)H * dk)) return ERR_BAD_ARGUMENT;
  if (!delta && !head_decay) return ERR_BAD_ARGUMENT;
  if (inv_freq && (!positions || rotary_dim <= 0 || rotary_dim > dk || (rotary_dim & 1))) return ERR_BAD_ARGUMENT;
  if (out_ld < (long)H * dv) return ERR_BAD_ARGUMENT;
  if (dk > LS_MAX_PER_LANE * WAVE || H > 65535 || lanes > 0x7fffffff) return ERR_UNSUPPORTED_SIZE;
  ScanArgs a;
  a.u = u; a.ld = ld; a.q_col = q_col; a.k_col = k_col; a.v_col = v_col; a.removal_col = removal_col;
  a.H = H; a.dk = dk; a.dv = dv; a.state = state; a.cu_seqlens = cu_seqlens; a.slot_ids = slot_ids;
  a.out = out; a.out_ld = out_ld; a.head_decay = head_decay; a.key_scale = key_scale; a.positions = positions;
  a.inv_freq = inv_freq; a.rotary_dim = inv_freq ? rotary_dim : 0; a.decay_logits = decay_logits;
  a.logits_ld = logits_ld; a.decay_bias = decay_bias; a.decay_floor = decay_floor; a.key_eps = key_eps;
  int R = 1;
  while (R * LS_MAX_PER_LANE < dk) R *= 2;
  a.R = R;
  a.per_lane = (dk + R - 1) / R;
  const int threads = max_query_len == 1 ? WAVE : LS_THREADS;
  a.columns = threads / R;
  if (a.columns > dv) a.columns = dv;
  const int splits = (dv + a.columns - 1) / a.columns;
  if (splits > 65535) return ERR_UNSUPPORTED_SIZE;
  const int token_floats = (delta ? 5 : 2) * R * a.per_lane + a.columns;
  int stage = LS_STAGE_BYTES / (token_floats * (int)sizeof(float));
  if (stage > LS_STAGE_MOST) stage = LS_STAGE_MOST;
  if (max_query_len > 0 && stage > max_query_len) stage = max_query_len;
  if (stage < 1) return ERR_UNSUPPORTED_SIZE;
  a.stage = stage;
  const size_t lds = (size_t)stage * token_floats * sizeof(float);
  const dim3 grid(lanes, H, splits);
#define LAUNCH(T_, DELTA_) linear_state_scan_kernel<T_, DELTA_><<<grid, threads, lds, stream>>>(a)
  if (dtype == DT_F32) { if (delta) LAUNCH(float, true); else LAUNCH(float, false); }
  else if (dtype == DT_BF16) { if (delta) LAUNCH(bf16_t, true); else LAUNCH(bf16_t, false); }
  else return ERR_BAD_ARGUMENT;
#undef LAUNCH
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
