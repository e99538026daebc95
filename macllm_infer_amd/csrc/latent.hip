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
  if (!down || !q_norm || !kv_norm || !positions || !q_latent || T <= 0 || q_rank <= 0 || kv_rank <= 0 || rope_dim < 0 ||
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
