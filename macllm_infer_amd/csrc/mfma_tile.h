// Tiles of a product out[row, feature] = sum_k x[row, k] * w[feature, k] on the matrix cores, for kernels whose
// rows or weights are found through a table (one product per head, rows grouped by expert): a workgroup of four
// waves owns NT tiles of 16 features and MT tiles of 16 rows, the waves split K into four contiguous runs of
// chunks, and their partial tiles are added through LDS in the order of the waves.  bfloat16 operands:
// v_mfma_f32_16x16x32_bf16, a chunk is 32 k; float32 operands: v_mfma_f32_16x16x4_f32 (products and sums in
// float32, no reduced-precision mode), a chunk is 16 k.  The order in which an element is summed depends on K
// alone, never on the rows beside it or on which tile a row stands in.
#pragma once
#include "common.h"

typedef float tile_floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 tile_bf16x8 __attribute__((ext_vector_type(8)));

#define TILE_WAVES 4
#define TILE_THREADS (TILE_WAVES * WAVE)

template <typename T> struct TileTraits;
template <> struct TileTraits<float> {
  static constexpr int CHUNK = 16;      // k of one round of a wave: four products of 4
  static constexpr int PIECE = 4;       // consecutive k a lane loads
  typedef tile_floatx4 Piece;
};
template <> struct TileTraits<bf16_t> {
  static constexpr int CHUNK = 32;
  static constexpr int PIECE = 8;
  typedef tile_bf16x8 Piece;
};

// PIECE consecutive k of one row from k on; a k at or past K gives zero.  VEC: one 16-byte load (K, the row's
// start and its stride are whole pieces); otherwise element by element.
template <typename T, bool VEC>
__device__ __forceinline__ typename TileTraits<T>::Piece tile_load(const T* row, int k, int K) {
  typedef typename TileTraits<T>::Piece Piece;
  constexpr int PIECE = TileTraits<T>::PIECE;
  Piece value;
  if (VEC) {
    value = *reinterpret_cast<const Piece*>(row + min(k, K - PIECE));
    if (k >= K) {
#pragma unroll
      for (int j = 0; j < PIECE; ++j) value[j] = (T)0.f;
    }
    return value;
  }
#pragma unroll
  for (int j = 0; j < PIECE; ++j) {
    const T element = row[min(k + j, K - 1)];
    value[j] = k + j < K ? element : (T)0.f;
  }
  return value;
}

__device__ __forceinline__ tile_floatx4 tile_mfma(const tile_floatx4& a, const tile_floatx4& b, tile_floatx4 acc) {
#pragma unroll
  for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], b[i], acc, 0, 0, 0);
  return acc;
}

__device__ __forceinline__ tile_floatx4 tile_mfma(const tile_bf16x8& a, const tile_bf16x8& b, tile_floatx4 acc) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
}

// This wave's share of the products: w_row[nt] / x_row[mt] point at the weight row / the row of x that this
// lane's column of the operands comes from (lane % 16), already clamped to valid rows.
template <typename T, int MT, int NT, bool VEC>
__device__ __forceinline__ void tile_accumulate(const T* const (&w_row)[NT], const T* const (&x_row)[MT], int K,
                                                tile_floatx4 (&acc)[NT][MT]) {
  typedef typename TileTraits<T>::Piece Piece;
  constexpr int CHUNK = TileTraits<T>::CHUNK;
  constexpr int PIECE = TileTraits<T>::PIECE;
  const int lane = threadIdx.x & (WAVE - 1);
  const int wave = threadIdx.x / WAVE;
  const int q = lane / 16;
  const int chunks = (K + CHUNK - 1) / CHUNK;
  const int per_wave = (chunks + TILE_WAVES - 1) / TILE_WAVES;
  const int first_chunk = wave * per_wave;
  const int iterations = max(0, min(per_wave, chunks - first_chunk));
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = tile_floatx4{0.f, 0.f, 0.f, 0.f};
  // two chunks are asked for before the first is used; a chunk past the wave's run reads as zeros
  for (int first = 0; first < iterations; first += 2) {
    Piece a[2][NT], b[2][MT];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int k = first + j < iterations ? (first_chunk + first + j) * CHUNK + PIECE * q : K;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) a[j][nt] = tile_load<T, VEC>(w_row[nt], k, K);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[j][mt] = tile_load<T, VEC>(x_row[mt], k, K);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = tile_mfma(a[j][nt], b[j][mt], acc[nt][mt]);
  }
}

// The sum of the four waves' partial tiles of one (nt, mt), in the order of the waves: thread tid gets element
// (feature 4 (l / 16) + i, row l % 16) with i = tid / 64, l = tid % 64.  `red` is LDS [TILE_WAVES][256]; the call
// has barriers, so every thread of the workgroup makes it.
__device__ __forceinline__ float tile_reduce(const tile_floatx4& acc, float (*red)[256]) {
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) red[wave][i * 64 + lane] = acc[i];
  __syncthreads();
  float value = red[0][tid];
#pragma unroll
  for (int w = 1; w < TILE_WAVES; ++w) value += red[w][tid];
  return value;
}
