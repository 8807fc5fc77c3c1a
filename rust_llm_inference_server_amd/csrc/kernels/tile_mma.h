// One wave's tile of a product on the matrix cores, for operands whose rows are contiguous
// along k: C[i][n] = sum_k A[i][k] * B[n][k] for 16 rows of A and NB blocks of 16 rows of B.
//
// Every lane loads straight into operand layout from the two rows it serves (row lane % 16 of
// A, row lane % 16 of each block of B; the k chunk lane / 16), so rows may be gathered: the
// caller hands each lane its own row pointers.  Rows past an operand's end are given a pointer
// that exists (the caller clamps) and their results are masked at the store.
//
//  * bfloat16: v_mfma_f32_16x16x32_bf16, 8 consecutive k per lane and step of 32.
//  * float32:  v_mfma_f32_16x16x4_f32 (a true 32-bit multiply-add, no reduced mode): a lane
//    loads 4 consecutive k per step of 16 and feeds them to four products; product i of a step
//    sums k = 4 g + i over the lane groups g, the same assignment on both operands.
//
// The result of block b is acc[b]: lane l holds column l % 16 (a row of B) of rows
// 4 (l / 16) + 0..3 (rows of A).  The order of the sums over k is fixed by K alone.
#pragma once
#include "common.h"

typedef __bf16 mma_bf16x8 __attribute__((ext_vector_type(8)));
typedef float mma_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t mma_u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct MmaChunk;
template <> struct MmaChunk<bf16_t> { static constexpr int kLane = 8, kStep = 32; };
template <> struct MmaChunk<float> { static constexpr int kLane = 4, kStep = 16; };

// A lane's chunk of a row: kLane elements from k on, zeros past K.  ALIGNED: the row starts on
// a 16-byte boundary and K is a multiple of kLane, so a chunk is one 16-byte load or nothing.
template <typename T, bool ALIGNED>
__device__ __forceinline__ mma_u32x4 mma_load(const T* row, int k, int K) {
  constexpr int n = MmaChunk<T>::kLane;
  mma_u32x4 out = {0u, 0u, 0u, 0u};
  if (ALIGNED) {
    // (the address is clamped, the value chosen: no load stands under a condition)
    const mma_u32x4 v = *reinterpret_cast<const mma_u32x4*>(row + (k < K ? k : 0));
    if (k < K) out = v;
    return out;
  }
  T tmp[n];
#pragma unroll
  for (int i = 0; i < n; ++i) {
    const T v = row[k + i < K ? k + i : 0];
    tmp[i] = k + i < K ? v : (T)0;
  }
  return __builtin_bit_cast(mma_u32x4, tmp);
}

template <typename T, int NB, bool ALIGNED>
__device__ __forceinline__ void wave_tile_product(const T* a_row, const T* const (&b_row)[NB],
                                                  int K, mma_f32x4 (&acc)[NB]) {
  constexpr int kLane = MmaChunk<T>::kLane, kStep = MmaChunk<T>::kStep;
  const int g = (threadIdx.x % kWave) / 16;
#pragma unroll
  for (int b = 0; b < NB; ++b) acc[b] = mma_f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += kStep) {
    const int k = k0 + g * kLane;
    const mma_u32x4 a = mma_load<T, ALIGNED>(a_row, k, K);
    mma_u32x4 bv[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) bv[b] = mma_load<T, ALIGNED>(b_row[b], k, K);
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      if constexpr (sizeof(T) == 2) {
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mma_bf16x8, a),
                                                         __builtin_bit_cast(mma_bf16x8, bv[b]),
                                                         acc[b], 0, 0, 0);
      } else {
        const mma_f32x4 af = __builtin_bit_cast(mma_f32x4, a);
        const mma_f32x4 bf = __builtin_bit_cast(mma_f32x4, bv[b]);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[i], bf[i], acc[b], 0, 0, 0);
      }
    }
  }
}

// Whether rows that start at `base`, `stride` elements apart (and `inner` elements apart inside
// a row group, 0: none), with K columns, can take the 16-byte loads.
template <typename T>
static inline bool mma_rows_aligned(const void* base, long long stride, long long inner, int K) {
  constexpr int n = MmaChunk<T>::kLane;
  return ((uintptr_t)base % 16 == 0) && stride % n == 0 && inner % n == 0 && K % n == 0;
}

// The same with MB blocks of 16 rows of A: acc[a][b] is block a of A against block b of B.  Every
// fragment of B that is loaded serves MB products (and every fragment of A NB of them), which
// is what a product with many rows needs: loads, not the matrix cores, bound the tile above.
template <typename T, int MB, int NB, bool ALIGNED>
__device__ __forceinline__ void wave_tile_product_rows(const T* const (&a_row)[MB],
                                                       const T* const (&b_row)[NB], int K,
                                                       mma_f32x4 (&acc)[MB][NB]) {
  constexpr int kLane = MmaChunk<T>::kLane, kStep = MmaChunk<T>::kStep;
  const int g = (threadIdx.x % kWave) / 16;
#pragma unroll
  for (int a = 0; a < MB; ++a)
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[a][b] = mma_f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += kStep) {
    const int k = k0 + g * kLane;
    mma_u32x4 av[MB], bv[NB];
#pragma unroll
    for (int a = 0; a < MB; ++a) av[a] = mma_load<T, ALIGNED>(a_row[a], k, K);
#pragma unroll
    for (int b = 0; b < NB; ++b) bv[b] = mma_load<T, ALIGNED>(b_row[b], k, K);
#pragma unroll
    for (int a = 0; a < MB; ++a)
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        if constexpr (sizeof(T) == 2) {
          acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              __builtin_bit_cast(mma_bf16x8, av[a]), __builtin_bit_cast(mma_bf16x8, bv[b]),
              acc[a][b], 0, 0, 0);
        } else {
          const mma_f32x4 af = __builtin_bit_cast(mma_f32x4, av[a]);
          const mma_f32x4 bf = __builtin_bit_cast(mma_f32x4, bv[b]);
#pragma unroll
          for (int i = 0; i < 4; ++i)
            acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[i], bf[i], acc[a][b], 0, 0, 0);
        }
      }
  }
}
