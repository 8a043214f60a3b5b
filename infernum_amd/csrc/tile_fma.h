// A 64 x 64 tile of C = A W^T on the vector ALUs with fp32 multiply-adds in the fixed three-level order of
// gemm_generic.hip (a chain of 16 from zero, 16 such chains, those sums in the order of k), for kernels whose
// rows of A are found through an index (gathered tokens, a head's stretch of a row): every output element is one
// chain of operations that depends on its own row of A and row of W alone, never on the rows beside it or on
// the tile it falls into.
#pragma once
#include "common.h"

#define TF_T 64   // tile of C: TF_T x TF_T
#define TF_K 16   // depth of one LDS stage

struct TileFmaLds {
  float a[TF_K][TF_T + 4];
  float w[TF_K][TF_T + 4];
};

// `a_row`: this thread's row of A (row tid >> 2 of the tile), or nullptr for a row that does not exist.
// `w_row`: its row of W (the same index), or nullptr.  256 threads; thread (ty = tid >> 4, tx = tid & 15) ends
// with rows ty*4 .. ty*4+3 and columns tx*4 .. tx*4+3 of the tile in acc.
template <typename TA, typename TW>
__device__ __forceinline__ void tile_fma_64(const TA* __restrict__ a_row, const TW* __restrict__ w_row, int K,
                                            float (&acc)[4][4], TileFmaLds& lds) {
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int lr = tid >> 2;
  const int lk = (tid & 3) * 4;
  float mid[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = mid[i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += TF_K) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = k0 + lk + e;
      lds.a[lk + e][lr] = (a_row && k < K) ? to_float(a_row[k]) : 0.f;
      lds.w[lk + e][lr] = (w_row && k < K) ? to_float(w_row[k]) : 0.f;
    }
    __syncthreads();
    float part[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) part[i][j] = 0.f;
#pragma unroll
    for (int kk = 0; kk < TF_K; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = lds.a[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = lds.w[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) part[i][j] = fmaf(a[i], b[j], part[i][j]);
    }
    const bool close = ((k0 / TF_K) & 15) == 15 || k0 + TF_K >= K;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        mid[i][j] += part[i][j];
        if (close) {
          acc[i][j] += mid[i][j];
          mid[i][j] = 0.f;
        }
      }
    __syncthreads();
  }
}
