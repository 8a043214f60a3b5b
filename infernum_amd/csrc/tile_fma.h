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

// The fp32 tile, handed to `emit(row of the tile, first of four consecutive columns, the four sums)`.
template <typename T, typename Emit>
__device__ __forceinline__ void tile_64(const T* __restrict__ a_row, const T* __restrict__ w_row, int K,
                                        TileFmaLds& lds, Emit emit) {
  float acc[4][4];
  tile_fma_64(a_row, w_row, K, acc, lds);
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) emit(ty * 4 + i, tx * 4, acc[i]);
}

// Whether rows that start at `p` and lie `stride` elements apart (and `stride2` for a second index) can be read
// 16 bytes at a time.
__host__ __device__ inline bool tile_rows_aligned(const void* p, long stride, long stride2 = 0) {
  return (reinterpret_cast<uintptr_t>(p) & 15) == 0 && (stride & 7) == 0 && (stride2 & 7) == 0;
}

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 tm_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float tm_f32x4;

// ---- a larger tile on the matrix cores: BM rows of A (128, or 32 for steps of few rows) x 128 rows of W ------------
// 256 threads = 4 waves, 2 x 2 over the tile at BM = 128 (64 x 64 a wave: 4 x 4 accumulators) and 1 x 4 at BM = 32
// (32 x 32 a wave).  K is walked in steps of 64 through one LDS stage; the global loads run two steps ahead of the
// matrix instructions in two sets of registers (the loads of step i + 2 are issued before the matrix instructions
// of step i and stored to LDS after those of step i + 1), every load unconditional so that a wait for the older
// set leaves the newer in flight: a row that the tile does not have is read from the tile's first row (its sums
// are never handed on), and values of k past K are read from the row's end and set to zero by a select.
// v_mfma_f32_16x16x32_bf16 with 16 rows of W as its first operand and 16 rows of A as its second: lane
// (r = lane % 16, q = lane / 16) ends with D[column 4 q + e of W's 16][row r of A's 16], e = 0..3, so a lane holds
// four consecutive columns of one row of the result, as a thread of the fp32 tile above does.  Every element is
// summed in an order that depends on K alone.
// `a_row(r)` / `w_row(r)`: row r of the tile's A / W (16-byte aligned, K a multiple of 8 and at least 8); row 0
// always exists.
#define TB_KS 64
#define TB_LD 72
#define TB_N 128

// BN = 256 (with BM = 128): eight waves, 2 x 4 over the tile, for products of many rows: the rows of A are read
// once for twice the columns (85 flops a byte read into LDS where 128 x 128 has 64).
template <int BM, int BN = TB_N>
struct TileBigLds {
  uint16_t a[BM][TB_LD];
  uint16_t w[BN][TB_LD];
};

template <int BM, int BN>
constexpr int tile_big_threads() { return BN == 256 ? 512 : 256; }

template <int BM, int BN = TB_N, typename ARow, typename WRow, typename Emit>
__device__ __forceinline__ void tile_mfma_big(ARow a_row, WRow w_row, int a_rows, int w_rows, int K,
                                              TileBigLds<BM, BN>& lds, Emit emit) {
  static_assert((BM == 128 || BM == 32) && (BN == 128 || (BN == 256 && BM == 128)), "tiles of 128 x 128, 32 x 128, 128 x 256");
  constexpr int WAVES = tile_big_threads<BM, BN>() / 64;
  constexpr int WM = BM == 128 ? 2 : 1, WN = WAVES / WM;       // waves along the rows and the columns
  constexpr int MT = BM / WM / 16, NT = BN / WN / 16;         // 16 x 16 tiles a wave
  constexpr int RP = WAVES * 8;                               // rows that the workgroup's threads read in one pass
  constexpr int AR = BM / RP, WR = BN / RP;                   // rows of A and of W that a thread loads a step
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, q = lane >> 4;
  const int wm0 = (wave / WN) * (BM / WM), wn0 = (wave % WN) * (BN / WN);
  const int lr = tid >> 3, lk = (tid & 7) * 8;                // 8 threads read a row's 64 values of k
  const bf16_t* ap[AR];
  const bf16_t* wp[WR];
#pragma unroll
  for (int s = 0; s < AR; ++s) ap[s] = a_row(lr + RP * s < a_rows ? lr + RP * s : 0);
#pragma unroll
  for (int s = 0; s < WR; ++s) wp[s] = w_row(lr + RP * s < w_rows ? lr + RP * s : 0);
  tm_f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = tm_f32x4{0.f, 0.f, 0.f, 0.f};
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
  uint4 ra[2][AR], rw[2][WR];
  auto fetch = [&](int k0, uint4 (&xa)[AR], uint4 (&xw)[WR]) {
    const int k = k0 + lk;
    const int kc = k < K ? k : K - 8;                          // stays inside the row
#pragma unroll
    for (int s = 0; s < AR; ++s) xa[s] = *reinterpret_cast<const uint4*>(ap[s] + kc);
#pragma unroll
    for (int s = 0; s < WR; ++s) xw[s] = *reinterpret_cast<const uint4*>(wp[s] + kc);
    if (k >= K) {
#pragma unroll
      for (int s = 0; s < AR; ++s) xa[s] = zero;
#pragma unroll
      for (int s = 0; s < WR; ++s) xw[s] = zero;
    }
  };
  auto stage = [&](const uint4 (&xa)[AR], const uint4 (&xw)[WR]) {
#pragma unroll
    for (int s = 0; s < AR; ++s) *reinterpret_cast<uint4*>(&lds.a[lr + RP * s][lk]) = xa[s];
#pragma unroll
    for (int s = 0; s < WR; ++s) *reinterpret_cast<uint4*>(&lds.w[lr + RP * s][lk]) = xw[s];
  };
  auto multiply = [&]() {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      uint4 wf[NT];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) wf[nt] = *reinterpret_cast<const uint4*>(&lds.w[wn0 + 16 * nt + r][q * 8 + 32 * h]);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const uint4 af = *reinterpret_cast<const uint4*>(&lds.a[wm0 + 16 * mt + r][q * 8 + 32 * h]);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(tm_bf16x8, wf[nt]),
                                                                __builtin_bit_cast(tm_bf16x8, af), acc[mt][nt], 0, 0, 0);
      }
    }
  };
  const int steps = (K + TB_KS - 1) / TB_KS;
  fetch(0, ra[0], rw[0]);
  fetch(TB_KS, ra[1], rw[1]);                                  // past K: zeros
  stage(ra[0], rw[0]);
  __syncthreads();
  for (int i = 0; i < steps; i += 2) {
    // step i: LDS holds it; set 0 is free for step i + 2, set 1 holds step i + 1
    fetch((i + 2) * TB_KS, ra[0], rw[0]);
    multiply();
    __syncthreads();
    if (i + 1 >= steps) break;
    stage(ra[1], rw[1]);
    __syncthreads();
    // step i + 1
    fetch((i + 3) * TB_KS, ra[1], rw[1]);
    multiply();
    __syncthreads();
    if (i + 2 >= steps) break;
    stage(ra[0], rw[0]);
    __syncthreads();
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const float v[4] = {acc[mt][nt][0], acc[mt][nt][1], acc[mt][nt][2], acc[mt][nt][3]};
      emit(wm0 + 16 * mt + r, wn0 + 16 * nt + 4 * q, v);
    }
}
