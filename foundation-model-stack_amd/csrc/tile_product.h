// A block's tile of C = A W^T for rows that are found through functions: the rows of A may be gathered (tokens
// sorted by expert), strided (one head of every token) or plain; the rows of W are K contiguous elements each.
//
//   tile_product_fma:  256 threads, 16 rows x 64 columns, any element type, any K, float32 FMA (the true 32-bit
//                      path, and the path for rows that are not 16-byte aligned).
//   tile_product_mfma: 256 threads = 4 waves, 16 rows x 128 columns (a wave: 32 columns as two 16x16 tiles),
//                      bfloat16 operands loaded straight from global memory into the operand layout of the
//                      16x16x32 matrix instruction (a lane holds 8 consecutive k of one row); K a multiple of 8
//                      and rows aligned to 16 bytes.  The weights stream through once: four steps of K are asked
//                      for before the first is multiplied, so that a wave keeps a dozen loads in flight.
//
//   tile_product_mfma_wide: the same for 64 rows x 128 columns, a wave 32 rows x 64 columns (2 x 4 tiles): eight
//                      products for six loads instead of two for three, for steps of many rows (prompts), whose
//                      products are bound by what the caches deliver.
//
// a_row(m), m < 16 (64 for the wide tile), and w_row(n) return the row's first element or nullptr for a row that is not there (zeros).
#pragma once

#include "common.h"

#define TILE_ROWS 16
#define TILE_FMA_COLS 64
#define TILE_MFMA_COLS 128
#define TILE_MFMA_WAVE_TILES 2  // 16-column tiles a wave
#define TILE_THREADS 256

// After the call, thread tid holds acc[i] = C[row (tid / 64) * 4 + i][column tid % 64].
template <typename T, typename ARow, typename WRow>
__device__ __forceinline__ void tile_product_fma(ARow a_row, WRow w_row, int K, float (&acc)[4]) {
  constexpr int BK = 32;
  __shared__ float As[TILE_ROWS][BK + 1];
  __shared__ float Ws[TILE_FMA_COLS][BK + 1];
  const int tid = threadIdx.x;
  const int n = tid % 64, mg = tid / 64;
  const int lk = tid % BK, lr = tid / BK;  // loads: element lk of rows lr, lr + 8, ...
  const T* arow[2];
  const T* wrow[8];
#pragma unroll
  for (int i = 0; i < 2; ++i) arow[i] = a_row(lr + 8 * i);
#pragma unroll
  for (int i = 0; i < 8; ++i) wrow[i] = w_row(lr + 8 * i);
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = 0.f;
  for (int k0 = 0; k0 < K; k0 += BK) {
    const bool in = k0 + lk < K;
#pragma unroll
    for (int i = 0; i < 2; ++i) As[lr + 8 * i][lk] = (in && arow[i]) ? to_f32(arow[i][k0 + lk]) : 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) Ws[lr + 8 * i][lk] = (in && wrow[i]) ? to_f32(wrow[i][k0 + lk]) : 0.f;
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      const float w = Ws[n][k];
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = fmaf(As[mg * 4 + i][k], w, acc[i]);
    }
    __syncthreads();
  }
}

// After the call, lane l of wave w holds acc[t][i] = C[row (l / 16) * 4 + i][column w * 32 + t * 16 + l % 16].
// w_row(n) takes n < 128, the column inside the block's tile.
template <typename ARow, typename WRow>
__device__ __forceinline__ void tile_product_mfma(ARow a_row, WRow w_row, int K, f32x4 (&acc)[TILE_MFMA_WAVE_TILES]) {
  constexpr int NT = TILE_MFMA_WAVE_TILES, AHEAD = 4;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, kq = (lane >> 4) * 8;
  const bf16* a = a_row(r);
  const bf16* w[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    w[t] = w_row(wave * (16 * NT) + t * 16 + r);
    acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int k0 = 0; k0 < K; k0 += 32 * AHEAD) {
    bf16x8 av[AHEAD], wv[AHEAD][NT];
#pragma unroll
    for (int s = 0; s < AHEAD; ++s) {
      const int k = k0 + 32 * s + kq;
      const bool in = k < K;
      av[s] = (in && a) ? *reinterpret_cast<const bf16x8*>(a + k) : zero;
#pragma unroll
      for (int t = 0; t < NT; ++t) wv[s][t] = (in && w[t]) ? *reinterpret_cast<const bf16x8*>(w[t] + k) : zero;
    }
#pragma unroll
    for (int s = 0; s < AHEAD; ++s) {
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[s], wv[s][t], acc[t], 0, 0, 0);
    }
  }
}

#define TILE_WIDE_ROWS 64
// After the call, lane l of wave w holds
//   acc[mt][nt][i] = C[row (w / 2) * 32 + mt * 16 + (l / 16) * 4 + i][column (w % 2) * 64 + nt * 16 + l % 16].
template <typename ARow, typename WRow>
__device__ __forceinline__ void tile_product_mfma_wide(ARow a_row, WRow w_row, int K, f32x4 (&acc)[2][4]) {
  constexpr int AHEAD = 2;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, kq = (lane >> 4) * 8;
  const bf16* a[2];
  const bf16* w[4];
#pragma unroll
  for (int mt = 0; mt < 2; ++mt) a[mt] = a_row((wave >> 1) * 32 + mt * 16 + r);
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) w[nt] = w_row((wave & 1) * 64 + nt * 16 + r);
#pragma unroll
  for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int k0 = 0; k0 < K; k0 += 32 * AHEAD) {
    bf16x8 av[AHEAD][2], wv[AHEAD][4];
#pragma unroll
    for (int s = 0; s < AHEAD; ++s) {
      const int k = k0 + 32 * s + kq;
      const bool in = k < K;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) av[s][mt] = (in && a[mt]) ? *reinterpret_cast<const bf16x8*>(a[mt] + k) : zero;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) wv[s][nt] = (in && w[nt]) ? *reinterpret_cast<const bf16x8*>(w[nt] + k) : zero;
    }
#pragma unroll
    for (int s = 0; s < AHEAD; ++s) {
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[s][mt], wv[s][nt], acc[mt][nt], 0, 0, 0);
      }
    }
  }
}
