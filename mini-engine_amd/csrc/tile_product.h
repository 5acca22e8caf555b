// A small tiled product for rows that are gathered, strided or grouped: 16 rows of x times 64 rows of a weight
// W [n, k] (row-major, as every weight is stored), float32 sums, by a block of 256 threads. Thread (tx, ty) = (tid % 64,
// tid / 64) owns column tx of the tile and rows ty, ty + 4, ty + 8, ty + 12. k is walked in steps of 32 through LDS;
// a row's sum is added up in ascending k whatever else the tile holds, so a row gives the same bits in any tile.
#pragma once

#include "common.h"

#define TP_ROWS 16
#define TP_COLS 64
#define TP_K 32

struct TileLds {
  float xs[TP_ROWS][TP_K + 1];
  float ws[TP_COLS][TP_K + 1];
};

// row_ptr(i): the k elements of row i < rows (storage type T). W points at the tile's first weight row; cols of them exist.
template <typename T, typename RowPtr>
__device__ __forceinline__ void tile_product(RowPtr row_ptr, int rows, const T* __restrict__ W, int cols, int k, float (&acc)[4],
                                             TileLds& lds) {
  const int tid = threadIdx.x, tx = tid & 63, ty = tid >> 6;
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = 0.f;
  const T* xrow[2];
  int xr[2], xk[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int idx = tid + 256 * u;
    xr[u] = idx / TP_K, xk[u] = idx % TP_K;
    xrow[u] = xr[u] < rows ? row_ptr(xr[u]) : nullptr;
  }
  for (int kc = 0; kc < k; kc += TP_K) {
#pragma unroll
    for (int u = 0; u < 2; ++u)
      lds.xs[xr[u]][xk[u]] = xrow[u] && kc + xk[u] < k ? to_float(xrow[u][kc + xk[u]]) : 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int idx = tid + 256 * u, c = idx / TP_K, kk = idx % TP_K;
      lds.ws[c][kk] = c < cols && kc + kk < k ? to_float(W[(size_t)c * k + kc + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TP_K; ++kk) {
      const float w = lds.ws[tx][kk];
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = fmaf(lds.xs[ty + 4 * i][kk], w, acc[i]);
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------------------------------------------------
// The same product on the matrix cores, bfloat16 operands and float32 sums: 16 * MT rows of x times ACCS tiles of 16 weight
// rows, by one wave, with v_mfma_f32_16x16x32_bf16 in the transposed arrangement (C^T[n, m] = sum_k W[n, k] X[m, k]): lane l
// feeds W[n0 + l % 16][k + 8 (l / 16) ..] and X[m0 + l % 16][k + 8 (l / 16) ..], eight elements (16 bytes) each, straight
// from memory, and receives C[m0 + l % 16][n0 + 4 (l / 16) .. + 4]. k is a multiple of 8 and every row starts at a multiple of
// 16 bytes (the callers check). Rows do not meet in the arithmetic: a row's sums are the same bits in any tile.
typedef __bf16 tp_bf16x8 __attribute__((ext_vector_type(8)));
typedef float tp_float4 __attribute__((ext_vector_type(4)));

// xrow[t]: the row of x that this lane feeds in row tile t (or null: zeros); wrow[a]: its weight row in tile a (or null).
template <int MT, int ACCS>
__device__ __forceinline__ void wave_product_bf16(const bf16_t* const (&xrow)[MT], const bf16_t* const (&wrow)[ACCS], int k,
                                                  tp_float4 (&acc)[MT][ACCS]) {
  const int g = (threadIdx.x & 63) >> 4;
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int a = 0; a < ACCS; ++a) acc[t][a] = (tp_float4){0.f, 0.f, 0.f, 0.f};
  constexpr int U = 2;  // chunks of 32 whose loads are asked for together
  for (int k0 = 0; k0 < k; k0 += 32 * U) {
    tp_bf16x8 wf[U][ACCS], xf[U][MT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int at = k0 + 32 * u + 8 * g;
#pragma unroll
      for (int a = 0; a < ACCS; ++a) {
        wf[u][a] = tp_bf16x8{};
        if (wrow[a] && at < k) wf[u][a] = *reinterpret_cast<const tp_bf16x8*>(wrow[a] + at);
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        xf[u][t] = tp_bf16x8{};
        if (xrow[t] && at < k) xf[u][t] = *reinterpret_cast<const tp_bf16x8*>(xrow[t] + at);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int a = 0; a < ACCS; ++a) acc[t][a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][a], xf[u][t], acc[t][a], 0, 0, 0);
  }
}
