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
