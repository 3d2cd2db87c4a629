// A plain tile product for the kernels whose matrices are picked per head or per expert:
// a workgroup of 256 threads computes 32 rows x 64 columns of a x w^T, K in steps of 32
// through LDS, every sum in 32-bit in the order of k.  A row's sums depend on nothing but
// that row and the weights, so a row gives the same result wherever it lies in a batch.
#pragma once
#include "common.h"

#define SG_ROWS 32
#define SG_COLS 64
#define SG_K 32

struct SmallTileSums {
    float v[2][4];      // rows (ty, ty + 16), columns tx + 16 * j
};

// a: rows of the tile [rows_valid, K] with row stride lda; w: [cols_valid, K] with row stride ldw
template <typename TA, typename TW>
__device__ __forceinline__ void small_tile_product(const TA* __restrict__ a, long long lda, int rows_valid,
                                                   const TW* __restrict__ w, long long ldw, int cols_valid, int K,
                                                   float (*as)[SG_K + 1], float (*ws)[SG_K + 1], SmallTileSums& sums) {
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) sums.v[i][j] = 0.f;
    for (int k0 = 0; k0 < K; k0 += SG_K) {
        for (int i = tid; i < SG_ROWS * SG_K; i += 256) {
            const int r = i / SG_K, k = i - r * SG_K;
            as[r][k] = (r < rows_valid && k0 + k < K) ? to_float(a[static_cast<size_t>(r) * lda + k0 + k]) : 0.f;
        }
        for (int i = tid; i < SG_COLS * SG_K; i += 256) {
            const int c = i / SG_K, k = i - c * SG_K;
            ws[c][k] = (c < cols_valid && k0 + k < K) ? to_float(w[static_cast<size_t>(c) * ldw + k0 + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int k = 0; k < SG_K; ++k) {
            const float a0 = as[ty][k], a1 = as[ty + 16][k];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float b = ws[tx + 16 * j][k];
                sums.v[0][j] = fmaf(a0, b, sums.v[0][j]);
                sums.v[1][j] = fmaf(a1, b, sums.v[1][j]);
            }
        }
        __syncthreads();
    }
}
