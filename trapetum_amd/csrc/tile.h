// A plain tiled product for kernels whose operands are gathered or strided: a block of 256 threads forms a
// TM x TN tile of A . W^T with fp32 accumulation, operands staged through LDS in steps of BK, one fixed order of
// additions per output element.  The callers supply the loads: la(m, k) and lw(n, k) return element (m, k) of the
// tile's rows of A and element (n, k) of its rows of W as float, zero outside the operand.
#pragma once
#include "common.h"

template <int TM, int TN, int BK>
struct TileShared {
    float a[BK][TM + 1];
    float w[BK][TN + 1];
};

// thread t: rows t / 16 + 16 i, columns t % 16 + 16 j
template <int TM, int TN, int BK, typename LoadA, typename LoadW>
__device__ __forceinline__ void tile_product(float (&acc)[TM / 16][TN / 16], int K, LoadA la, LoadW lw, TileShared<TM, TN, BK>& sh) {
    const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
#pragma unroll
    for (int i = 0; i < TM / 16; i++)
#pragma unroll
        for (int j = 0; j < TN / 16; j++) acc[i][j] = 0.f;
    for (int k0 = 0; k0 < K; k0 += BK) {
        for (int idx = tid; idx < TM * BK; idx += 256) {
            const int m = idx / BK, k = idx - m * BK;
            sh.a[k][m] = k0 + k < K ? la(m, k0 + k) : 0.f;
        }
        for (int idx = tid; idx < TN * BK; idx += 256) {
            const int n = idx / BK, k = idx - n * BK;
            sh.w[k][n] = k0 + k < K ? lw(n, k0 + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; k++) {
            float av[TM / 16], wv[TN / 16];
#pragma unroll
            for (int i = 0; i < TM / 16; i++) av[i] = sh.a[k][ty + 16 * i];
#pragma unroll
            for (int j = 0; j < TN / 16; j++) wv[j] = sh.w[k][tx + 16 * j];
#pragma unroll
            for (int i = 0; i < TM / 16; i++)
#pragma unroll
                for (int j = 0; j < TN / 16; j++) acc[i][j] = __builtin_fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
}
