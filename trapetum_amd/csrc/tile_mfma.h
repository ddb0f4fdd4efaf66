// The tiled product of tile.h on the matrix cores, for bf16 operands whose rows can be read in 16-byte pieces (K a
// multiple of 8, rows starting on 16 bytes): a block of 256 threads forms TM x 64 outputs of A . W^T (TM = 64: the
// four waves in a 2 x 2 arrangement, 32 x 32 each; TM = 16: the waves side by side, 16 x 16 each) with
// v_mfma_f32_16x16x32_bf16, fp32 accumulation.  GATED: the block stages 64 gate rows and the 64 up rows of the same
// units, and every lane ends up with a unit's gate and up sum in accumulators of the same index.
// K is walked in steps of 64 through one LDS buffer; the next step's pieces are asked for before the current step is
// multiplied and written to LDS after it.  The callers supply the loads: la8(m, k) and lw8(n, k) return the 8
// elements from k on of the tile's row m of A and row n of W (n < 128 when GATED: 64 gate rows, then 64 up rows),
// zeros outside the operand.
#pragma once
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 tm_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float tm_f32x4;

constexpr int TMF_BK = 64, TMF_ROW = TMF_BK + 8;      // elements of an LDS row: a step and 16 bytes that spread rows over the banks

template <int TM, bool GATED>
struct MfmaTile {
    static constexpr int WN = GATED ? 128 : 64;
    static constexpr int MI = TM == 64 ? 2 : 1, NJ = TM == 64 ? 2 : 1, SETS = GATED ? 2 : 1;
    static constexpr int A_PIECES = TM * 8 / 256 > 0 ? TM * 8 / 256 : 1, W_PIECES = WN * 8 / 256;
    struct Shared { bf16_t a[TM][TMF_ROW]; bf16_t w[WN][TMF_ROW]; };
    tm_f32x4 acc[SETS][MI][NJ];

    // where the lane's accumulators lie in the tile: row m_of(i) (lane's r), columns n_of(j) + v, v = 0 .. 3
    __device__ __forceinline__ static int wave_m() { return TM == 64 ? 32 * ((threadIdx.x >> 6) >> 1) : 0; }
    __device__ __forceinline__ static int wave_n() { return TM == 64 ? 32 * ((threadIdx.x >> 6) & 1) : 16 * (threadIdx.x >> 6); }
    __device__ __forceinline__ static int m_of(int i) { return wave_m() + 16 * i + (threadIdx.x & 15); }
    __device__ __forceinline__ static int n_of(int j) { return wave_n() + 16 * j + ((threadIdx.x & 63) >> 4) * 4; }

    template <typename LoadA, typename LoadW>
    __device__ __forceinline__ void run(int K, LoadA la8, LoadW lw8, Shared& sh) {
        const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, g = lane >> 4;
#pragma unroll
        for (int s = 0; s < SETS; s++)
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int j = 0; j < NJ; j++) acc[s][i][j] = tm_f32x4{0.f, 0.f, 0.f, 0.f};
        uint4 pa[A_PIECES], pw[W_PIECES];
        const uint4 zero = make_uint4(0, 0, 0, 0);
        auto fetch = [&](int k0) {
#pragma unroll
            for (int p = 0; p < A_PIECES; p++) {
                const int idx = tid + 256 * p, row = idx >> 3, k = k0 + (idx & 7) * 8;
                pa[p] = (row < TM && k < K) ? la8(row, k) : zero;
            }
#pragma unroll
            for (int p = 0; p < W_PIECES; p++) {
                const int idx = tid + 256 * p, row = idx >> 3, k = k0 + (idx & 7) * 8;
                pw[p] = k < K ? lw8(row, k) : zero;
            }
        };
        fetch(0);
        for (int k0 = 0; k0 < K; k0 += TMF_BK) {
#pragma unroll
            for (int p = 0; p < A_PIECES; p++) {
                const int idx = tid + 256 * p, row = idx >> 3;
                if (row < TM) *reinterpret_cast<uint4*>(&sh.a[row][(idx & 7) * 8]) = pa[p];
            }
#pragma unroll
            for (int p = 0; p < W_PIECES; p++) {
                const int idx = tid + 256 * p;
                *reinterpret_cast<uint4*>(&sh.w[idx >> 3][(idx & 7) * 8]) = pw[p];
            }
            __syncthreads();
            if (k0 + TMF_BK < K) fetch(k0 + TMF_BK);
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                union { uint4 u; tm_bf16x8 v; } fa[MI], fw[SETS][NJ];
#pragma unroll
                for (int i = 0; i < MI; i++) fa[i].u = *reinterpret_cast<const uint4*>(&sh.a[wave_m() + 16 * i + r][(ks * 4 + g) * 8]);
#pragma unroll
                for (int s = 0; s < SETS; s++)
#pragma unroll
                    for (int j = 0; j < NJ; j++)
                        fw[s][j].u = *reinterpret_cast<const uint4*>(&sh.w[64 * s + wave_n() + 16 * j + r][(ks * 4 + g) * 8]);
#pragma unroll
                for (int s = 0; s < SETS; s++)
#pragma unroll
                    for (int i = 0; i < MI; i++)
#pragma unroll
                        for (int j = 0; j < NJ; j++)
                            acc[s][i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[s][j].v, fa[i].v, acc[s][i][j], 0, 0, 0);
            }
            __syncthreads();
        }
    }
};
