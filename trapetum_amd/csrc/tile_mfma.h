// The tiled product of tile.h on the matrix cores, for bf16 operands whose rows can be read in 16-byte pieces (K a
// multiple of 8, rows starting on 16 bytes): a block of 256 threads forms TM x 64 outputs of A . W^T (TM = 128 or 64:
// the four waves in a 2 x 2 arrangement, 64 x 32 or 32 x 32 each; TM = 16: the waves side by side, 16 x 16 each) with
// v_mfma_f32_16x16x32_bf16, fp32 accumulation.  GATED (two sets of 64 rows of W): the block stages 64 gate rows and
// the 64 up rows of the same units, and every lane ends up with a unit's gate and up sum in accumulators of the same
// index; or the two sets are 128 neighbouring columns of a plain product.
// K is walked in steps of 64 through one LDS buffer; the pieces of the step DEPTH steps ahead are asked for before the
// current step is multiplied and written to LDS when their turn comes (few rows stream W: four steps in flight then).  The callers supply the loads: la8(m, k) and lw8(n, k) return the 8
// elements from k on of the tile's row m of A and row n of W (n < 128 when GATED: 64 gate rows, then 64 up rows),
// zeros outside the operand.
#pragma once
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 tm_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float tm_f32x4;

// An LDS row is one step long (128 bytes); its 16-byte pieces are stored at piece ^ (row & 7), so that the 16 rows a
// fragment read touches spread over the banks.
constexpr int TMF_BK = 64, TMF_ROW = TMF_BK;

template <int TM, bool GATED>
struct MfmaTile {
    static constexpr int WN = GATED ? 128 : 64;
    static constexpr int MI = TM >= 64 ? TM / 32 : 1, NJ = TM >= 64 ? 2 : 1, SETS = GATED ? 2 : 1;
    static constexpr int DEPTH = TM >= 64 ? 1 : 4;
    static constexpr int A_PIECES = TM * 8 / 256 > 0 ? TM * 8 / 256 : 1, W_PIECES = WN * 8 / 256;
    struct Shared { alignas(16) bf16_t a[TM][TMF_ROW]; alignas(16) bf16_t w[WN][TMF_ROW]; };
    tm_f32x4 acc[SETS][MI][NJ];

    // where the lane's accumulators lie in the tile: row m_of(i) (lane's r), columns n_of(j) + v, v = 0 .. 3
    __device__ __forceinline__ static int wave_m() { return TM >= 64 ? (TM / 2) * ((threadIdx.x >> 6) >> 1) : 0; }
    __device__ __forceinline__ static int wave_n() { return TM >= 64 ? 32 * ((threadIdx.x >> 6) & 1) : 16 * (threadIdx.x >> 6); }
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
        uint4 pa[DEPTH][A_PIECES], pw[DEPTH][W_PIECES];
        const uint4 zero = make_uint4(0, 0, 0, 0);
        auto fetch = [&](int k0, uint4 (&qa)[A_PIECES], uint4 (&qw)[W_PIECES]) {
#pragma unroll
            for (int p = 0; p < A_PIECES; p++) {
                const int idx = tid + 256 * p, row = idx >> 3, k = k0 + (idx & 7) * 8;
                qa[p] = (row < TM && k < K) ? la8(row, k) : zero;
            }
#pragma unroll
            for (int p = 0; p < W_PIECES; p++) {
                const int idx = tid + 256 * p, row = idx >> 3, k = k0 + (idx & 7) * 8;
                qw[p] = k < K ? lw8(row, k) : zero;
            }
        };
#pragma unroll
        for (int d = 0; d < DEPTH; d++) fetch(d * TMF_BK, pa[d], pw[d]);
        for (int kb = 0; kb < K; kb += TMF_BK * DEPTH) {
#pragma unroll
          for (int d = 0; d < DEPTH; d++) {
            const int k0 = kb + d * TMF_BK;
            if (k0 >= K) break;
#pragma unroll
            for (int p = 0; p < A_PIECES; p++) {
                const int idx = tid + 256 * p, row = idx >> 3;
                if (row < TM) *reinterpret_cast<uint4*>(&sh.a[row][(((idx & 7) ^ (row & 7))) * 8]) = pa[d][p];
            }
#pragma unroll
            for (int p = 0; p < W_PIECES; p++) {
                const int idx = tid + 256 * p;
                *reinterpret_cast<uint4*>(&sh.w[idx >> 3][((idx & 7) ^ ((idx >> 3) & 7)) * 8]) = pw[d][p];
            }
            __syncthreads();
            if (k0 + TMF_BK * DEPTH < K) fetch(k0 + TMF_BK * DEPTH, pa[d], pw[d]);
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                union { uint4 u; tm_bf16x8 v; } fa[MI], fw[SETS][NJ];
#pragma unroll
                for (int i = 0; i < MI; i++) fa[i].u = *reinterpret_cast<const uint4*>(&sh.a[wave_m() + 16 * i + r][((ks * 4 + g) ^ (r & 7)) * 8]);
#pragma unroll
                for (int s = 0; s < SETS; s++)
#pragma unroll
                    for (int j = 0; j < NJ; j++)
                        fw[s][j].u = *reinterpret_cast<const uint4*>(&sh.w[64 * s + wave_n() + 16 * j + r][((ks * 4 + g) ^ (r & 7)) * 8]);
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
    }
};
