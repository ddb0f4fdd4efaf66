// A mixture of experts: the router's choice, the step's (token, expert) pairs sorted by expert, the experts' two
// products over runs of pairs, and the weighted sum per token.  Nothing here returns to the host: the number of pairs
// an expert gets lives on the device, and launches are sized for the worst case.
#include "common.h"
#include "tile.h"
#include "tile_mfma.h"

// ---- scores = softmax(logits) over all experts, or sigmoid(logits) of each; the `top` largest (ties: the smaller
// index) and their scores.  grid (rows), one wave a row; dynamic LDS: E floats
enum { TP_ROUTE_SOFTMAX = 0, TP_ROUTE_SIGMOID = 1 };
__global__ void __launch_bounds__(64)
route_top_k(const float* __restrict__ logits, int E, int top, int renormalize, int score, int* __restrict__ chosen, float* __restrict__ weight) {
    extern __shared__ float sc[];
    const int r = blockIdx.x, lane = threadIdx.x;
    const float* z = logits + (size_t)r * E;
    float sum = 1.f;
    if (score == TP_ROUTE_SIGMOID) {
        for (int e = lane; e < E; e += 64) sc[e] = 1.f / (1.f + expf(-z[e]));
    } else {
        float mx = -INFINITY;
        for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
        mx = wave_max(mx);
        sum = 0.f;
        for (int e = lane; e < E; e += 64) { const float p = expf(z[e] - mx); sc[e] = p; sum += p; }
        sum = wave_sum(sum);
    }
    __syncthreads();
    float kept = 0.f;
    for (int k = 0; k < top; k++) {
        float best = -1.f;
        int at = E;
        for (int e = lane; e < E; e += 64) if (sc[e] > best) { best = sc[e]; at = e; }     // ascending e: the first of equals stays
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oa = __shfl_xor(at, o, 64);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
        }
        if (lane == 0) {
            chosen[(size_t)r * top + k] = at;
            weight[(size_t)r * top + k] = best / sum;
            sc[at] = -1.f;                               // scores are positive: a chosen expert is not chosen again
        }
        kept += best / sum;
        __syncthreads();
    }
    if (renormalize && lane == 0)
        for (int k = 0; k < top; k++) weight[(size_t)r * top + k] /= kept;
}

extern "C" int tp_route_top(const float* logits, int M, int E, int top, int renormalize, int score, int* chosen, float* weight, void* stream) {
    TP_REQUIRE(score == TP_ROUTE_SOFTMAX || score == TP_ROUTE_SIGMOID, "route_top: unknown kind of score %d", score);
    TP_REQUIRE(M > 0 && E > 0 && top > 0 && top <= E, "route_top: %d of %d experts for %d rows", top, E, M);
    TP_REQUIRE(logits && chosen && weight, "route_top: a null operand");
    TP_REQUIRE((size_t)E * sizeof(float) <= 60000, "route_top: %d experts exceed the kernel's table", E);
    route_top_k<<<M, 64, (size_t)E * sizeof(float), (hipStream_t)stream>>>(logits, E, top, renormalize, score, chosen, weight);
    return tp_check_launch("route_top");
}

// ---- pairs sorted by expert: order[i] = the pair at sorted place i, place[pair] = its sorted place, first[e] = where
// expert e's run starts (first[E] = P).  Pairs of one expert keep their order.  grid (experts), 256 threads ---------
__global__ void __launch_bounds__(256)
expert_sort_k(const int* __restrict__ chosen, int P, int E, int* __restrict__ order, int* __restrict__ place, int* __restrict__ first) {
    __shared__ int wave_n[4];
    __shared__ int below_s[4];
    const int e = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int below = 0;
    for (int p = tid; p < P; p += 256) below += chosen[p] < e ? 1 : 0;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) below += __shfl_xor(below, o, 64);
    if (lane == 0) below_s[wave] = below;
    __syncthreads();
    const int start = below_s[0] + below_s[1] + below_s[2] + below_s[3];
    int base = start;
    for (int p0 = 0; p0 < P; p0 += 256) {
        const int p = p0 + tid;
        const bool mine = p < P && chosen[p] == e;
        const unsigned long long mask = __ballot(mine);
        if (lane == 0) wave_n[wave] = __popcll(mask);
        __syncthreads();
        int before = __popcll(mask & ((1ull << lane) - 1ull));
        for (int w = 0; w < wave; w++) before += wave_n[w];
        if (mine) { order[base + before] = p; place[p] = base + before; }
        base += wave_n[0] + wave_n[1] + wave_n[2] + wave_n[3];
        __syncthreads();
    }
    if (tid == 0) {
        first[e] = start;
        if (e == E - 1) first[E] = P;
    }
}

// ---- an expert's products over its run of pairs.  Tiles of TM pairs of one expert x TN columns; grid (column tiles,
// row tiles for the worst case): a block finds its expert and tile by walking first[], one past the end leaves.
// GATED: rows of X gathered by pair (token = pair / top), W [E, 2 F, K] (gate rows, then up rows),
//        y = min(g, limit) * sigmoid(alpha min(g, limit)) * (clamp(u, -limit, limit) + shift)  -> T [P, F] by sorted place;
// else:  rows of A = sorted places themselves, W [E, N, K], out float [P, N] by sorted place.
template <typename T, bool GATED, int TM>
__global__ void __launch_bounds__(256)
expert_linear_k(const T* __restrict__ a, const T* __restrict__ w, const int* __restrict__ order, const int* __restrict__ first,
                int E, int top, int N, int K, float limit, float alpha, float shift, const float* __restrict__ in_scale, void* __restrict__ out) {
    constexpr int TN = 64, BK = 16;
    __shared__ TileShared<TM, GATED ? 2 * TN : TN, BK> sh;
    int t = blockIdx.y, e = 0, lo = 0, hi = 0;
    for (; e < E; e++) {
        lo = first[e]; hi = first[e + 1];
        const int tiles = (hi - lo + TM - 1) / TM;
        if (t < tiles) break;
        t -= tiles;
    }
    if (e == E) return;
    const int p0 = lo + t * TM, n0 = blockIdx.x * TN;
    const T* we = w + (size_t)e * (GATED ? 2 : 1) * N * K;
    const int ty = threadIdx.x >> 4, tx = threadIdx.x & 15;
    if constexpr (GATED) {
        float acc[TM / 16][2 * TN / 16];                 // columns 0 .. TN - 1: gate, TN .. 2 TN - 1: up, of the same units
        tile_product<TM, 2 * TN, BK>(acc, K,
            [&](int m, int k) { return p0 + m < hi ? ld_f32(a + (size_t)(order[p0 + m] / top) * K + k) : 0.f; },
            [&](int n, int k) { const int u = n0 + (n & (TN - 1)); return u < N ? ld_f32(we + ((size_t)(n >= TN ? N : 0) + u) * K + k) : 0.f; }, sh);
#pragma unroll
        for (int i = 0; i < TM / 16; i++)
#pragma unroll
            for (int j = 0; j < TN / 16; j++) {
                const int p = p0 + ty + 16 * i, n = n0 + tx + 16 * j;
                if (p >= hi || n >= N) continue;
                const float sc = in_scale ? in_scale[order[p]] : 1.f;      // the pair's weight on the expert's input: W (s h) = s (W h)
                const float g = fminf(acc[i][j] * sc, limit), u = fminf(fmaxf(acc[i][j + TN / 16] * sc, -limit), limit);
                st_f32((T*)out + (size_t)p * N + n, g / (1.f + expf(-alpha * g)) * (u + shift));
            }
    } else {
        float acc[TM / 16][TN / 16];
        tile_product<TM, TN, BK>(acc, K,
            [&](int m, int k) { return p0 + m < hi ? ld_f32(a + (size_t)(p0 + m) * K + k) : 0.f; },
            [&](int n, int k) { return n0 + n < N ? ld_f32(we + (size_t)(n0 + n) * K + k) : 0.f; }, sh);
#pragma unroll
        for (int i = 0; i < TM / 16; i++)
#pragma unroll
            for (int j = 0; j < TN / 16; j++) {
                const int p = p0 + ty + 16 * i, n = n0 + tx + 16 * j;
                if (p < hi && n < N) ((float*)out)[(size_t)p * N + n] = acc[i][j];
            }
    }
}

// the same on the matrix cores: bf16, K a multiple of 8 (rows of A and W then start on 16 bytes).
// MODE 0: 64 columns a block; 1: gated, 64 units (their gate and up rows); 2: 128 columns a block (two sets of 64).
template <int MODE, int TM>
__global__ void __launch_bounds__(256)
expert_linear_mfma_k(const bf16_t* __restrict__ a, const bf16_t* __restrict__ w, const int* __restrict__ order, const int* __restrict__ first,
                     int E, int top, int N, int K, float limit, float alpha, float shift, const float* __restrict__ in_scale, void* __restrict__ out, int k_slice, long out_slice) {
    constexpr bool GATED = MODE == 1;
    constexpr int COLS = MODE == 2 ? 128 : 64;
    using Tile = MfmaTile<TM, MODE != 0>;
    __shared__ typename Tile::Shared sh;
    __shared__ int rows[TM];                             // the tile's rows of A
    int t = blockIdx.y, e = 0, lo = 0, hi = 0;
    for (; e < E; e++) {
        lo = first[e]; hi = first[e + 1];
        const int tiles = (hi - lo + TM - 1) / TM;
        if (t < tiles) break;
        t -= tiles;
    }
    if (e == E) return;
    const int p0 = lo + t * TM, n0 = blockIdx.x * COLS;
    if (threadIdx.x < TM) {
        const int p = p0 + threadIdx.x;
        rows[threadIdx.x] = p < hi ? (GATED ? order[p] / top : p) : -1;
    }
    __syncthreads();
    const bf16_t* we = w + (size_t)e * (GATED ? 2 : 1) * N * K;
    const uint4 zero = make_uint4(0, 0, 0, 0);
    // a plain product of few rows may come in K slices (grid z): slice z sums k in [z k_slice, (z + 1) k_slice) into its
    // own copy of the output, and the consumer adds the copies in slice order
    const int kz = blockIdx.z * k_slice, klen = min(K - kz, k_slice);
    if (!GATED) out = (float*)out + (size_t)blockIdx.z * out_slice;
    Tile tile;
    tile.run(klen,
        [&](int m, int k) { const int row = rows[m]; return row >= 0 ? *reinterpret_cast<const uint4*>(a + (size_t)row * K + kz + k) : zero; },
        [&](int n, int k) {
            const int u = GATED ? n0 + (n & 63) : n0 + n;          // gated: the staged rows 64 .. 127 are the units' up rows
            return u < N ? *reinterpret_cast<const uint4*>(we + ((size_t)(GATED && n >= 64 ? N : 0) + u) * K + kz + k) : zero;
        }, sh);
#pragma unroll
    for (int i = 0; i < Tile::MI; i++)
#pragma unroll
        for (int j = 0; j < Tile::NJ; j++) {
            const int p = p0 + Tile::m_of(i);
            if (p >= hi) continue;
            if constexpr (GATED) {
                const int n = n0 + Tile::n_of(j);
                const float sc = in_scale ? in_scale[order[p]] : 1.f;
                bf16_t o[4];
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const float g = fminf(tile.acc[0][i][j][v] * sc, limit), u = fminf(fmaxf(tile.acc[1][i][j][v] * sc, -limit), limit);
                    o[v] = f32_to_bf16(g / (1.f + expf(-alpha * g)) * (u + shift));
                }
                bf16_t* dst = (bf16_t*)out + (size_t)p * N + n;
                if ((N & 3) == 0 && n + 3 < N) {         // the lane's four neighbours in one store
                    uint2 pk;
                    pk.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
                    pk.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
                    *reinterpret_cast<uint2*>(dst) = pk;
                } else {
#pragma unroll
                    for (int v = 0; v < 4; v++) if (n + v < N) dst[v] = o[v];
                }
            } else {
#pragma unroll
                for (int set = 0; set < Tile::SETS; set++) {
                    const int n = n0 + 64 * set + Tile::n_of(j);
                    float* dst = (float*)out + (size_t)p * N + n;
                    if ((N & 3) == 0 && n + 3 < N)
                        *reinterpret_cast<float4*>(dst) = make_float4(tile.acc[set][i][j][0], tile.acc[set][i][j][1], tile.acc[set][i][j][2], tile.acc[set][i][j][3]);
                    else {
#pragma unroll
                        for (int v = 0; v < 4; v++) if (n + v < N) dst[v] = tile.acc[set][i][j][v];
                    }
                }
            }
        }
}

// The products of many pairs (a prefill) when K is whole steps of 64: tiles of 128 pairs x 128 rows of W (GATED: 64 units'
// gate rows and up rows; else 128 columns), the step's tile straight from global memory into LDS
// (global_load_lds_dwordx4: no staging registers, no LDS writes), as the dense products' loop does it: a step reads all
// its fragments into registers, a barrier, the next step's loads are issued into the same buffer and fly while the
// step's 32 matrix instructions run, a second barrier when they have landed.  A lane's place in LDS is fixed by its
// lane number, so the swizzle (piece ^ (row & 7)) is applied on the global side; a row of A is the pair's token row
// (gathered through `order`), rows past a run's end or past N fetch a row that exists and are never stored.
template <bool GATED>
__global__ void __launch_bounds__(256, 2)
expert_direct_k(const bf16_t* __restrict__ a, const bf16_t* __restrict__ w, const int* __restrict__ order, const int* __restrict__ first,
                int E, int top, int N, int K, float limit, float alpha, float shift, const float* __restrict__ in_scale, void* __restrict__ out) {
    constexpr int BM = 128, BN = 128, BK = 64, LDS = BK, TM = 4, TN = 4;
    __shared__ __attribute__((aligned(16))) bf16_t As[BM * LDS];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[BN * LDS];
    int t = blockIdx.y, e = 0, lo = 0, hi = 0;
    for (; e < E; e++) {
        lo = first[e]; hi = first[e + 1];
        const int tiles = (hi - lo + BM - 1) / BM;
        if (t < tiles) break;
        t -= tiles;
    }
    if (e == E) return;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;
    const int p0 = lo + t * BM, n0 = blockIdx.x * (GATED ? 64 : 128);
    const bf16_t* we = w + (size_t)e * (GATED ? 2 : 1) * N * K;
    // load i of a thread: row (tid >> 3) + 32 i of the tile, the piece that belongs at the lane's place
    const int srow = tid >> 3, chunk = (lane & 7) ^ (srow & 7);
    unsigned xo[TM], wo[TN];
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int p = min(p0 + srow + 32 * i, hi - 1);
        const int row = GATED ? order[p] / top : p;
        xo[i] = (unsigned)row * (unsigned)K * 2u + chunk * 16u;
    }
#pragma unroll
    for (int i = 0; i < TN; i++) {
        const int sr = srow + 32 * i;                    // staged row of W: gated 0 .. 63 gate, 64 .. 127 up of the same units
        const int wrow = GATED ? (sr >= 64 ? N : 0) + min(n0 + (sr & 63), N - 1) : min(n0 + sr, N - 1);
        wo[i] = (unsigned)wrow * (unsigned)K * 2u + chunk * 16u;
    }
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    bf16_t* const a_dst = As + wave_u * 8 * LDS;         // the wave's 8 rows of every group of 32
    bf16_t* const b_dst = Bs + wave_u * 8 * LDS;
    auto fill = [&](int k0) {
        const char* xb = reinterpret_cast<const char*>(a) + (size_t)k0 * 2;
        const char* wb = reinterpret_cast<const char*>(we) + (size_t)k0 * 2;
#pragma unroll
        for (int i = 0; i < TM; i++)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(xb + xo[i]),
                                             (__attribute__((address_space(3))) void*)(a_dst + 32 * i * LDS), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < TN; i++)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(wb + wo[i]),
                                             (__attribute__((address_space(3))) void*)(b_dst + 32 * i * LDS), 16, 0, 0);
    };
    union Frag { uint4 u; tm_bf16x8 v; };
    tm_f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = tm_f32x4{0.f, 0.f, 0.f, 0.f};
    // the wave's rows of W in the staged tile: gated, accumulators j and j + 2 are a unit's gate and up sums
    auto w_row = [&](int j) { return GATED ? (j >= 2 ? 64 : 0) + wn * 32 + (j & 1) * 16 : wn * 64 + j * 16; };
    auto frags = [&](int ks, Frag (&fa)[TM], Frag (&fb)[TN]) {
        const int kc = (((ks >> 3) + g) ^ (r & 7)) * 8;
#pragma unroll
        for (int i = 0; i < TM; i++) fa[i].u = *reinterpret_cast<const uint4*>(As + (wm * 64 + i * 16 + r) * LDS + kc);
#pragma unroll
        for (int j = 0; j < TN; j++) fb[j].u = *reinterpret_cast<const uint4*>(Bs + (w_row(j) + r) * LDS + kc);
    };
    auto mma = [&](Frag (&fa)[TM], Frag (&fb)[TN]) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[j].v, fa[i].v, acc[i][j], 0, 0, 0);
    };
    fill(0);
    __builtin_amdgcn_s_waitcnt(0);                       // every counter at zero: the loads have reached LDS
    __syncthreads();
    for (int k0 = 0; k0 < K; k0 += BK) {
        Frag a0[TM], b0[TN], a1[TM], b1[TN];
        frags(0, a0, b0);
        frags(32, a1, b1);
        __builtin_amdgcn_s_waitcnt(0);                   // the fragments are in registers ...
        __syncthreads();                                 // ... everyone's: the buffer may be refilled
        if (k0 + BK < K) fill(k0 + BK);
        mma(a0, b0);
        mma(a1, b1);
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
    }
    // the lane holds pair row wm * 64 + i * 16 + r, rows of W w_row(j) + g * 4 + v
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int p = p0 + wm * 64 + i * 16 + r;
        if (p >= hi) continue;
        if constexpr (GATED) {
            const float sc = in_scale ? in_scale[order[p]] : 1.f;
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int n = n0 + wn * 32 + j * 16 + g * 4;
                bf16_t o[4];
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const float gg = fminf(acc[i][j][v] * sc, limit), uu = fminf(fmaxf(acc[i][j + 2][v] * sc, -limit), limit);
                    o[v] = f32_to_bf16(gg / (1.f + expf(-alpha * gg)) * (uu + shift));
                }
                bf16_t* dst = (bf16_t*)out + (size_t)p * N + n;
                if ((N & 3) == 0 && n + 3 < N) {
                    uint2 pk;
                    pk.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
                    pk.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
                    *reinterpret_cast<uint2*>(dst) = pk;
                } else {
#pragma unroll
                    for (int v = 0; v < 4; v++) if (n + v < N) dst[v] = o[v];
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const int n = n0 + wn * 64 + j * 16 + g * 4;
                float* dst = (float*)out + (size_t)p * N + n;
                if ((N & 3) == 0 && n + 3 < N) *reinterpret_cast<float4*>(dst) = make_float4(acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]);
                else {
#pragma unroll
                    for (int v = 0; v < 4; v++) if (n + v < N) dst[v] = acc[i][j][v];
                }
            }
        }
    }
}

// The same for the few pairs of a decode step, where the experts' matrices are streamed once and nothing is reused:
// no LDS and no barrier.  A block takes 16 pairs of one expert x 64 columns, a wave 16 of the columns (GATED: the gate
// and the up rows of 16 units); a lane reads its row of W and its pair's row of A straight into the matrix
// instruction's operands, UN k steps of 32 asked for at once, so that a wave alone keeps a dozen kilobytes in flight.
template <bool GATED>
__global__ void __launch_bounds__(256)
expert_stream_k(const bf16_t* __restrict__ a, const bf16_t* __restrict__ w, const int* __restrict__ order, const int* __restrict__ first,
                int E, int top, int N, int K, float limit, float alpha, float shift, const float* __restrict__ in_scale, void* __restrict__ out, int k_slice, long out_slice) {
    constexpr int TM = 16, UN = 8;
    int t = blockIdx.y, e = 0, lo = 0, hi = 0;
    for (; e < E; e++) {
        lo = first[e]; hi = first[e + 1];
        const int tiles = (hi - lo + TM - 1) / TM;
        if (t < tiles) break;
        t -= tiles;
    }
    if (e == E) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, g = lane >> 4;
    const int p0 = lo + t * TM, n0 = blockIdx.x * 64 + wave * 16;
    if (n0 >= N) return;
    const int kz = blockIdx.z * k_slice, klen = min(K - kz, k_slice);
    const int p = p0 + r, nw = n0 + r;
    const bool a_ok = p < hi, w_ok = nw < N;
    const size_t arow = a_ok ? (size_t)(GATED ? order[p] / top : p) : 0;
    const bf16_t* ap = a + arow * K + kz + g * 8;
    const bf16_t* we = w + (size_t)e * (GATED ? 2 : 1) * N * K;
    const bf16_t* wg = we + (size_t)(w_ok ? nw : 0) * K + kz + g * 8;
    const bf16_t* wu = wg + (size_t)N * K;               // the unit's up row (gated)
    tm_f32x4 acc_g = {0.f, 0.f, 0.f, 0.f}, acc_u = {0.f, 0.f, 0.f, 0.f};
    const uint4 zero = make_uint4(0, 0, 0, 0);
    union F { uint4 u; tm_bf16x8 v; };
    for (int k0 = 0; k0 < klen; k0 += 32 * UN) {
        F fa[UN], fg[UN], fu[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const int k = k0 + 32 * u;
            const bool in = k + g * 8 < klen;
            fa[u].u = (in && a_ok) ? *reinterpret_cast<const uint4*>(ap + k) : zero;
            fg[u].u = (in && w_ok) ? *reinterpret_cast<const uint4*>(wg + k) : zero;
            if (GATED) fu[u].u = (in && w_ok) ? *reinterpret_cast<const uint4*>(wu + k) : zero;
        }
#pragma unroll
        for (int u = 0; u < UN; u++) {
            acc_g = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fg[u].v, fa[u].v, acc_g, 0, 0, 0);
            if (GATED) acc_u = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fu[u].v, fa[u].v, acc_u, 0, 0, 0);
        }
    }
    // the lane holds pair r, columns n0 + g * 4 + v
    if (!a_ok) return;
    const int n = n0 + g * 4;
    if constexpr (GATED) {
        bf16_t* dst = (bf16_t*)out + (size_t)p * N + n;
        const float sc = in_scale ? in_scale[order[p]] : 1.f;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            if (n + v >= N) continue;
            const float gg = fminf(acc_g[v] * sc, limit), uu = fminf(fmaxf(acc_u[v] * sc, -limit), limit);
            dst[v] = f32_to_bf16(gg / (1.f + expf(-alpha * gg)) * (uu + shift));
        }
    } else {
        float* dst = (float*)out + (size_t)blockIdx.z * out_slice + (size_t)p * N + n;
#pragma unroll
        for (int v = 0; v < 4; v++) if (n + v < N) dst[v] = acc_g[v];
    }
}

// ---- out[m] = sum_k weight[m, k] * pair_out[place[m top + k]], k ascending, float32.  grid (rows, column blocks) ------
// K slices the down product of a decode step is cut in (when the experts' width allows slices of whole steps)
static int down_slices(int P, int F) { return (P <= 64 && F >= 1024 && F % 256 == 0) ? 4 : 1; }
__global__ void __launch_bounds__(256)
expert_combine_k(const float* __restrict__ pair_out, int n_slices, long slice_stride, const int* __restrict__ place,
                 const float* __restrict__ weight, int top, int D, float* __restrict__ out) {
    const int m = blockIdx.x, d = blockIdx.y * 256 + threadIdx.x;
    if (d >= D) return;
    float acc = 0.f;
    for (int k = 0; k < top; k++) {
        const float* src = pair_out + (size_t)place[(size_t)m * top + k] * D + d;
        float v = src[0];
        for (int z = 1; z < n_slices; z++) v += src[(size_t)z * slice_stride];       // the K slices of a pair's output, in slice order
        acc = weight ? __builtin_fmaf(weight[(size_t)m * top + k], v, acc) : acc + v;
    }
    out[(size_t)m * D + d] = acc;
}

// workspace: order [P], place [P], first [E + 1] (int32), then y [P, F] of the activation dtype, then pair_out [P, D] float
static size_t align256(size_t n) { return (n + 255) / 256 * 256; }
extern "C" long tp_expert_ffn_workspace_bytes(int dtype, int M, int top, int E, int F, int D) {
    const size_t P = (size_t)M * top, el = dtype == TP_BF16 ? 2 : 4;
    return (long)(align256((2 * P + E + 1) * sizeof(int)) + align256(P * F * el) + align256(P * D * sizeof(float) * down_slices((int)P, F)));
}

extern "C" int tp_expert_ffn(const void* x, int dtype, int M, int D, const int* chosen, const float* weight, int top, int E, int F,
                             const void* w_gate_up, const void* w_down, float limit, float alpha, float shift, int weight_input,
                             void* workspace, long workspace_bytes, float* out, int plain, void* stream) {
    // weight_input: a pair's weight multiplies the expert's input (inside the activation) instead of its output
    const float* in_scale = weight_input ? weight : nullptr;
    const float* out_weight = weight_input ? nullptr : weight;
    TP_REQUIRE(M > 0 && D > 0 && top > 0 && E > 0 && F > 0, "expert_ffn: empty shape M=%d D=%d top=%d E=%d F=%d", M, D, top, E, F);
    TP_REQUIRE(x && chosen && weight && w_gate_up && w_down && workspace && out, "expert_ffn: a null operand");
    TP_REQUIRE(dtype == TP_BF16 || dtype == TP_F32, "expert_ffn: unknown dtype %d", dtype);
    TP_REQUIRE(workspace_bytes >= tp_expert_ffn_workspace_bytes(dtype, M, top, E, F, D), "expert_ffn: a workspace of %ld bytes is too small", workspace_bytes);
    TP_REQUIRE(E <= 65535 && (long)M * top < (1L << 30), "expert_ffn: too many experts or pairs for one launch");
    hipStream_t s = (hipStream_t)stream;
    const int P = M * top;
    const size_t el = dtype == TP_BF16 ? 2 : 4;
    int* order = (int*)workspace;
    int* place = order + P;
    int* first = place + P;
    char* y = (char*)workspace + align256((2 * (size_t)P + E + 1) * sizeof(int));
    float* pair_out = (float*)(y + align256((size_t)P * F * el));
    expert_sort_k<<<E, 256, 0, s>>>(chosen, P, E, order, place, first);
    if (int rc = tp_check_launch("expert_ffn (sort)")) return rc;
    const bool few = P <= 64;                            // a decode step: most runs hold a pair or two
    const bool cores = dtype == TP_BF16 && !plain && D % 8 == 0 && F % 8 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)w_gate_up % 16 == 0 &&
                       (uintptr_t)w_down % 16 == 0;
    const bool many = cores && P >= 128 * E;             // runs of a hundred pairs and more: tiles of 128 rows
    const int TM = few ? 16 : (many ? 128 : 64);
    const int row_tiles = tp_cdiv(P, TM) + (E < P ? E : P);
    TP_REQUIRE(row_tiles <= 65535, "expert_ffn: %d row tiles exceed one launch", row_tiles);
#define TP_EXPERT(T, G, TMv, Nv, Kv, A, W, S, O) expert_linear_k<T, G, TMv><<<dim3(tp_cdiv(Nv, 64), row_tiles), 256, 0, s>>>( \
        (const T*)(A), (const T*)(W), order, first, E, top, Nv, Kv, limit, alpha, shift, S, O)
#define TP_EXPERT_MFMA(G, TMv, Nv, Kv, A, W, S, O, Z) expert_linear_mfma_k<G, TMv><<<dim3(tp_cdiv(Nv, (G) == 2 ? 128 : 64), row_tiles, Z), 256, 0, s>>>( \
        (const bf16_t*)(A), (const bf16_t*)(W), order, first, E, top, Nv, Kv, limit, alpha, shift, S, O, (Kv) / (Z), (long)P * (Nv))
    if (cores) {
        if (few) expert_stream_k<true><<<dim3(tp_cdiv(F, 64), row_tiles, 1), 256, 0, s>>>((const bf16_t*)x, (const bf16_t*)w_gate_up, order, first, E, top, F, D,
                                                                                             limit, alpha, shift, in_scale, y, D, 0);
        else if (many && D % 64 == 0 && (long)M * D * 2 < (1L << 32) && 2L * F * D * 2 < (1L << 32))
            expert_direct_k<true><<<dim3(tp_cdiv(F, 64), row_tiles), 256, 0, s>>>((const bf16_t*)x, (const bf16_t*)w_gate_up, order, first, E, top, F, D,
                                                                                  limit, alpha, shift, in_scale, y);
        else if (many) TP_EXPERT_MFMA(1, 128, F, D, x, w_gate_up, in_scale, y, 1); else TP_EXPERT_MFMA(1, 64, F, D, x, w_gate_up, in_scale, y, 1);
        if (int rc = tp_check_launch("expert_ffn (gate, up; matrix cores)")) return rc;
        const int zs = down_slices(P, F);
        if (few) expert_stream_k<false><<<dim3(tp_cdiv(D, 64), row_tiles, zs), 256, 0, s>>>((const bf16_t*)y, (const bf16_t*)w_down, order, first, E, top, D, F,
                                                                                               limit, alpha, shift, nullptr, pair_out, F / zs, (long)P * D);
        else if (many && F % 64 == 0 && (long)P * F * 2 < (1L << 32) && (long)D * F * 2 < (1L << 32))
            expert_direct_k<false><<<dim3(tp_cdiv(D, 128), row_tiles), 256, 0, s>>>((const bf16_t*)y, (const bf16_t*)w_down, order, first, E, top, D, F,
                                                                                    limit, alpha, shift, nullptr, pair_out);
        else if (many) TP_EXPERT_MFMA(2, 128, D, F, y, w_down, nullptr, pair_out, 1); else TP_EXPERT_MFMA(0, 64, D, F, y, w_down, nullptr, pair_out, 1);
        if (int rc = tp_check_launch("expert_ffn (down; matrix cores)")) return rc;
        expert_combine_k<<<dim3(M, tp_cdiv(D, 256)), 256, 0, s>>>(pair_out, zs, (long)P * D, place, out_weight, top, D, out);
        return tp_check_launch("expert_ffn (combine)");
    }
#undef TP_EXPERT_MFMA
    if (dtype == TP_BF16) { if (few) TP_EXPERT(bf16_t, true, 16, F, D, x, w_gate_up, in_scale, y); else TP_EXPERT(bf16_t, true, 64, F, D, x, w_gate_up, in_scale, y); }
    else { if (few) TP_EXPERT(float, true, 16, F, D, x, w_gate_up, in_scale, y); else TP_EXPERT(float, true, 64, F, D, x, w_gate_up, in_scale, y); }
    if (int rc = tp_check_launch("expert_ffn (gate, up)")) return rc;
    if (dtype == TP_BF16) { if (few) TP_EXPERT(bf16_t, false, 16, D, F, y, w_down, nullptr, pair_out); else TP_EXPERT(bf16_t, false, 64, D, F, y, w_down, nullptr, pair_out); }
    else { if (few) TP_EXPERT(float, false, 16, D, F, y, w_down, nullptr, pair_out); else TP_EXPERT(float, false, 64, D, F, y, w_down, nullptr, pair_out); }
#undef TP_EXPERT
    if (int rc = tp_check_launch("expert_ffn (down)")) return rc;
    expert_combine_k<<<dim3(M, tp_cdiv(D, 256)), 256, 0, s>>>(pair_out, 1, 0, place, out_weight, top, D, out);
    return tp_check_launch("expert_ffn (combine)");
}
