// A state-space mixer's own kernels (a decaying matrix state per head, after a short convolution), and the two small
// row-wise kernels of a mixer that runs two mixers side by side.
//
//   conv_act      out_t = act(b + sum_j w[:, j] u_(t - taps + 1 + j)) on every channel of the step's rows, the rows before
//                 the step kept per sequence as a state (float32, the projection's values as they were)
//   ssd_scan      S_t = exp(-exp(a) dt_t) S_(t-1) + dt_t B_t x_t^T,  y_t = (S_t^T C_t + D x_t) * silu(z_t),
//                 dt_t = softplus(raw_t + bias); S, dt, the decay and y in float32
//   pair_norm_mean  0.5 (a / rms(a) * wa + b / rms(b) * wb) over rows
//   mul_sigmoid   x *= sigmoid(g)
#include "common.h"

enum { TP_CONV_ACT_NONE = 0, TP_CONV_ACT_SILU = 1 };

// grid (rows, channel blocks of 256).  wt: taps transposed [taps, C].  state [slots, taps - 1, C], oldest row first.
template <typename TI, typename TO>
__global__ void __launch_bounds__(256)
conv_act_k(const TI* __restrict__ x, long x_stride, const float* __restrict__ wt, const float* __restrict__ bias,
           float* __restrict__ state, const int* __restrict__ slot_ids, const int* __restrict__ cu_rows,
           const int* __restrict__ row_seq, TO* __restrict__ out, long out_stride, int C, int taps, int act, int one_row_each) {
    const int r = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int seq = row_seq[r], i = r - cu_rows[seq], S = taps - 1;
    float* st = S > 0 ? state + (size_t)slot_ids[seq] * S * C + c : nullptr;
    const float xr = ld_f32(x + (size_t)r * x_stride + c);
    float acc = bias ? bias[c] : 0.f;
    for (int j = 0; j < taps; j++) {
        const int src = i - (S - j);                     // the step's row this tap reads; negative: before the step
        const float v = j == S ? xr : (src >= 0 ? ld_f32(x + (size_t)(r - (S - j)) * x_stride + c) : st[(size_t)(S + src) * C]);
        acc = __builtin_fmaf(wt[(size_t)j * C + c], v, acc);
    }
    if (act == TP_CONV_ACT_SILU) acc = acc / (1.f + expf(-acc));
    st_f32(out + (size_t)r * out_stride + c, acc);
    if (one_row_each && S > 0) {
        for (int s = 0; s + 1 < S; s++) st[(size_t)s * C] = st[(size_t)(s + 1) * C];
        st[(size_t)(S - 1) * C] = xr;
    }
}

// VEC neighbouring elements of T as one load or store
template <typename T, int VEC> struct alignas(sizeof(T) * VEC) Pack { T v[VEC]; };

// The same for channel counts and strides in whole packs of VEC: a thread takes VEC neighbouring channels.
template <typename T, int VEC>
__global__ void __launch_bounds__(256)
conv_act_vec_k(const T* __restrict__ x, long x_stride, const float* __restrict__ wt, const float* __restrict__ bias,
               float* __restrict__ state, const int* __restrict__ slot_ids, const int* __restrict__ cu_rows,
               const int* __restrict__ row_seq, T* __restrict__ out, long out_stride, int C, int taps, int act, int one_row_each) {
    using P = Pack<T, VEC>;
    using PF = Pack<float, VEC>;
    const int r = blockIdx.x, c = (blockIdx.y * 256 + threadIdx.x) * VEC;
    if (c >= C) return;
    const int seq = row_seq[r], i = r - cu_rows[seq], S = taps - 1;
    float* st = S > 0 ? state + (size_t)slot_ids[seq] * S * C + c : nullptr;
    const P xr = *reinterpret_cast<const P*>(x + (size_t)r * x_stride + c);
    float acc[VEC];
    if (bias) {
        const PF b = *reinterpret_cast<const PF*>(bias + c);
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[e] = b.v[e];
    } else {
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[e] = 0.f;
    }
    for (int j = 0; j < taps; j++) {
        const int src = i - (S - j);
        const PF w = *reinterpret_cast<const PF*>(wt + (size_t)j * C + c);
        if (j == S || src >= 0) {
            const P v = j == S ? xr : *reinterpret_cast<const P*>(x + (size_t)(r - (S - j)) * x_stride + c);
#pragma unroll
            for (int e = 0; e < VEC; e++) acc[e] = __builtin_fmaf(w.v[e], ld_f32(&v.v[e]), acc[e]);
        } else {
            const PF v = *reinterpret_cast<const PF*>(st + (size_t)(S + src) * C);
#pragma unroll
            for (int e = 0; e < VEC; e++) acc[e] = __builtin_fmaf(w.v[e], v.v[e], acc[e]);
        }
    }
    P o;
#pragma unroll
    for (int e = 0; e < VEC; e++) {
        const float v = act == TP_CONV_ACT_SILU ? acc[e] / (1.f + expf(-acc[e])) : acc[e];
        st_f32(&o.v[e], v);
    }
    *reinterpret_cast<P*>(out + (size_t)r * out_stride + c) = o;
    if (one_row_each && S > 0) {
        for (int s = 0; s + 1 < S; s++) *reinterpret_cast<PF*>(st + (size_t)s * C) = *reinterpret_cast<const PF*>(st + (size_t)(s + 1) * C);
        PF last;
#pragma unroll
        for (int e = 0; e < VEC; e++) last.v[e] = ld_f32(&xr.v[e]);
        *reinterpret_cast<PF*>(st + (size_t)(S - 1) * C) = last;
    }
}

// grid (sequences, channel blocks): the state takes the last taps - 1 rows of (state, the step's rows)
template <typename TI>
__global__ void __launch_bounds__(256)
conv_act_state_k(const TI* __restrict__ x, long x_stride, float* __restrict__ state, const int* __restrict__ slot_ids,
                 const int* __restrict__ cu_rows, int C, int taps) {
    const int seq = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int first = cu_rows[seq], count = cu_rows[seq + 1] - first, S = taps - 1;
    float* st = state + (size_t)slot_ids[seq] * S * C + c;
    for (int s = 0; s < S; s++) {                        // ascending: a row of the old state is read before it is overwritten
        const int src = count - S + s;
        st[(size_t)s * C] = src >= 0 ? ld_f32(x + (size_t)(first + src) * x_stride + c) : st[(size_t)(s + count) * C];
    }
}

extern "C" int tp_conv_act(const void* x, long x_stride, int in_dtype, const float* wt, const float* bias, float* state,
                           const int* slot_ids, const int* cu_rows, const int* row_seq, void* out, long out_stride, int out_dtype,
                           int M, int n_seq, int C, int taps, int act, int one_row_each, void* stream) {
    TP_REQUIRE(M > 0 && n_seq > 0 && C > 0 && taps >= 1, "conv_act: empty shape M=%d sequences=%d C=%d taps=%d", M, n_seq, C, taps);
    TP_REQUIRE(x && wt && out && cu_rows && row_seq, "conv_act: a null operand");
    TP_REQUIRE(taps == 1 || (state && slot_ids), "conv_act: %d taps need the sequences' states", taps);
    TP_REQUIRE(!one_row_each || M == n_seq, "conv_act: one row each, but %d rows for %d sequences", M, n_seq);
    TP_REQUIRE(act == TP_CONV_ACT_NONE || act == TP_CONV_ACT_SILU, "conv_act: unknown activation %d", act);
    TP_REQUIRE(in_dtype == out_dtype && (in_dtype == TP_BF16 || in_dtype == TP_F32), "conv_act: rows and output share one dtype, bfloat16 or float32");
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(M, tp_cdiv(C, 256));
    const int vec = in_dtype == TP_BF16 ? 8 : 4;         // 16 bytes of the rows a thread; few rows: a thread a channel, more blocks
    const bool packs = (long)M * C >= (1L << 18) && C % vec == 0 && x_stride % vec == 0 && out_stride % vec == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)out % 16 == 0 &&
                       (uintptr_t)wt % 32 == 0 && (!bias || (uintptr_t)bias % 32 == 0) && (!state || (uintptr_t)state % 32 == 0);
    if (packs) {
        dim3 vgrid(M, tp_cdiv(C / vec, 256));
        if (in_dtype == TP_BF16)
            conv_act_vec_k<bf16_t, 8><<<vgrid, 256, 0, s>>>((const bf16_t*)x, x_stride, wt, bias, state, slot_ids, cu_rows, row_seq, (bf16_t*)out, out_stride, C, taps, act, one_row_each);
        else
            conv_act_vec_k<float, 4><<<vgrid, 256, 0, s>>>((const float*)x, x_stride, wt, bias, state, slot_ids, cu_rows, row_seq, (float*)out, out_stride, C, taps, act, one_row_each);
    } else if (in_dtype == TP_BF16)
        conv_act_k<bf16_t, bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)x, x_stride, wt, bias, state, slot_ids, cu_rows, row_seq, (bf16_t*)out, out_stride, C, taps, act, one_row_each);
    else
        conv_act_k<float, float><<<grid, 256, 0, s>>>((const float*)x, x_stride, wt, bias, state, slot_ids, cu_rows, row_seq, (float*)out, out_stride, C, taps, act, one_row_each);
    if (int rc = tp_check_launch("conv_act")) return rc;
    if (taps > 1 && !one_row_each) {
        dim3 sgrid(n_seq, tp_cdiv(C, 256));
        if (in_dtype == TP_BF16) conv_act_state_k<bf16_t><<<sgrid, 256, 0, s>>>((const bf16_t*)x, x_stride, state, slot_ids, cu_rows, C, taps);
        else conv_act_state_k<float><<<sgrid, 256, 0, s>>>((const float*)x, x_stride, state, slot_ids, cu_rows, C, taps);
        return tp_check_launch("conv_act (state)");
    }
    return 0;
}

// ---- the scan ---------------------------------------------------------------------------------------------------
struct SsdArgs {
    const void* xbc; long xbc_stride;                    // rows [x: heads P | B: groups N | C: groups N] after convolution and activation
    const void* z; long z_stride;                        // gate rows [heads P]
    const void* dt; long dt_stride;                      // raw step sizes [heads]
    const float* dt_bias; const float* a_log; const float* skip;
    float* state;                                        // [slots, heads, N, P]
    const int* slot_ids; const int* cu_rows;
    float* y;                                            // [rows, heads P]
    int heads, groups, N, P;
    // a scan cut into pieces (chunk > 0): piece c of a sequence covers its rows [c chunk, (c + 1) chunk)
    int chunk, max_chunks;
    float* carry;                                        // [sequences, max_chunks, heads, N, P]: the state a piece ends with, started from zero
    float* decay;                                        // [sequences, max_chunks, heads]: the product of its rows' decays
};

__device__ __forceinline__ float softplus_f(float v) { return log1pf(expf(-fabsf(v))) + fmaxf(v, 0.f); }

// A block of four waves owns R units of one group of heads, a unit being 64 value channels of one head: wave q keeps a
// quarter of the state's rows, lane p column p of them for each of the R units, R NR / 4 elements in registers, so that
// several blocks fit a SIMD and one's waits are another's work.  The rows' B and C vectors (one pair for the whole
// group, read from LDS once for all R units), step sizes, decays, inputs and gates are staged in LDS TC rows at a time
// (every load of a round is asked for at once); a row then costs a lane 3 R N / 4 vector instructions, and the four
// waves' parts of y meet in LDS once a round.  Rows of B and C stand NR apart in LDS, zero beyond N, so the inner loop
// has no bounds.  VEC: elements of B and C a load takes.
// MODE 0: the whole scan from the slot's state, which it leaves updated.
// MODE 1: a piece (not the last) from a zero state: writes the state it ends with and its total decay, no outputs.
// MODE 2: a piece from the state `carry` holds for its start: writes outputs; the last piece leaves the slot's state.
template <typename T, int NR, int MODE, int VEC, int R>
__global__ void __launch_bounds__(256)
ssd_scan_k(SsdArgs a) {
    constexpr int TC = 16 / R, NQ = NR / 4, PAIRS = TC * R;        // PAIRS = 16 (row, unit) pairs a round
    constexpr int J = (TC * NR / VEC + 255) / 256;       // packs of B (and of C) a thread stages a round
    using Pk = Pack<T, VEC>;
    extern __shared__ __attribute__((aligned(16))) float lds[];      // B [TC][NR], C [TC][NR], dt [PAIRS], decay [PAIRS], x [PAIRS][64], z [PAIRS][64], parts [4][PAIRS][64]
    const int seq = blockIdx.x, tid = threadIdx.x, lane = tid & 63, q = tid >> 6;
    const int N = a.N, P = a.P, hpg = a.heads / a.groups, pcs = (P + 63) / 64, units = hpg * pcs, bpg = (units + R - 1) / R;
    const int g = blockIdx.y / bpg, u0 = (blockIdx.y - g * bpg) * R;
    const int piece = MODE == 0 ? 0 : blockIdx.z;
    const int first = a.cu_rows[seq], count = a.cu_rows[seq + 1] - first;
    int r0 = first, r1 = first + count;
    if (MODE != 0) {
        r0 = first + piece * a.chunk;
        r1 = min(r0 + a.chunk, first + count);
        if (r0 >= r1) return;
    }
    const bool last_piece = MODE == 0 || r1 == first + count;
    if (MODE == 1 && last_piece) return;                 // nobody starts from the state the last piece ends with
    float* Bs = lds; float* Cs = lds + TC * NR; float* dts = Cs + TC * NR; float* dec = dts + PAIRS;
    float* xs = dec + PAIRS; float* zs = xs + PAIRS * 64; float* parts = zs + PAIRS * 64;
    // unit r of the block: its head, the lane's channel, whether the lane has one (worked out once: the divisions are
    // as many instructions as a row of the scan)
    int unit_head[R], unit_chan[R];
    bool unit_live[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int u = min(u0 + r, units - 1), hl = u / pcs;
        unit_head[r] = g * hpg + hl;
        unit_chan[r] = (u - hl * pcs) * 64 + lane;
        unit_live[r] = u0 + r < units && unit_chan[r] < P;
    }
    auto head_of = [&](int r) { int v = unit_head[0]; for (int i = 1; i < R; i++) v = r == i ? unit_head[i] : v; return v; };
    auto chan_of = [&](int r) { int v = unit_chan[0]; for (int i = 1; i < R; i++) v = r == i ? unit_chan[i] : v; return v; };
    auto live_of = [&](int r) { bool v = unit_live[0]; for (int i = 1; i < R; i++) v = r == i ? unit_live[i] : v; return v; };
    const int n0 = q * NQ;                               // the wave's rows of the state
    float S[R][NQ], total[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const bool live = live_of(r);
        const int head = head_of(r), p = live ? chan_of(r) : 0;
        const float* from = a.state + (((size_t)a.slot_ids[seq] * a.heads + head) * N) * P + p;
        if (MODE == 2) from = a.carry + ((((size_t)seq * a.max_chunks + piece) * a.heads + head) * N) * P + p;
        // all of them asked for at once, from addresses that exist, and masked afterwards: a load behind a condition is
        // waited for on the spot
        if (MODE != 1) {
#pragma unroll
            for (int n = 0; n < NQ; n++) S[r][n] = from[(size_t)min(n0 + n, N - 1) * P];
        }
#pragma unroll
        for (int n = 0; n < NQ; n++) S[r][n] = (MODE != 1 && live && n0 + n < N) ? S[r][n] : 0.f;
        total[r] = 1.f;
    }
    if (N < NR) {                                        // the columns beyond N stay zero
        for (int i = tid; i < 2 * TC * NR; i += 256) lds[i] = 0.f;
    }
    const size_t inner = (size_t)a.heads * P;
    // what does not change from round to round is fetched once, beside the state: the constants of the head whose step
    // size this thread prepares, and of the heads whose outputs it stores
    const int mt = min(tid, PAIRS - 1) / R, mr = min(tid, PAIRS - 1) % R;
    const float my_bias = a.dt_bias[head_of(mr)], my_rate = expf(a.a_log[head_of(mr)]);
    float skip[R];
#pragma unroll
    for (int r = 0; r < R; r++) skip[r] = a.skip[head_of(r)];
    for (int t0 = r0; t0 < r1; t0 += TC) {
        const int tn = min(TC, r1 - t0);
        // every load of the round is asked for before the first is used (loads past the round's end read its last row,
        // from an address that exists, and are dropped): a round waits for memory once
        const int per_row = N / VEC, packs = tn * per_row;
        Pk rb[J], rc[J];
        T rx[4], rz[4];
#pragma unroll
        for (int j = 0; j < J; j++) {
            const int c = min(tid + 256 * j, packs - 1), t = c / per_row, k = c - t * per_row;
            const T* row = (const T*)a.xbc + (size_t)(t0 + t) * a.xbc_stride + inner + (size_t)g * N + k * VEC;
            rb[j] = *reinterpret_cast<const Pk*>(row);
            rc[j] = *reinterpret_cast<const Pk*>(row + (size_t)a.groups * N);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {                    // pair q + 4 i of the round: row (q + 4 i) / R, unit (q + 4 i) % R
            const int pr = q + 4 * i, t = pr / R, r = pr % R;
            const size_t row = (size_t)(t0 + min(t, tn - 1));
            const int p = live_of(r) ? chan_of(r) : 0;
            rx[i] = *((const T*)a.xbc + row * a.xbc_stride + (size_t)head_of(r) * P + p);
            if (MODE != 1) rz[i] = *((const T*)a.z + row * a.z_stride + (size_t)head_of(r) * P + p);
        }
        const float draw = ld_f32((const T*)a.dt + (size_t)(t0 + min(mt, tn - 1)) * a.dt_stride + head_of(mr));
        __syncthreads();                                 // the round before has been read by every wave
#pragma unroll
        for (int j = 0; j < J; j++) {
            const int c = tid + 256 * j;
            if (c < packs) {
                const int t = c / per_row, k = c - t * per_row;
#pragma unroll
                for (int e = 0; e < VEC; e++) { Bs[t * NR + k * VEC + e] = ld_f32(&rb[j].v[e]); Cs[t * NR + k * VEC + e] = ld_f32(&rc[j].v[e]); }
            }
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int pr = q + 4 * i, r = pr % R;
            xs[pr * 64 + lane] = live_of(r) ? ld_f32(&rx[i]) : 0.f;
            if (MODE != 1) zs[pr * 64 + lane] = live_of(r) ? ld_f32(&rz[i]) : 0.f;
        }
        if (tid < PAIRS) {
            const float d = softplus_f(draw + my_bias);
            dts[tid] = d;
            dec[tid] = expf(-my_rate * d);
        }
        __syncthreads();
        for (int t = 0; t < tn; t++) {
            float d[R], dx[R], acc[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                d[r] = dec[t * R + r];
                dx[r] = dts[t * R + r] * xs[(t * R + r) * 64 + lane];
                acc[r] = 0.f;
            }
            // four neighbouring elements of B and of C a read (rows start on 16 bytes: NR and a wave's first row are multiples of 4)
            const float4* Bt = reinterpret_cast<const float4*>(Bs + t * NR + n0);
            const float4* Ct = reinterpret_cast<const float4*>(Cs + t * NR + n0);
#pragma unroll
            for (int n4 = 0; n4 < NQ / 4; n4++) {
                const float4 b4 = Bt[n4], c4 = Ct[n4];
                const float bn[4] = {b4.x, b4.y, b4.z, b4.w}, cn[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int n = 4 * n4 + e;
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        S[r][n] = __builtin_fmaf(d[r], S[r][n], dx[r] * bn[e]);
                        if (MODE != 1) acc[r] = __builtin_fmaf(S[r][n], cn[e], acc[r]);
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                if (MODE == 1) total[r] *= d[r];
                else parts[(q * PAIRS + t * R + r) * 64 + lane] = acc[r];
            }
        }
        if (MODE != 1) {
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 4; i++) {                // pair q + 4 i of the round: the four waves' parts in wave order
                const int pr = q + 4 * i, t = pr / R, r = pr % R;
                if (t < tn && live_of(r)) {
                    const float acc = ((parts[pr * 64 + lane] + parts[(PAIRS + pr) * 64 + lane]) + parts[(2 * PAIRS + pr) * 64 + lane]) +
                                      parts[(3 * PAIRS + pr) * 64 + lane];
                    const float zz = zs[pr * 64 + lane];
                    a.y[(size_t)(t0 + t) * inner + (size_t)head_of(r) * P + chan_of(r)] =
                        __builtin_fmaf(skip[r], xs[pr * 64 + lane], acc) * (zz / (1.f + expf(-zz)));
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (u0 + r >= units) continue;
        const int head = head_of(r), p = chan_of(r);
        if (MODE == 1) {
            float* to = a.carry + ((((size_t)seq * a.max_chunks + piece) * a.heads + head) * N) * P + p;
            if (p < P) {
#pragma unroll
                for (int n = 0; n < NQ; n++) if (n0 + n < N) to[(size_t)(n0 + n) * P] = S[r][n];
            }
            if (tid == 0 && (u0 + r) % pcs == 0) a.decay[((size_t)seq * a.max_chunks + piece) * a.heads + head] = total[r];
        } else if (last_piece && p < P) {
            float* slot_state = a.state + (((size_t)a.slot_ids[seq] * a.heads + head) * N) * P + p;
#pragma unroll
            for (int n = 0; n < NQ; n++) if (n0 + n < N) slot_state[(size_t)(n0 + n) * P] = S[r][n];
        }
    }
}

// The states at the pieces' starts from the pieces' own end states: walking the pieces, carry[c] (what piece c ends
// with when started from zero) gives way to the state piece c starts from, s, and s <- decay[c] s + carry[c].
// grid (sequences, heads, blocks of N P / 256)
__global__ void __launch_bounds__(256)
ssd_carry_k(SsdArgs a) {
    const int seq = blockIdx.x, head = blockIdx.y;
    const int e = blockIdx.z * 256 + threadIdx.x, NP = a.N * a.P;
    if (e >= NP) return;
    const int count = a.cu_rows[seq + 1] - a.cu_rows[seq];
    const int pieces = (count + a.chunk - 1) / a.chunk;
    float s = a.state[((size_t)a.slot_ids[seq] * a.heads + head) * NP + e];
    for (int c = 0; c < pieces; c++) {
        float* at = a.carry + (((size_t)seq * a.max_chunks + c) * a.heads + head) * NP + e;
        const float ended = c + 1 < pieces ? *at : 0.f;  // the last piece wrote none
        *at = s;
        if (c + 1 < pieces) s = __builtin_fmaf(a.decay[((size_t)seq * a.max_chunks + c) * a.heads + head], s, ended);
    }
}

// Units of 64 channels a block takes.  Two (where a group of heads has two), which halves the reads of B and C from LDS,
// measured slower than one (209 against 170 us for 2,048 rows of 36 heads x 64 channels with a state of 128; a decode step
// 9.2 against 8.2): the kernel keeps the parameter, one unit is what is compiled.
static int scan_units(const SsdArgs&) { return 1; }
static int scan_nr(int N) { return N <= 16 ? 16 : N <= 32 ? 32 : N <= 64 ? 64 : N <= 128 ? 128 : 256; }
static size_t scan_lds(int N) { return (size_t)(2 * 16 * scan_nr(N) + 32 + 6 * 16 * 64) * sizeof(float); }     // 16 rows x 1 unit, or 8 x 2

template <typename T, int MODE>
static int launch_scan(const SsdArgs& a, int n_seq, int pieces, hipStream_t s) {
    constexpr int V = sizeof(T) == 2 ? 8 : 4;             // 16 bytes of B or C a load, where rows and sizes allow
    const bool packs = a.N % V == 0 && a.xbc_stride % V == 0 && ((size_t)a.heads * a.P) % V == 0 && (uintptr_t)a.xbc % 16 == 0;
    const int R = scan_units(a), units = (a.heads / a.groups) * ((a.P + 63) / 64);
    dim3 grid(n_seq, a.groups * ((units + R - 1) / R), pieces);
    const size_t lds = scan_lds(a.N);
#define TP_SSD(NR) do { \
        if (packs) ssd_scan_k<T, NR, MODE, V, 1><<<grid, 256, lds, s>>>(a); \
        else ssd_scan_k<T, NR, MODE, 1, 1><<<grid, 256, lds, s>>>(a); } while (0)
    switch (scan_nr(a.N)) {
        case 16: TP_SSD(16); break;
        case 32: TP_SSD(32); break;
        case 64: TP_SSD(64); break;
        case 128: TP_SSD(128); break;
        default: TP_SSD(256);
    }
#undef TP_SSD
    return tp_check_launch("ssd_scan");
}

extern "C" long tp_ssd_scan_workspace_bytes(int n_seq, int max_count, int heads, int N, int P, int chunk) {
    if (chunk <= 0 || max_count <= chunk) return 0;
    const long pieces = (max_count + chunk - 1) / chunk;
    return (long)n_seq * pieces * heads * ((long)N * P + 1) * (long)sizeof(float);
}

// chunk 0: one pass per sequence.  chunk > 0 and a sequence longer than it: three passes over pieces of `chunk` rows.
extern "C" int tp_ssd_scan(const void* xbc, long xbc_stride, const void* z, long z_stride, const void* dt, long dt_stride, int dtype,
                           const float* dt_bias, const float* a_log, const float* skip, float* state, const int* slot_ids,
                           const int* cu_rows, float* y, int n_seq, int max_count, int heads, int groups, int N, int P,
                           int chunk, void* workspace, long workspace_bytes, void* stream) {
    TP_REQUIRE(n_seq > 0 && max_count > 0 && heads > 0 && groups > 0 && N > 0 && P > 0, "ssd_scan: empty shape sequences=%d heads=%d groups=%d N=%d P=%d", n_seq, heads, groups, N, P);
    TP_REQUIRE(heads % groups == 0, "ssd_scan: %d heads are no multiple of %d groups", heads, groups);
    TP_REQUIRE(N <= 256, "ssd_scan: a state of %d rows per head exceeds 256", N);
    TP_REQUIRE(xbc && z && dt && dt_bias && a_log && skip && state && slot_ids && cu_rows && y, "ssd_scan: a null operand");
    TP_REQUIRE(dtype == TP_BF16 || dtype == TP_F32, "ssd_scan: unknown dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    SsdArgs a{};
    a.xbc = xbc; a.xbc_stride = xbc_stride; a.z = z; a.z_stride = z_stride; a.dt = dt; a.dt_stride = dt_stride;
    a.dt_bias = dt_bias; a.a_log = a_log; a.skip = skip; a.state = state; a.slot_ids = slot_ids; a.cu_rows = cu_rows; a.y = y;
    a.heads = heads; a.groups = groups; a.N = N; a.P = P;
    TP_REQUIRE((long)a.groups * (a.heads / a.groups) * ((P + 63) / 64) <= 65535, "ssd_scan: too many heads or channels for one launch");
    const long need = tp_ssd_scan_workspace_bytes(n_seq, max_count, heads, N, P, chunk);
    if (need == 0)
        return dtype == TP_BF16 ? launch_scan<bf16_t, 0>(a, n_seq, 1, s) : launch_scan<float, 0>(a, n_seq, 1, s);
    TP_REQUIRE(workspace && workspace_bytes >= need, "ssd_scan: a workspace of %ld bytes is too small (%ld)", workspace_bytes, need);
    a.chunk = chunk; a.max_chunks = (max_count + chunk - 1) / chunk;
    TP_REQUIRE(a.max_chunks <= 65535, "ssd_scan: %d pieces exceed one launch", a.max_chunks);
    a.carry = (float*)workspace;
    a.decay = a.carry + (size_t)n_seq * a.max_chunks * heads * N * P;
    if (int rc = dtype == TP_BF16 ? launch_scan<bf16_t, 1>(a, n_seq, a.max_chunks, s) : launch_scan<float, 1>(a, n_seq, a.max_chunks, s)) return rc;
    ssd_carry_k<<<dim3(n_seq, heads, tp_cdiv((long)N * P, 256)), 256, 0, s>>>(a);
    if (int rc = tp_check_launch("ssd_scan (carry)")) return rc;
    return dtype == TP_BF16 ? launch_scan<bf16_t, 2>(a, n_seq, a.max_chunks, s) : launch_scan<float, 2>(a, n_seq, a.max_chunks, s);
}

// ---- 0.5 (a / rms(a) * wa + b / rms(b) * wb), one block a row ------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
pair_norm_mean_k(const T* __restrict__ a, const T* __restrict__ b, const float* __restrict__ wa, const float* __restrict__ wb,
                 float eps, float* __restrict__ out, int D) {
    __shared__ float red[32];
    const T* ar = a + (size_t)blockIdx.x * D; const T* br = b + (size_t)blockIdx.x * D;
    float sa = 0.f, sb = 0.f;
    for (int i = threadIdx.x; i < D; i += 256) { const float x = ld_f32(ar + i), y = ld_f32(br + i); sa += x * x; sb += y * y; }
    sa = block_sum_once(sa, red);
    sb = block_sum_once(sb, red + 16);
    const float ra = rsqrtf(sa / (float)D + eps), rb = rsqrtf(sb / (float)D + eps);
    float* o = out + (size_t)blockIdx.x * D;
    for (int i = threadIdx.x; i < D; i += 256) o[i] = 0.5f * ((ld_f32(ar + i) * ra) * wa[i] + (ld_f32(br + i) * rb) * wb[i]);
}

extern "C" int tp_pair_norm_mean(const void* a, const void* b, int dtype, const float* wa, const float* wb, float eps, float* out,
                                 int M, int D, void* stream) {
    TP_REQUIRE(M > 0 && D > 0 && a && b && wa && wb && out, "pair_norm_mean: empty shape or null operand (M=%d D=%d)", M, D);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TP_BF16) pair_norm_mean_k<bf16_t><<<M, 256, 0, s>>>((const bf16_t*)a, (const bf16_t*)b, wa, wb, eps, out, D);
    else if (dtype == TP_F32) pair_norm_mean_k<float><<<M, 256, 0, s>>>((const float*)a, (const float*)b, wa, wb, eps, out, D);
    else return tp_fail("pair_norm_mean: unknown dtype %d", dtype);
    return tp_check_launch("pair_norm_mean");
}

// ---- x[r, c] *= sigmoid(g[r, c]) ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
mul_sigmoid_k(T* __restrict__ x, long x_stride, const T* __restrict__ g, long g_stride, int M, int C) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= (long)M * C) return;
    const long r = i / C, c = i - r * C;
    T* xp = x + r * x_stride + c;
    const float gv = ld_f32(g + r * g_stride + c);
    st_f32(xp, ld_f32(xp) / (1.f + expf(-gv)));
}

extern "C" int tp_mul_sigmoid(void* x, long x_stride, const void* g, long g_stride, int dtype, int M, int C, void* stream) {
    TP_REQUIRE(M > 0 && C > 0 && x && g, "mul_sigmoid: empty shape or null operand (M=%d C=%d)", M, C);
    hipStream_t s = (hipStream_t)stream;
    const int blocks = tp_cdiv((long)M * C, 256);
    if (dtype == TP_BF16) mul_sigmoid_k<bf16_t><<<blocks, 256, 0, s>>>((bf16_t*)x, x_stride, (const bf16_t*)g, g_stride, M, C);
    else if (dtype == TP_F32) mul_sigmoid_k<float><<<blocks, 256, 0, s>>>((float*)x, x_stride, (const float*)g, g_stride, M, C);
    else return tp_fail("mul_sigmoid: unknown dtype %d", dtype);
    return tp_check_launch("mul_sigmoid");
}
