// A short causal convolution over time on every channel of the fp32 stream, with the rows before a step kept as a
// state per sequence:  out[r] = (x[r]) + sum_j w[:, j] * x[r - (taps - 1) + j], rows before the sequence's start zero.
#include "common.h"

// grid (rows, channel blocks).  state: [slots, taps - 1, D], oldest row first; a row of the step whose tap reaches
// before the step's first row reads there.  one_row_each: every sequence brings one row, and the thread that read
// the state's column moves it on by that row.
// The same for widths in whole 16-byte pieces: a thread takes four neighbouring channels; wt is the taps transposed, [taps, D].
template <typename T>
__global__ void __launch_bounds__(256)
causal_conv_vec_k(const float* __restrict__ x, const float* __restrict__ wt, float* __restrict__ state,
                  const int* __restrict__ slot_ids, const int* __restrict__ cu_rows, const int* __restrict__ row_seq,
                  T* __restrict__ out, int D, int taps, int residual, int one_row_each) {
    const int r = blockIdx.x, d = (blockIdx.y * blockDim.x + threadIdx.x) * 4;
    if (d >= D) return;
    const int seq = row_seq[r], i = r - cu_rows[seq], S = taps - 1;
    float* st = S > 0 ? state + (size_t)slot_ids[seq] * S * D + d : nullptr;
    const float4 xr = *reinterpret_cast<const float4*>(x + (size_t)r * D + d);
    float4 acc = residual ? xr : make_float4(0.f, 0.f, 0.f, 0.f);
    for (int j = 0; j < taps; j++) {
        const int src = i - (S - j);
        const float4 v = src >= 0 ? *reinterpret_cast<const float4*>(x + (size_t)(r - (S - j)) * D + d)
                                  : *reinterpret_cast<const float4*>(st + (size_t)(S + src) * D);
        const float4 wv = *reinterpret_cast<const float4*>(wt + (size_t)j * D + d);
        acc.x = __builtin_fmaf(wv.x, v.x, acc.x); acc.y = __builtin_fmaf(wv.y, v.y, acc.y);
        acc.z = __builtin_fmaf(wv.z, v.z, acc.z); acc.w = __builtin_fmaf(wv.w, v.w, acc.w);
    }
    T* o = out + (size_t)r * D + d;
    if constexpr (sizeof(T) == 2) {
        uint2 pk;
        pk.x = (uint32_t)f32_to_bf16(acc.x) | ((uint32_t)f32_to_bf16(acc.y) << 16);
        pk.y = (uint32_t)f32_to_bf16(acc.z) | ((uint32_t)f32_to_bf16(acc.w) << 16);
        *reinterpret_cast<uint2*>(o) = pk;
    } else *reinterpret_cast<float4*>(o) = acc;
    if (one_row_each && S > 0) {
        for (int s = 0; s + 1 < S; s++)
            *reinterpret_cast<float4*>(st + (size_t)s * D) = *reinterpret_cast<const float4*>(st + (size_t)(s + 1) * D);
        *reinterpret_cast<float4*>(st + (size_t)(S - 1) * D) = xr;
    }
}

template <typename T>
__global__ void __launch_bounds__(256)
causal_conv_k(const float* __restrict__ x, const float* __restrict__ w, float* __restrict__ state,
              const int* __restrict__ slot_ids, const int* __restrict__ cu_rows, const int* __restrict__ row_seq,
              T* __restrict__ out, int D, int taps, int residual, int one_row_each) {
    const int r = blockIdx.x, d = blockIdx.y * 256 + threadIdx.x;
    if (d >= D) return;
    const int seq = row_seq[r], i = r - cu_rows[seq], S = taps - 1;
    float* st = S > 0 ? state + (size_t)slot_ids[seq] * S * D + d : nullptr;
    const float xr = x[(size_t)r * D + d];
    float acc = residual ? xr : 0.f;
    for (int j = 0; j < taps; j++) {
        const int src = i - (S - j);                     // the step's row this tap reads, negative: before the step
        const float v = src >= 0 ? x[(size_t)(r - (S - j)) * D + d] : st[(size_t)(S + src) * D];
        acc = __builtin_fmaf(w[(size_t)d * taps + j], v, acc);
    }
    st_f32(out + (size_t)r * D + d, acc);
    if (one_row_each && S > 0) {
        for (int s = 0; s + 1 < S; s++) st[(size_t)s * D] = st[(size_t)(s + 1) * D];
        st[(size_t)(S - 1) * D] = xr;
    }
}

// grid (sequences, channel blocks): the state takes the last taps - 1 rows of (state, the step's rows)
__global__ void __launch_bounds__(256)
causal_conv_state_k(const float* __restrict__ x, float* __restrict__ state, const int* __restrict__ slot_ids,
                    const int* __restrict__ cu_rows, int D, int taps) {
    const int seq = blockIdx.x, d = blockIdx.y * 256 + threadIdx.x;
    if (d >= D) return;
    const int first = cu_rows[seq], count = cu_rows[seq + 1] - first, S = taps - 1;
    float* st = state + (size_t)slot_ids[seq] * S * D + d;
    for (int s = 0; s < S; s++) {                        // ascending: a row of the old state is read before it is overwritten
        const int src = count - S + s;
        st[(size_t)s * D] = src >= 0 ? x[(size_t)(first + src) * D + d] : st[(size_t)(s + count) * D];
    }
}

extern "C" int tp_causal_conv(const float* x, const float* w, const float* wt, float* state, const int* slot_ids, const int* cu_rows,
                              const int* row_seq, void* out, int out_dtype, int M, int n_seq, int D, int taps,
                              int residual, int one_row_each, void* stream) {
    TP_REQUIRE(M > 0 && n_seq > 0 && D > 0 && taps >= 1, "causal_conv: empty shape M=%d sequences=%d D=%d taps=%d", M, n_seq, D, taps);
    TP_REQUIRE(x && w && out && cu_rows && row_seq, "causal_conv: a null operand");
    TP_REQUIRE(taps == 1 || (state && slot_ids), "causal_conv: %d taps need the sequences' states", taps);
    TP_REQUIRE(!one_row_each || M == n_seq, "causal_conv: one row each, but %d rows for %d sequences", M, n_seq);
    hipStream_t s = (hipStream_t)stream;
    if (wt && D % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)wt % 16 == 0 && (uintptr_t)out % 16 == 0 && (!state || (uintptr_t)state % 16 == 0) &&
        (out_dtype == TP_BF16 || out_dtype == TP_F32)) {
        const int chunks = D / 4, threads = chunks >= 256 ? 256 : (chunks + 63) / 64 * 64;
        dim3 vgrid(M, tp_cdiv(chunks, threads));
        if (out_dtype == TP_BF16) causal_conv_vec_k<bf16_t><<<vgrid, threads, 0, s>>>(x, wt, state, slot_ids, cu_rows, row_seq, (bf16_t*)out, D, taps, residual, one_row_each);
        else causal_conv_vec_k<float><<<vgrid, threads, 0, s>>>(x, wt, state, slot_ids, cu_rows, row_seq, (float*)out, D, taps, residual, one_row_each);
        if (int rc = tp_check_launch("causal_conv")) return rc;
        if (taps > 1 && !one_row_each) {
            causal_conv_state_k<<<dim3(n_seq, tp_cdiv(D, 256)), 256, 0, s>>>(x, state, slot_ids, cu_rows, D, taps);
            return tp_check_launch("causal_conv (state)");
        }
        return 0;
    }
    dim3 grid(M, tp_cdiv(D, 256));
    if (out_dtype == TP_BF16) causal_conv_k<bf16_t><<<grid, 256, 0, s>>>(x, w, state, slot_ids, cu_rows, row_seq, (bf16_t*)out, D, taps, residual, one_row_each);
    else if (out_dtype == TP_F32) causal_conv_k<float><<<grid, 256, 0, s>>>(x, w, state, slot_ids, cu_rows, row_seq, (float*)out, D, taps, residual, one_row_each);
    else return tp_fail("causal_conv: unknown dtype %d", out_dtype);
    if (int rc = tp_check_launch("causal_conv")) return rc;
    if (taps > 1 && !one_row_each) {
        causal_conv_state_k<<<dim3(n_seq, tp_cdiv(D, 256)), 256, 0, s>>>(x, state, slot_ids, cu_rows, D, taps);
        return tp_check_launch("causal_conv (state)");
    }
    return 0;
}
