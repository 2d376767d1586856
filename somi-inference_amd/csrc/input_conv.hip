// A short causal convolution over time on every channel of the residual stream, added to its input:
//
//     out[t, c] = h[t, c] + sum_d taps[c, last - d] * h[t - d, c],   d = 0 .. taps - 1,   zeros before a sequence's start
//
// The step's rows are float32; what lies before an entry's first token comes from the request's state, its last
// taps - 1 rows (oldest first), which a second kernel brings up to date after the first has read it.  The sums are
// float32 and run in one order per (token, channel) however a prompt is cut; the result is rounded once to the compute
// dtype.
#include "common.h"

#define CONV_MAX_TAPS 17

template <typename TO>
__global__ void __launch_bounds__(256)
input_conv_kernel(const float* __restrict__ h, const float* __restrict__ taps_w, int taps,
                  const float* __restrict__ state, const int* __restrict__ token_entry,
                  const int* __restrict__ entry_start, const int* __restrict__ state_slots, int C,
                  TO* __restrict__ out) {
    const int64_t t = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int e = token_entry[t];
    const int i = (int)t - entry_start[e];
    const int64_t slot = state_slots[e];
    float acc = 0.f;
    // oldest input first, so that the order of the additions is the order of time
#pragma unroll
    for (int d = CONV_MAX_TAPS - 1; d >= 0; --d) {
        if (d >= taps) continue;
        const float w = taps_w[c * taps + taps - 1 - d];
        const float xv = i - d >= 0 ? h[(t - d) * C + c] : state[(slot * (taps - 1) + (taps - 1 + i - d)) * C + c];
        acc = fmaf(w, xv, acc);
    }
    out[t * C + c] = from_float<TO>(h[t * C + c] + acc);
}

// A thread reads all of a channel's values before it writes any, so entries shorter than the taps shift the state.
__global__ void __launch_bounds__(256)
input_conv_state_kernel(const float* __restrict__ h, int taps, float* __restrict__ state,
                        const int* __restrict__ entry_start, const int* __restrict__ state_slots, int C) {
    const int e = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int start = entry_start[e], len = entry_start[e + 1] - start;
    float* st = state + (int64_t)state_slots[e] * (taps - 1) * C;
    float vals[CONV_MAX_TAPS - 1];
#pragma unroll
    for (int s = 0; s < CONV_MAX_TAPS - 1; ++s) {
        if (s >= taps - 1) break;
        const int j = len - (taps - 1) + s;          // index among the entry's tokens; negative: before the entry
        vals[s] = j >= 0 ? h[(int64_t)(start + j) * C + c] : st[(taps - 1 + j) * C + c];
    }
#pragma unroll
    for (int s = 0; s < CONV_MAX_TAPS - 1; ++s) {
        if (s >= taps - 1) break;
        st[s * C + c] = vals[s];
    }
}

// h: [n_tokens, C] float32; taps_w: [C, taps] float32; state: [slots, max(taps - 1, 1), C] float32, read and then
// advanced by the step's entries; out: [n_tokens, C] in out_dtype.
extern "C" int somi_input_conv(const float* h, const float* taps_w, int taps, float* state, const int* token_entry,
                               const int* entry_start, const int* state_slots, int n_tokens, int n_entries, int C,
                               void* out, int out_dtype, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && n_entries >= 0 && C > 0, "input_conv: bad sizes");
    SOMI_REQUIRE(taps >= 1 && taps <= CONV_MAX_TAPS, "input_conv: %d taps, 1 to %d are supported", taps, CONV_MAX_TAPS);
    SOMI_REQUIRE(ceil_div(C, 256) <= 65535, "input_conv: too many channels");
    if (n_tokens == 0) return 0;
    const dim3 grid(n_tokens, ceil_div(C, 256));
    if (out_dtype == SOMI_F32)
        hipLaunchKernelGGL(input_conv_kernel<float>, grid, dim3(256), 0, stream, h, taps_w, taps, state, token_entry,
                           entry_start, state_slots, C, (float*)out);
    else if (out_dtype == SOMI_BF16)
        hipLaunchKernelGGL(input_conv_kernel<bf16>, grid, dim3(256), 0, stream, h, taps_w, taps, state, token_entry,
                           entry_start, state_slots, C, (bf16*)out);
    else
        return somi_fail("input_conv: unknown dtype %d", out_dtype);
    SOMI_LAUNCH_CHECK("input_conv");
    if (taps > 1 && n_entries > 0) {
        hipLaunchKernelGGL(input_conv_state_kernel, dim3(n_entries, ceil_div(C, 256)), dim3(256), 0, stream, h, taps,
                           state, entry_start, state_slots, C);
        SOMI_LAUNCH_CHECK("input_conv_state");
    }
    return 0;
}
