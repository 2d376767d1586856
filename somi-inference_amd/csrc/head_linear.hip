// Per-head matrix products: every head has a small matrix of its own, and head h of every row is multiplied by
// matrix h,
//
//     out[t, h, :] = W[h] x[t, h, :],        W: [heads, n_out, K],   x[t, h, :] at x + t * x_row + h * x_head
//
// The plain kernel: a workgroup owns 16 rows x 64 outputs of one head, x and W tiles go through LDS 32 channels at a
// time, float32 sums in one order per output.
#include "common.h"

#define HL_ROWS 16
#define HL_COLS 64
#define HL_K 32

template <typename T>
__global__ void __launch_bounds__(256)
head_linear_plain_kernel(const T* __restrict__ x, int64_t x_row, int64_t x_head, const T* __restrict__ w, int n_rows,
                         int n_out, int K, T* __restrict__ out, int64_t out_row, int64_t out_head) {
    __shared__ float xs[HL_ROWS][HL_K + 1];
    __shared__ float ws[HL_COLS][HL_K + 1];
    const int h = blockIdx.z;
    const int row0 = blockIdx.x * HL_ROWS, col0 = blockIdx.y * HL_COLS;
    const int tid = threadIdx.x;
    const int c = tid & 63, rg = tid >> 6;            // a thread: output column c, rows rg, rg + 4, rg + 8, rg + 12
    const T* wh = w + (int64_t)h * n_out * K;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < K; k0 += HL_K) {
        __syncthreads();
        for (int i = tid; i < HL_ROWS * HL_K; i += 256) {
            const int r = i / HL_K, k = i % HL_K;
            xs[r][k] = (row0 + r < n_rows && k0 + k < K) ? to_float(x[(int64_t)(row0 + r) * x_row + h * x_head + k0 + k]) : 0.f;
        }
        for (int i = tid; i < HL_COLS * HL_K; i += 256) {
            const int o = i / HL_K, k = i % HL_K;
            ws[o][k] = (col0 + o < n_out && k0 + k < K) ? to_float(wh[(int64_t)(col0 + o) * K + k0 + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int k = 0; k < HL_K; ++k) {
            const float wv = ws[c][k];
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] = fmaf(xs[rg + 4 * j][k], wv, acc[j]);
        }
    }
    if (col0 + c < n_out)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int r = row0 + rg + 4 * j;
            if (r < n_rows) out[(int64_t)r * out_row + h * out_head + col0 + c] = from_float<T>(acc[j]);
        }
}

extern "C" int somi_head_linear(const void* x, int64_t x_row, int64_t x_head, const void* w, int dtype, int n_rows,
                                int heads, int n_out, int K, void* out, int64_t out_row, int64_t out_head,
                                hipStream_t stream) {
    SOMI_REQUIRE(n_rows >= 0 && heads > 0 && n_out > 0 && K > 0, "head_linear: bad sizes");
    SOMI_REQUIRE(heads <= 65535 && ceil_div(n_out, HL_COLS) <= 65535, "head_linear: too many heads or columns");
    if (n_rows == 0) return 0;
    const dim3 grid(ceil_div(n_rows, HL_ROWS), ceil_div(n_out, HL_COLS), heads);
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(head_linear_plain_kernel<float>, grid, dim3(256), 0, stream, (const float*)x, x_row, x_head,
                           (const float*)w, n_rows, n_out, K, (float*)out, out_row, out_head);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(head_linear_plain_kernel<bf16>, grid, dim3(256), 0, stream, (const bf16*)x, x_row, x_head,
                           (const bf16*)w, n_rows, n_out, K, (bf16*)out, out_row, out_head);
    else
        return somi_fail("head_linear: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("head_linear");
    return 0;
}
