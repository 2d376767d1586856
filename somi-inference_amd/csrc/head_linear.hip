// Per-head matrix products: every head has a small matrix of its own, and head h of every row is multiplied by
// matrix h,
//
//     out[t, h, :] = W[h] x[t, h, :],        W: [heads, n_out, K],   x[t, h, :] at x + t * x_row + h * x_head
//
// The plain kernel: a workgroup owns 16 rows x 64 outputs of one head, x and W tiles go through LDS 32 channels at a
// time, float32 sums in one order per output.  The matrix-core kernel (bfloat16, K and the strides multiples of 8,
// outputs a multiple of 16): a workgroup owns 64 rows x 64 outputs of one head, a wavefront 16 of the rows; out^T = W x^T
// by `16x16x32` products whose fragments come straight from memory (16 bytes a lane, K contiguous in both operands), so
// a lane ends with 4 consecutive outputs of one row.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 hl_bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 hl_bf16x4;
typedef __attribute__((ext_vector_type(4))) float hl_f32x4;
#define HLM_ROWS 64
#define HLM_TILES 4               // 16-output tiles of a workgroup

__global__ void __launch_bounds__(256)
head_linear_mfma_kernel(const bf16* __restrict__ x, int64_t x_row, int64_t x_head, const bf16* __restrict__ w, int n_rows,
                        int n_out, int K, bf16* __restrict__ out, int64_t out_row, int64_t out_head) {
    const int h = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const int row = blockIdx.x * HLM_ROWS + wave * 16 + col;
    const int out0 = blockIdx.y * (HLM_TILES * 16);
    const bf16* xr = x + (int64_t)min(row, n_rows - 1) * x_row + h * x_head;
    const bf16* wh = w + (int64_t)h * n_out * K;
    hl_f32x4 acc[HLM_TILES];
#pragma unroll
    for (int j = 0; j < HLM_TILES; ++j) acc[j] = hl_f32x4{0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < K; k0 += 32) {
        const int k = k0 + quad * 8;
        hl_bf16x8 xf, wf[HLM_TILES];
#pragma unroll
        for (int i = 0; i < 8; ++i) xf[i] = (__bf16)0.f;
        if (k < K) xf = *reinterpret_cast<const hl_bf16x8*>(xr + k);
#pragma unroll
        for (int j = 0; j < HLM_TILES; ++j) {
            const int o = out0 + j * 16 + col;
#pragma unroll
            for (int i = 0; i < 8; ++i) wf[j][i] = (__bf16)0.f;
            if (k < K && o < n_out) wf[j] = *reinterpret_cast<const hl_bf16x8*>(wh + (int64_t)o * K + k);
        }
#pragma unroll
        for (int j = 0; j < HLM_TILES; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j], xf, acc[j], 0, 0, 0);
    }
    if (row >= n_rows) return;
#pragma unroll
    for (int j = 0; j < HLM_TILES; ++j) {
        const int o = out0 + j * 16 + quad * 4;
        if (o >= n_out) continue;
        hl_bf16x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = (__bf16)acc[j][i];
        *reinterpret_cast<hl_bf16x4*>(out + (int64_t)row * out_row + h * out_head + o) = v;
    }
}

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
    if (dtype == SOMI_BF16 && K % 8 == 0 && n_out % 16 == 0 && x_row % 8 == 0 && x_head % 8 == 0 && out_row % 4 == 0
        && out_head % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0 && (uintptr_t)out % 8 == 0) {
        const dim3 tiles(ceil_div(n_rows, HLM_ROWS), ceil_div(n_out, HLM_TILES * 16), heads);
        hipLaunchKernelGGL(head_linear_mfma_kernel, tiles, dim3(256), 0, stream, (const bf16*)x, x_row, x_head,
                           (const bf16*)w, n_rows, n_out, K, (bf16*)out, out_row, out_head);
        SOMI_LAUNCH_CHECK("head_linear_mfma");
        return 0;
    }
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
