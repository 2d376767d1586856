// Layer norm with weight and bias over rows, in float32 statistics:
//
//     ln(y) = (y - mean(y)) / sqrt(mean((y - mean(y))^2) + eps) * w + b
//
// Two entry points: the norm of the float32 residual rows themselves (rounded once to the compute dtype), and the
// add of a sublayer's normed output into the residual stream, h += ln(y), which can also leave the new rows in the
// compute dtype for the next sublayer to read.  One workgroup per row; the mean is taken first and the variance from
// the deviations, so a row of nearly equal values keeps its digits.
#include "common.h"

template <typename TY>
__device__ __forceinline__ void row_stats(const TY* __restrict__ y, int width, float eps, float* red, float& mean,
                                          float& inv) {
    float s = 0.f;
    for (int i = threadIdx.x; i < width; i += 256) s += to_float(y[i]);
    mean = block_sum<256>(s, red) / (float)width;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += 256) {
        const float d = to_float(y[i]) - mean;
        ss = fmaf(d, d, ss);
    }
    inv = 1.0f / sqrtf(block_sum<256>(ss, red) / (float)width + eps);
}

template <typename TO>
__global__ void __launch_bounds__(256)
layernorm_kernel(const float* __restrict__ h, const float* __restrict__ w, const float* __restrict__ b, float eps,
                 TO* __restrict__ out, int width) {
    __shared__ float red[16];
    const float* row = h + (int64_t)blockIdx.x * width;
    float mean, inv;
    row_stats(row, width, eps, red, mean, inv);
    TO* o = out + (int64_t)blockIdx.x * width;
    for (int i = threadIdx.x; i < width; i += 256) o[i] = from_float<TO>(fmaf((row[i] - mean) * inv, w[i], b[i]));
}

// h: [n, width] float32; out: [n, width] in out_dtype.
extern "C" int somi_layernorm(const float* h, const float* w, const float* b, float eps, void* out, int out_dtype, int n,
                              int width, hipStream_t stream) {
    SOMI_REQUIRE(n >= 0 && width > 0, "layernorm: bad sizes n=%d width=%d", n, width);
    if (n == 0) return 0;
    if (out_dtype == SOMI_F32)
        hipLaunchKernelGGL(layernorm_kernel<float>, dim3(n), dim3(256), 0, stream, h, w, b, eps, (float*)out, width);
    else if (out_dtype == SOMI_BF16)
        hipLaunchKernelGGL(layernorm_kernel<bf16>, dim3(n), dim3(256), 0, stream, h, w, b, eps, (bf16*)out, width);
    else
        return somi_fail("layernorm: unknown dtype %d", out_dtype);
    SOMI_LAUNCH_CHECK("layernorm");
    return 0;
}

template <typename TY, typename TC, bool COPY>
__global__ void __launch_bounds__(256)
layernorm_add_kernel(float* __restrict__ h, const TY* __restrict__ y, const float* __restrict__ w,
                     const float* __restrict__ b, float eps, TC* __restrict__ copy, int width) {
    __shared__ float red[16];
    const TY* row = y + (int64_t)blockIdx.x * width;
    float mean, inv;
    row_stats(row, width, eps, red, mean, inv);
    float* hr = h + (int64_t)blockIdx.x * width;
    for (int i = threadIdx.x; i < width; i += 256) {
        const float v = hr[i] + fmaf((to_float(row[i]) - mean) * inv, w[i], b[i]);
        hr[i] = v;
        if (COPY) copy[(int64_t)blockIdx.x * width + i] = from_float<TC>(v);
    }
}

// h += ln(y) in place on float32 rows; y: [n, width] in y_dtype; copy (may be null): the new rows in copy_dtype.
extern "C" int somi_layernorm_add(float* h, const void* y, int y_dtype, const float* w, const float* b, float eps,
                                  void* copy, int copy_dtype, int n, int width, hipStream_t stream) {
    SOMI_REQUIRE(n >= 0 && width > 0, "layernorm_add: bad sizes n=%d width=%d", n, width);
    SOMI_REQUIRE(y_dtype == SOMI_F32 || y_dtype == SOMI_BF16, "layernorm_add: unknown dtype %d", y_dtype);
    SOMI_REQUIRE(copy == nullptr || copy_dtype == SOMI_F32 || copy_dtype == SOMI_BF16, "layernorm_add: unknown copy dtype %d", copy_dtype);
    if (n == 0) return 0;
#define SOMI_LNA(TY, TC, COPY)                                                                                      \
    hipLaunchKernelGGL((layernorm_add_kernel<TY, TC, COPY>), dim3(n), dim3(256), 0, stream, h, (const TY*)y, w, b, eps, \
                       (TC*)copy, width)
    if (y_dtype == SOMI_F32) {
        if (copy == nullptr) SOMI_LNA(float, float, false);
        else if (copy_dtype == SOMI_F32) SOMI_LNA(float, float, true);
        else SOMI_LNA(float, bf16, true);
    } else {
        if (copy == nullptr) SOMI_LNA(bf16, float, false);
        else if (copy_dtype == SOMI_F32) SOMI_LNA(bf16, float, true);
        else SOMI_LNA(bf16, bf16, true);
    }
#undef SOMI_LNA
    SOMI_LAUNCH_CHECK("layernorm_add");
    return 0;
}
