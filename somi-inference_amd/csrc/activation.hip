// SwiGLU gate: out[t, i] = silu(gu[t, i]) * gu[t, I + i], silu(z) = z * sigmoid(z).
// Reference: somi_inference/models/qwen2.py:226-229 (chunk(2) of the merged projection, SiLU on the first half).
#include "common.h"

// block == 0: gu = [gate columns | up columns]; block == b > 0: gate and up columns interleaved in blocks of b
// (gate 0..b-1, up 0..b-1, gate b..2b-1, ...), the layout the fused decode kernel's weight has.
template <typename T>
__global__ void __launch_bounds__(256)
silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, int block, int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) {
        const int64_t t = i / inter;
        const int c = (int)(i - t * inter);
        const int at_gate = block > 0 ? (c / block) * 2 * block + c % block : c;
        const int at_up = block > 0 ? at_gate + block : inter + c;
        const float g = to_float(gu[t * 2 * inter + at_gate]);
        const float u = to_float(gu[t * 2 * inter + at_up]);
        const float s = g / (1.0f + expf(-g));
        out[i] = from_float<T>(s * u);
    }
}

// bfloat16, eight columns per thread (16-byte loads and stores); inter a multiple of 8 and, when
// interleaved, block a multiple of 8.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

__global__ void __launch_bounds__(256)
silu_mul_vec_kernel(const bf16* __restrict__ gu, bf16* __restrict__ out, int inter, int block, int64_t groups) {
    const int per_row = inter / 8;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < groups; i += (int64_t)gridDim.x * 256) {
        const int64_t t = i / per_row;
        const int c = (int)(i - t * per_row) * 8;
        const int at_gate = block > 0 ? (c / block) * 2 * block + c % block : c;
        const int at_up = block > 0 ? at_gate + block : inter + c;
        const bf16x8 g = *reinterpret_cast<const bf16x8*>(gu + t * 2 * inter + at_gate);
        const bf16x8 u = *reinterpret_cast<const bf16x8*>(gu + t * 2 * inter + at_up);
        bf16x8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float gj = (float)g[j];
            o[j] = (bf16)(gj / (1.0f + expf(-gj)) * (float)u[j]);
        }
        *reinterpret_cast<bf16x8*>(out + t * inter + c) = o;
    }
}

extern "C" int somi_silu_mul(const void* gate_up, void* out, int dtype, int n_tokens, int inter, int block,
                             hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && inter > 0, "silu_mul: bad sizes n=%d inter=%d", n_tokens, inter);
    SOMI_REQUIRE(block >= 0 && (block == 0 || inter % block == 0), "silu_mul: block %d does not divide %d", block, inter);
    const int64_t count = (int64_t)n_tokens * inter;
    if (count == 0) return 0;
    const int grid = (int)(ceil_div64(count, 256) < 65536 ? ceil_div64(count, 256) : 65536);
    if (dtype == SOMI_BF16 && inter % 8 == 0 && (block == 0 || block % 8 == 0) && (uintptr_t)gate_up % 16 == 0 &&
        (uintptr_t)out % 16 == 0) {
        const int64_t groups = count / 8;
        const int vgrid = (int)(ceil_div64(groups, 256) < 65536 ? ceil_div64(groups, 256) : 65536);
        hipLaunchKernelGGL(silu_mul_vec_kernel, dim3(vgrid), dim3(256), 0, stream, (const bf16*)gate_up, (bf16*)out,
                           inter, block, groups);
        SOMI_LAUNCH_CHECK("silu_mul");
        return 0;
    }
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(silu_mul_kernel<float>, dim3(grid), dim3(256), 0, stream, (const float*)gate_up,
                           (float*)out, inter, block, count);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(silu_mul_kernel<bf16>, dim3(grid), dim3(256), 0, stream, (const bf16*)gate_up,
                           (bf16*)out, inter, block, count);
    else
        return somi_fail("silu_mul: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("silu_mul");
    return 0;
}

// The gated product with a choice of activation: out[t, i] = act(gate[t, i]) * up[t, i]; gu = [gate columns | up
// columns] (block == 0) or gate and up columns interleaved in blocks of `block` columns, as for somi_silu_mul.
// act 0: SiLU; act 1: the tanh form of GELU, 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))).
__device__ __forceinline__ float gelu_tanh(float z) {
    const float inner = 0.7978845608028654f * (z + 0.044715f * z * z * z);
    return 0.5f * z * (1.0f + tanhf(inner));
}

template <typename T>
__global__ void __launch_bounds__(256)
act_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, int act, int block, int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) {
        const int64_t t = i / inter;
        const int c = (int)(i - t * inter);
        const int at_gate = block > 0 ? (c / block) * 2 * block + c % block : c;
        const int at_up = block > 0 ? at_gate + block : inter + c;
        const float g = to_float(gu[t * 2 * inter + at_gate]);
        const float u = to_float(gu[t * 2 * inter + at_up]);
        const float a = act == 1 ? gelu_tanh(g) : g / (1.0f + expf(-g));
        out[i] = from_float<T>(a * u);
    }
}

extern "C" int somi_act_mul(const void* gate_up, void* out, int dtype, int n_tokens, int inter, int act, int block,
                            hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && inter > 0, "act_mul: bad sizes n=%d inter=%d", n_tokens, inter);
    SOMI_REQUIRE(block >= 0 && (block == 0 || inter % block == 0), "act_mul: block %d does not divide %d", block, inter);
    SOMI_REQUIRE(act == 0 || act == 1, "act_mul: unknown activation %d", act);
    const int64_t count = (int64_t)n_tokens * inter;
    if (count == 0) return 0;
    const int grid = (int)(ceil_div64(count, 256) < 65536 ? ceil_div64(count, 256) : 65536);
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(act_mul_kernel<float>, dim3(grid), dim3(256), 0, stream, (const float*)gate_up, (float*)out,
                           inter, act, block, count);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(act_mul_kernel<bf16>, dim3(grid), dim3(256), 0, stream, (const bf16*)gate_up, (bf16*)out,
                           inter, act, block, count);
    else
        return somi_fail("act_mul: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("act_mul");
    return 0;
}

// Soft cap of float32 logits in place: x <- cap * tanh(x / cap).
__global__ void __launch_bounds__(256)
softcap_kernel(float* __restrict__ x, float cap, float inv_cap, int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256)
        x[i] = cap * tanhf(x[i] * inv_cap);
}

extern "C" int somi_softcap(float* x, float cap, int64_t count, hipStream_t stream) {
    SOMI_REQUIRE(count >= 0 && cap > 0.f, "softcap: bad arguments");
    if (count == 0) return 0;
    const int grid = (int)(ceil_div64(count, 256) < 65536 ? ceil_div64(count, 256) : 65536);
    hipLaunchKernelGGL(softcap_kernel, dim3(grid), dim3(256), 0, stream, x, cap, 1.0f / cap, count);
    SOMI_LAUNCH_CHECK("softcap");
    return 0;
}

// A polynomial activation with normed powers: for a row z of float32 sums,
//
//     out = a N(z) + b N(z^2) + c N(z^3) + e,     N(u) = u / sqrt(mean(u^2) + eps) over the row,
//
// powers element by element; coef = (a, b, c, e) on the device.  One workgroup per row; the three mean squares are
// float32, the result is rounded once.
template <typename TO>
__global__ void __launch_bounds__(256)
poly_norm_kernel(const float* __restrict__ z, const float* __restrict__ coef, float eps, TO* __restrict__ out, int width) {
    __shared__ float red[16];
    const float* row = z + (int64_t)blockIdx.x * width;
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int i = threadIdx.x; i < width; i += 256) {
        const float v = row[i], v2 = v * v, v3 = v2 * v;
        s1 = fmaf(v, v, s1);
        s2 = fmaf(v2, v2, s2);
        s3 = fmaf(v3, v3, s3);
    }
    s1 = block_sum<256>(s1, red);
    s2 = block_sum<256>(s2, red);
    s3 = block_sum<256>(s3, red);
    const float n = (float)width;
    const float r1 = coef[0] / sqrtf(s1 / n + eps), r2 = coef[1] / sqrtf(s2 / n + eps), r3 = coef[2] / sqrtf(s3 / n + eps);
    const float shift = coef[3];
    TO* o = out + (int64_t)blockIdx.x * width;
    for (int i = threadIdx.x; i < width; i += 256) {
        const float v = row[i], v2 = v * v;
        o[i] = from_float<TO>(r1 * v + r2 * v2 + r3 * (v2 * v) + shift);
    }
}

extern "C" int somi_poly_norm(const float* z, const float* coef, float eps, void* out, int out_dtype, int n_tokens, int width,
                              hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && width > 0, "poly_norm: bad sizes");
    if (n_tokens == 0) return 0;
    if (out_dtype == SOMI_F32)
        hipLaunchKernelGGL(poly_norm_kernel<float>, dim3(n_tokens), dim3(256), 0, stream, z, coef, eps, (float*)out, width);
    else if (out_dtype == SOMI_BF16)
        hipLaunchKernelGGL(poly_norm_kernel<bf16>, dim3(n_tokens), dim3(256), 0, stream, z, coef, eps, (bf16*)out, width);
    else
        return somi_fail("poly_norm: unknown dtype %d", out_dtype);
    SOMI_LAUNCH_CHECK("poly_norm");
    return 0;
}

// xIELU: a unit with a quadratic positive side and an exponential negative side, two stored numbers (p, q) on the device:
//
//     z > 0:   softplus(p) z^2 + z / 2            z <= 0:   (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2.
//
// z: float32 sums of the product in front (its bias added); float32 arithmetic, rounded once.
__device__ __forceinline__ float somi_softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

template <typename TO>
__global__ void __launch_bounds__(256)
xielu_kernel(const float* __restrict__ z, const float* __restrict__ pq, TO* __restrict__ out, int64_t count) {
    const float ap = somi_softplus(pq[0]), an = 0.5f + somi_softplus(pq[1]);
    auto unit = [&](float v) { return v > 0.f ? fmaf(ap * v, v, 0.5f * v) : fmaf(an, expm1f(v) - v, 0.5f * v); };
    // four values a thread and round (16 bytes in), then what is left one by one
    const int64_t quads = count >> 2;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < quads; i += (int64_t)gridDim.x * 256) {
        const float4 v = reinterpret_cast<const float4*>(z)[i];
        TO r[4] = {from_float<TO>(unit(v.x)), from_float<TO>(unit(v.y)), from_float<TO>(unit(v.z)), from_float<TO>(unit(v.w))};
#pragma unroll
        for (int e = 0; e < 4; ++e) out[i * 4 + e] = r[e];
    }
    for (int64_t i = quads * 4 + (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256)
        out[i] = from_float<TO>(unit(z[i]));
}

extern "C" int somi_xielu(const float* z, const float* pq, void* out, int out_dtype, int64_t count, hipStream_t stream) {
    SOMI_REQUIRE(count >= 0, "xielu: bad sizes");
    SOMI_REQUIRE(((uintptr_t)z & 15) == 0, "xielu: rows must start at a multiple of 16 bytes");
    if (count == 0) return 0;
    const int grid = (int)(ceil_div64(count, 1024) < 65536 ? ceil_div64(count, 1024) : 65536);
    if (out_dtype == SOMI_F32)
        hipLaunchKernelGGL(xielu_kernel<float>, dim3(grid), dim3(256), 0, stream, z, pq, (float*)out, count);
    else if (out_dtype == SOMI_BF16)
        hipLaunchKernelGGL(xielu_kernel<bf16>, dim3(grid), dim3(256), 0, stream, z, pq, (bf16*)out, count);
    else
        return somi_fail("xielu: unknown dtype %d", out_dtype);
    SOMI_LAUNCH_CHECK("xielu");
    return 0;
}

// A sigmoid gate on rows: out = x * sigmoid(g) element by element; g: float32 sums of the gate's product, rows
// g_stride apart; x and out: [n, width] of one type.
template <typename T>
__global__ void __launch_bounds__(256)
sigmoid_gate_kernel(const T* __restrict__ x, const float* __restrict__ g, int64_t g_stride, T* __restrict__ out, int width,
                    int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) {
        const int64_t row = i / width;
        const float gate = g[row * g_stride + (i - row * width)];
        out[i] = from_float<T>(to_float(x[i]) / (1.0f + expf(-gate)));
    }
}

extern "C" int somi_sigmoid_gate(const void* x, int dtype, const float* g, int64_t g_stride, void* out, int64_t n_rows,
                                 int width, hipStream_t stream) {
    SOMI_REQUIRE(n_rows >= 0 && width > 0 && g_stride >= width, "sigmoid_gate: bad sizes");
    const int64_t count = n_rows * width;
    if (count == 0) return 0;
    const int grid = (int)(ceil_div64(count, 256) < 65536 ? ceil_div64(count, 256) : 65536);
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(sigmoid_gate_kernel<float>, dim3(grid), dim3(256), 0, stream, (const float*)x, g, g_stride,
                           (float*)out, width, count);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(sigmoid_gate_kernel<bf16>, dim3(grid), dim3(256), 0, stream, (const bf16*)x, g, g_stride,
                           (bf16*)out, width, count);
    else
        return somi_fail("sigmoid_gate: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("sigmoid_gate");
    return 0;
}
