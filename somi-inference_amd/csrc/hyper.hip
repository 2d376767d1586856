// Several residual streams side by side (hyper-connections), float32 throughout.
//
// A layer's sublayer reads one weighted sum of the S streams and writes back into all of them:
//
//     u = sum_s a[s] x_s,        y = sublayer(norm(u)),        x_t <- sum_s M[s, t] x_s + b[t] y     (all t at once).
//
// One kernel does what lies between two sublayers for a row: the write of the sublayer that just ran (M, b, y), then
// the read of the next one (a) with its RMS norm, u / sqrt(mean(u^2) + eps) * w.  Each half may be left out: without
// y nothing is written; without a the streams are summed with weight 1; without w the sum is written as it is.  The
// result may be written several times over (`copies`: a first row fanned out into S equal streams).
//
// lanes: [S, n, width] float32, updated in place.  One workgroup a row; a thread owns the columns tid, tid + 256, ...
// of all S streams, so the update of a column needs nobody else's values.
#include "common.h"

#define HC_MAX_STREAMS 8
#define HC_NT 256

// VEC: columns a thread takes at a time (4 where the width is a multiple of 4: 16-byte accesses of the streams).
template <typename TY, typename TO, int VEC>
__global__ void __launch_bounds__(HC_NT)
hc_step_kernel(float* __restrict__ lanes, int S, int64_t n, int width, const float* __restrict__ mix,
               const float* __restrict__ out_w, const TY* __restrict__ y, const float* __restrict__ in_w, int read,
               const float* __restrict__ norm_w, float eps, TO* __restrict__ out, int copies) {
    __shared__ float red[16];
    __shared__ float coef[HC_MAX_STREAMS * HC_MAX_STREAMS + 2 * HC_MAX_STREAMS];
    float* m_s = coef;                                        // [S, S] from, to
    float* b_s = coef + HC_MAX_STREAMS * HC_MAX_STREAMS;      // [S]
    float* a_s = b_s + HC_MAX_STREAMS;                        // [S]
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    if (tid < S * S && y != nullptr) m_s[tid] = mix[tid];
    if (tid < S) {
        b_s[tid] = y != nullptr ? out_w[tid] : 0.f;
        a_s[tid] = in_w != nullptr ? in_w[tid] : 1.f;
    }
    __syncthreads();
    const int64_t plane = n * (int64_t)width;
    float* base = lanes + row * width;
    float ss = 0.f;
    for (int c = tid * VEC; c < width; c += HC_NT * VEC) {
        float x[HC_MAX_STREAMS][VEC];
#pragma unroll
        for (int s = 0; s < HC_MAX_STREAMS; ++s)
            if (s < S) {
                if (VEC == 4) {
                    const float4 v = *reinterpret_cast<const float4*>(base + s * plane + c);
                    x[s][0] = v.x; x[s][1] = v.y; x[s][2 % VEC] = v.z; x[s][3 % VEC] = v.w;
                } else {
                    x[s][0] = base[s * plane + c];
                }
            }
        if (y != nullptr) {
            float yv[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) yv[e] = to_float(y[row * width + c + e]);
            float fresh[HC_MAX_STREAMS][VEC];
#pragma unroll
            for (int t = 0; t < HC_MAX_STREAMS; ++t)
                if (t < S) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        float v = 0.f;
#pragma unroll
                        for (int s = 0; s < HC_MAX_STREAMS; ++s)
                            if (s < S) v = fmaf(m_s[s * S + t], x[s][e], v);
                        fresh[t][e] = fmaf(b_s[t], yv[e], v);
                    }
                }
#pragma unroll
            for (int t = 0; t < HC_MAX_STREAMS; ++t)
                if (t < S) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) x[t][e] = fresh[t][e];
                    if (VEC == 4)
                        *reinterpret_cast<float4*>(base + t * plane + c) = make_float4(fresh[t][0], fresh[t][1 % VEC], fresh[t][2 % VEC], fresh[t][3 % VEC]);
                    else
                        base[t * plane + c] = fresh[t][0];
                }
        }
        if (read) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float u = 0.f;
#pragma unroll
                for (int s = 0; s < HC_MAX_STREAMS; ++s)
                    if (s < S) u = fmaf(a_s[s], x[s][e], u);
                ss = fmaf(u, u, ss);
                if (norm_w == nullptr)
                    for (int k = 0; k < copies; ++k) out[k * plane + row * width + c + e] = from_float<TO>(u);
            }
        }
    }
    if (!read || norm_w == nullptr) return;
    ss = block_sum<HC_NT>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)width + eps);
    // the sums once more, from the values this thread itself has just written (or only read)
    for (int c = tid * VEC; c < width; c += HC_NT * VEC) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float u = 0.f;
#pragma unroll
            for (int s = 0; s < HC_MAX_STREAMS; ++s)
                if (s < S) u = fmaf(a_s[s], base[s * plane + c + e], u);
            const TO v = from_float<TO>(u * inv * norm_w[c + e]);
            for (int k = 0; k < copies; ++k) out[k * plane + row * width + c + e] = v;
        }
    }
}

template <typename TY, typename TO>
static void hc_launch(float* lanes, int S, int64_t n, int width, const float* mix, const float* out_w, const void* y,
                      const float* in_w, int read, const float* norm_w, float eps, void* out, int copies,
                      hipStream_t stream) {
    if (width % 4 == 0 && ((uintptr_t)lanes & 15) == 0)
        hipLaunchKernelGGL((hc_step_kernel<TY, TO, 4>), dim3((unsigned)n), dim3(HC_NT), 0, stream, lanes, S, n, width, mix,
                           out_w, (const TY*)y, in_w, read, norm_w, eps, (TO*)out, copies);
    else
        hipLaunchKernelGGL((hc_step_kernel<TY, TO, 1>), dim3((unsigned)n), dim3(HC_NT), 0, stream, lanes, S, n, width, mix,
                           out_w, (const TY*)y, in_w, read, norm_w, eps, (TO*)out, copies);
}

// y: [n, width] of y_dtype or null (then mix and out_w are not read).  read != 0: out gets the (normed) sum, in
// out_dtype, `copies` times ([copies, n, width]); `out` must not overlap `lanes` unless S == 1, copies == 1 and the
// row is only read (a norm in place).
extern "C" int somi_hc_step(float* lanes, int S, int64_t n, int width, const float* mix, const float* out_w, const void* y,
                            int y_dtype, const float* in_w, int read, const float* norm_w, float eps, void* out,
                            int out_dtype, int copies, hipStream_t stream) {
    SOMI_REQUIRE(S >= 1 && S <= HC_MAX_STREAMS, "hc_step: %d streams, at most %d are supported", S, HC_MAX_STREAMS);
    SOMI_REQUIRE(n >= 0 && n <= 0x7fffffffLL && width > 0, "hc_step: bad sizes");
    SOMI_REQUIRE(y == nullptr || (mix != nullptr && out_w != nullptr), "hc_step: a write needs its matrix and weights");
    SOMI_REQUIRE(!read || (out != nullptr && copies >= 1), "hc_step: a read needs somewhere to go");
    SOMI_REQUIRE(y != nullptr || read, "hc_step: nothing to do");
    if (n == 0) return 0;
    const bool yb = y != nullptr && y_dtype == SOMI_BF16;
    SOMI_REQUIRE(y == nullptr || yb || y_dtype == SOMI_F32, "hc_step: unknown dtype %d", y_dtype);
    if (out_dtype == SOMI_F32) {
        if (yb) hc_launch<bf16, float>(lanes, S, n, width, mix, out_w, y, in_w, read, norm_w, eps, out, copies, stream);
        else hc_launch<float, float>(lanes, S, n, width, mix, out_w, y, in_w, read, norm_w, eps, out, copies, stream);
    } else if (out_dtype == SOMI_BF16) {
        if (yb) hc_launch<bf16, bf16>(lanes, S, n, width, mix, out_w, y, in_w, read, norm_w, eps, out, copies, stream);
        else hc_launch<float, bf16>(lanes, S, n, width, mix, out_w, y, in_w, read, norm_w, eps, out, copies, stream);
    } else {
        return somi_fail("hc_step: unknown dtype %d", out_dtype);
    }
    SOMI_LAUNCH_CHECK("hc_step");
    return 0;
}
