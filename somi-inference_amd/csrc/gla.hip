// Gated linear attention: a recurrent state per request and head, carried from token to token.
//
//   alpha[t, h, d] = sigmoid(z)^(1/tau),  z = W2 (a[t]) + b           (a: the low-rank projection of the input; z
//                                                                    comes from the engine's matrix products)
//   S_t[d, c]      = alpha[t, h, d] * S_(t-1)[d, c] + k[t, h, d] * v[t, h, c]          S: [dim, vdim] per head
//   o[t, h, c]     = sum_d S_t[d, c] * q[t, h, d] * q_scale
//   y[t, h, c]     = o / sqrt(mean_c(o^2) + eps) * w[c] * silu(g[t, h, c])
//
// The state, the decays (sigmoid, its logarithm through softplus, the exponential), the sums over d and the norm are
// float32 whatever the storage type of q, k, v, g and a.  Every column c of a head's state evolves by itself, so the
// columns are dealt to wavefronts; tokens of one request run in order from the state that earlier steps left in the
// request's slot, so a prompt cut into portions, or decoded token by token, performs the same operations in the
// same order as the whole prompt in one step.
#include "common.h"

// ------------------------------------------------------------------------------------------------ decays
// alpha = sigmoid(z)^(1 / tau) = exp(-softplus(-z) / tau), in place on the float32 sums z of the decay's projection.
__global__ void __launch_bounds__(256)
gla_alpha_kernel(float* __restrict__ z, float inv_tau, int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) {
        const float x = z[i];
        // log sigmoid(x) = -softplus(-x) = -(max(-x, 0) + log1p(exp(-|x|)))
        const float log_sigmoid = -(fmaxf(-x, 0.f) + log1pf(expf(-fabsf(x))));
        z[i] = expf(log_sigmoid * inv_tau);
    }
}

extern "C" int somi_gla_alpha(float* z, float tau, int64_t count, hipStream_t stream) {
    SOMI_REQUIRE(count >= 0 && tau > 0.f, "gla_alpha: bad arguments");
    if (count == 0) return 0;
    const int grid = (int)(ceil_div64(count, 256) < 65536 ? ceil_div64(count, 256) : 65536);
    hipLaunchKernelGGL(gla_alpha_kernel, dim3(grid), dim3(256), 0, stream, z, 1.0f / tau, count);
    SOMI_LAUNCH_CHECK("gla_alpha");
    return 0;
}

// ------------------------------------------------------------------------------------------------ the recurrence
// A wavefront (a workgroup of its own) owns GLA_COLS columns of one (entry, head) (4 with 16 lanes a column, see the
// kernel): lane = 4 * column + row group, and
// row group g of the four holds the rows d = g * RPL .. g * RPL + RPL - 1 of its column in registers (rows past dim are
// padding that stays zero).  The tokens' alpha, k, scaled q and v of the head go through LDS STAGE tokens at a time,
// laid out so that a lane reads its rows four at a time.  The next tokens' values are asked of memory, as they are
// stored (no arithmetic touches them, so nothing waits for them), before the staged ones are worked on; they are
// converted on their way into LDS.  Per token a lane updates its rows and sums its share of o, the row groups' shares
// are added by two exchanges inside the column's four lanes, always in the same order, and the stage's o leaves
// through LDS in whole rows.
#define GLA_COLS 16
#define GLA_GROUPS 4

typedef __attribute__((ext_vector_type(4))) float gla_f32x4;

// The value of another lane of the same group of four lanes (a data-parallel move: no LDS, no wait).
template <int PATTERN> __device__ __forceinline__ float quad_swap(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), PATTERN, 0xF, 0xF, true));
}

// G consecutive elements as they are stored.
template <typename T, int G> struct GlaRaw { T v[G]; };
template <typename T, int G> __device__ __forceinline__ GlaRaw<T, G> gla_load(const T* p) {
    GlaRaw<T, G> out;
    if (G == 4) {
        typedef __attribute__((ext_vector_type(4))) T vec4;
        const vec4 x = *reinterpret_cast<const vec4*>(p);
#pragma unroll
        for (int i = 0; i < 4; ++i) out.v[i] = x[i];
    } else {
        out.v[0] = p[0];
    }
    return out;
}

// G: elements moved at a time, 4 where dim, vdim and the row strides are multiples of 4 and the rows aligned, else 1.
// LPC: lanes that share a column of the state (4, or 16 where 4 would leave the device short of wavefronts: a wavefront
// then owns 4 columns and a lane a sixteenth of the rows; the row groups' shares are added by two more data-parallel
// moves, rotations inside the column's row of 16 lanes).
template <typename T, int RPL, int G, int LPC>
__global__ void __launch_bounds__(64)
gla_scan_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, int64_t row_stride,
                const float* __restrict__ alpha, const int* __restrict__ entry_start,
                const int* __restrict__ state_slots, float* __restrict__ state, int heads, int dim, int vdim,
                float q_scale, float* __restrict__ o) {
    constexpr int STAGE = RPL * LPC <= 64 ? 16 : (RPL * LPC <= 128 ? 8 : 4);   // tokens staged at a time
    constexpr int COLS = 64 / LPC;                                     // columns of a wavefront
    constexpr int ROWS = LPC * RPL;                                    // padded rows of a head
    constexpr int PIECES = STAGE * ROWS / G / 64;                      // pieces of G rows of each array a lane moves
    constexpr int VPIECES = (STAGE * COLS / G + 63) / 64;          // pieces of G columns of v a lane moves
    __shared__ __attribute__((aligned(16))) float sa[STAGE * ROWS];
    __shared__ __attribute__((aligned(16))) float sk[STAGE * ROWS];
    __shared__ __attribute__((aligned(16))) float sq[STAGE * ROWS];
    __shared__ __attribute__((aligned(16))) float sv[STAGE * COLS];
    __shared__ __attribute__((aligned(16))) float so[STAGE * COLS];
    const int e = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int col0 = blockIdx.z * COLS;
    const int colidx = lane / LPC, group = lane % LPC;
    const int col = col0 + colidx;
    const bool live = col < vdim;
    const int t0 = entry_start[e], t1 = entry_start[e + 1];
    float* S = state + (((int64_t)state_slots[e] * heads + h) * dim) * (int64_t)vdim;
    float s[RPL];
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
        const int d = group * RPL + i;
        s[i] = (live && d < dim) ? S[(int64_t)d * vdim + col] : 0.f;
    }
    GlaRaw<float, G> ra[PIECES];
    GlaRaw<T, G> rk[PIECES], rq[PIECES], rv[VPIECES];

    // piece p of a stage's rows: token p / (ROWS / G) of the stage, rows G * (p % (ROWS / G)) ..; where that lies past
    // the entry's tokens or the head's rows, a piece that exists is read instead and is not used
    auto fetch = [&](int base) {
#pragma unroll
        for (int j = 0; j < PIECES; ++j) {
            const int piece = lane + 64 * j;
            const int t = min(base + piece / (ROWS / G), t1 - 1), d = min(G * (piece % (ROWS / G)), dim - G);
            const int64_t at = (int64_t)t * row_stride + (int64_t)h * dim + d;
            ra[j] = gla_load<float, G>(alpha + ((int64_t)t * heads + h) * dim + d);
            rk[j] = gla_load<T, G>(k + at);
            rq[j] = gla_load<T, G>(q + at);
        }
#pragma unroll
        for (int j = 0; j < VPIECES; ++j) {
            const int piece = lane + 64 * j;
            const int t = min(base + piece / (COLS / G), t1 - 1);
            const int c = min(col0 + G * (piece % (COLS / G)), vdim - G);
            rv[j] = gla_load<T, G>(v + (int64_t)t * row_stride + (int64_t)h * vdim + c);
        }
    };

    if (t0 < t1) fetch(t0);
    for (int base = t0; base < t1; base += STAGE) {
        const int count = min(STAGE, t1 - base);
        // into LDS, converted: a row past dim keeps its zero; a token past the entry's last leaves the state as it is
        // (alpha 1, k 0)
#pragma unroll
        for (int j = 0; j < PIECES; ++j) {
            const int piece = lane + 64 * j;
            const int tt = piece / (ROWS / G), d = G * (piece % (ROWS / G));
            const bool token_there = base + tt < t1;
#pragma unroll
            for (int x = 0; x < G; ++x) {
                const bool row_there = d + x < dim;          // with G == 4 a piece is there whole or not at all
                const bool there = token_there && row_there;
                sa[piece * G + x] = there ? ra[j].v[x] : (row_there ? 1.f : 0.f);
                sk[piece * G + x] = there ? to_float(rk[j].v[x]) : 0.f;
                sq[piece * G + x] = there ? to_float(rq[j].v[x]) * q_scale : 0.f;
            }
        }
#pragma unroll
        for (int j = 0; j < VPIECES; ++j) {
            const int piece = lane + 64 * j;
            if (piece < STAGE * COLS / G) {
                const int tt = piece / (COLS / G), c = G * (piece % (COLS / G));
#pragma unroll
                for (int x = 0; x < G; ++x)
                    sv[piece * G + x] = (base + tt < t1 && col0 + c + x < vdim) ? to_float(rv[j].v[x]) : 0.f;
            }
        }
        __syncthreads();                           // one wavefront a workgroup: its stores to LDS before its reads
        if (base + STAGE < t1) fetch(base + STAGE);
        // every staged token is worked on, also those past the entry's last (they change nothing and store nothing), so
        // that the tokens' instructions can be woven into each other
#pragma unroll
        for (int tt = 0; tt < STAGE; ++tt) {
            const float* a = sa + tt * ROWS + group * RPL;
            const float* kk = sk + tt * ROWS + group * RPL;
            const float* qq = sq + tt * ROWS + group * RPL;
            const float vt = sv[tt * COLS + colidx];
            float part[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < RPL; i += 4) {
                const gla_f32x4 a4 = *reinterpret_cast<const gla_f32x4*>(a + i);
                const gla_f32x4 k4 = *reinterpret_cast<const gla_f32x4*>(kk + i);
                const gla_f32x4 q4 = *reinterpret_cast<const gla_f32x4*>(qq + i);
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    s[i + x] = fmaf(a4[x], s[i + x], k4[x] * vt);
                    part[x] = fmaf(s[i + x], q4[x], part[x]);
                }
            }
            float acc = (part[0] + part[1]) + (part[2] + part[3]);
            acc += quad_swap<0xB1>(acc);           // the neighbour in the quad, then the other pair: the four row groups
            acc += quad_swap<0x4E>(acc);
            if (LPC == 16) {
                acc += quad_swap<0x124>(acc);      // the quad four lanes on in the column's row of 16, then the pair of quads
                acc += quad_swap<0x128>(acc);
            }
            if (group == 0) so[tt * COLS + colidx] = acc;
        }
        __syncthreads();                           // the reads, before the next tokens are staged; so is whole
        // the stage's o in pieces of 4 columns: token lane / (COLS / 4), columns 4 * (lane % (COLS / 4)) .. + 3
        if (lane < STAGE * (COLS / 4)) {
            const int tt = lane / (COLS / 4), c = 4 * (lane % (COLS / 4));
            if (tt < count) {
                float* row = o + ((int64_t)(base + tt) * heads + h) * vdim + col0 + c;
                if (G == 4) {
                    if (col0 + c < vdim) *reinterpret_cast<gla_f32x4*>(row) = *reinterpret_cast<const gla_f32x4*>(so + tt * COLS + c);
                } else {
#pragma unroll
                    for (int x = 0; x < 4; ++x)
                        if (col0 + c + x < vdim) row[x] = so[tt * COLS + c + x];
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
        const int d = group * RPL + i;
        if (live && d < dim) S[(int64_t)d * vdim + col] = s[i];
    }
}

// q, k: [n_tokens, row_stride] with head h at columns h * dim ..; v: the same with head h at h * vdim ..
// alpha: [n_tokens, heads, dim] float32.  entry_start: [n_entries + 1] offsets of the entries' tokens;
// state_slots: [n_entries]; state: [slots, heads, dim, vdim] float32, read and written in place.
// o: [n_tokens, heads, vdim] float32.
extern "C" int somi_gla_scan(const void* q, const void* k, const void* v, int dtype, int64_t row_stride,
                             const float* alpha, const int* entry_start, const int* state_slots, float* state,
                             int n_entries, int heads, int dim, int vdim, float q_scale, int lanes, float* o,
                             hipStream_t stream) {
    SOMI_REQUIRE(n_entries >= 0 && heads > 0 && dim > 0 && vdim > 0, "gla_scan: bad sizes");
    SOMI_REQUIRE(dim <= 64 * GLA_GROUPS, "gla_scan: a key size of %d is more than the supported %d", dim, 64 * GLA_GROUPS);
    SOMI_REQUIRE(row_stride >= (int64_t)heads * dim && row_stride >= (int64_t)heads * vdim, "gla_scan: rows too narrow");
    SOMI_REQUIRE(heads <= 65535 && ceil_div(vdim, GLA_COLS) <= 65535, "gla_scan: too many heads or columns");
    if (n_entries == 0) return 0;
    // lanes a column: from the model's sizes and the device only, never from the step, so that a request's sums have one
    // order in every batch; 16 where 4 would leave fewer than two wavefronts a compute unit for one request (and the
    // rows are enough for 16 lanes)
    SOMI_REQUIRE(lanes == 0 || lanes == 4 || lanes == 16, "gla_scan: %d lanes a column; 4 or 16", lanes);
    const int lpc = lanes ? lanes : (heads * ceil_div(vdim, GLA_COLS) < 2 * somi_units() && dim >= 64 ? 16 : 4);
    const dim3 grid(n_entries, heads, ceil_div(vdim, 64 / lpc));
    const int rpl = lpc == 16 ? ceil_div(dim, 16) : ceil_div(dim, GLA_GROUPS);
    // four elements at a time where every piece of four is whole and aligned
    const bool wide = dim % 4 == 0 && vdim % 4 == 0 && row_stride % 4 == 0 && (uintptr_t)q % 16 == 0 && (uintptr_t)k % 8 == 0 &&
                      (uintptr_t)v % 8 == 0 && (uintptr_t)alpha % 16 == 0 && (uintptr_t)o % 16 == 0 &&
                      (dtype == SOMI_BF16 || ((uintptr_t)k % 16 == 0 && (uintptr_t)v % 16 == 0));
#define GLA_LAUNCH(T, R, L)                                                                                           \
    do {                                                                                                              \
        if (wide)                                                                                                     \
            hipLaunchKernelGGL((gla_scan_kernel<T, R, 4, L>), grid, dim3(64), 0, stream, (const T*)q, (const T*)k,    \
                               (const T*)v, row_stride, alpha, entry_start, state_slots, state, heads, dim, vdim,     \
                               q_scale, o);                                                                           \
        else                                                                                                          \
            hipLaunchKernelGGL((gla_scan_kernel<T, R, 1, L>), grid, dim3(64), 0, stream, (const T*)q, (const T*)k,    \
                               (const T*)v, row_stride, alpha, entry_start, state_slots, state, heads, dim, vdim,     \
                               q_scale, o);                                                                           \
    } while (0)
#define GLA_BY_ROWS(T)                                                                                                \
    do {                                                                                                              \
        if (lpc == 16) {                                                                                              \
            if (rpl <= 4) GLA_LAUNCH(T, 4, 16);                                                                       \
            else if (rpl <= 8) GLA_LAUNCH(T, 8, 16);                                                                  \
            else if (rpl <= 12) GLA_LAUNCH(T, 12, 16);                                                                \
            else GLA_LAUNCH(T, 16, 16);                                                                               \
        } else if (rpl <= 4) GLA_LAUNCH(T, 4, 4);                                                                     \
        else if (rpl <= 8) GLA_LAUNCH(T, 8, 4);                                                                       \
        else if (rpl <= 12) GLA_LAUNCH(T, 12, 4);                                                                     \
        else if (rpl <= 16) GLA_LAUNCH(T, 16, 4);                                                                     \
        else if (rpl <= 24) GLA_LAUNCH(T, 24, 4);                                                                     \
        else if (rpl <= 32) GLA_LAUNCH(T, 32, 4);                                                                     \
        else if (rpl <= 48) GLA_LAUNCH(T, 48, 4);                                                                     \
        else GLA_LAUNCH(T, 64, 4);                                                                                    \
    } while (0)
    if (dtype == SOMI_F32) GLA_BY_ROWS(float);
    else if (dtype == SOMI_BF16) GLA_BY_ROWS(bf16);
    else return somi_fail("gla_scan: unknown dtype %d", dtype);
#undef GLA_BY_ROWS
#undef GLA_LAUNCH
    SOMI_LAUNCH_CHECK("gla_scan");
    return 0;
}

// ------------------------------------------------------------------------------------------------ norm and gate
// y[t, h, c] = o / sqrt(mean_c(o^2) + eps) * w[c] * silu(g[t, h, c]); without a gate (GATE false) the last factor is
// left out.  One wavefront per (token, head).
template <typename T, bool GATE>
__global__ void __launch_bounds__(64)
gla_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w, const T* __restrict__ g,
                     int64_t g_stride, float eps, T* __restrict__ y, int heads, int vdim) {
    const int64_t t = blockIdx.x;
    const int h = blockIdx.y, lane = threadIdx.x;
    const float* orow = o + (t * heads + h) * vdim;
    float ss = 0.f;
    for (int c = lane; c < vdim; c += 64) ss = fmaf(orow[c], orow[c], ss);
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)vdim + eps);
    T* yrow = y + (t * heads + h) * vdim;
    if (!GATE) {
        for (int c = lane; c < vdim; c += 64) yrow[c] = from_float<T>(orow[c] * inv * w[c]);
        return;
    }
    const T* grow = g + t * g_stride + (int64_t)h * vdim;
    for (int c = lane; c < vdim; c += 64) {
        const float gate = to_float(grow[c]);
        const float silu = gate / (1.0f + expf(-gate));
        yrow[c] = from_float<T>(orow[c] * inv * w[c] * silu);
    }
}

// o: [n_tokens, heads, vdim] float32; w: [vdim] float32; g: [n_tokens, g_stride] with head h at h * vdim .., or null
// for a mixer without a gate; y: [n_tokens, heads * vdim] in the storage type.
extern "C" int somi_gla_norm_gate(const float* o, const float* w, const void* g, int dtype, int64_t g_stride, float eps,
                                  void* y, int n_tokens, int heads, int vdim, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && heads > 0 && vdim > 0 && (g == nullptr || g_stride >= (int64_t)heads * vdim),
                 "gla_norm_gate: bad sizes");
    SOMI_REQUIRE(heads <= 65535, "gla_norm_gate: too many heads");
    if (n_tokens == 0) return 0;
    const dim3 grid(n_tokens, heads);
#define GLA_NORM(T, GATE)                                                                                            \
    hipLaunchKernelGGL((gla_norm_gate_kernel<T, GATE>), grid, dim3(64), 0, stream, o, w, (const T*)g, g_stride, eps, \
                       (T*)y, heads, vdim)
    if (dtype == SOMI_F32) {
        if (g) GLA_NORM(float, true); else GLA_NORM(float, false);
    } else if (dtype == SOMI_BF16) {
        if (g) GLA_NORM(bf16, true); else GLA_NORM(bf16, false);
    } else {
        return somi_fail("gla_norm_gate: unknown dtype %d", dtype);
    }
#undef GLA_NORM
    SOMI_LAUNCH_CHECK("gla_norm_gate");
    return 0;
}

// ------------------------------------------------------------------------------------------------ bounded forget gates
// For a recurrence whose forget gate also decides what is written (S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, o_t =
// S_t^T q_t): from rows [q as projected | z, the gate's projection | ...] of float32 sums, in place,
//
//     q <- silu(q);     f = lower + (1 - lower) sigmoid(z + bias);     z <- 1 - f = (1 - lower) sigmoid(-(z + bias))
//
// and f itself into `decay`, so that the recurrence above reads q, k = 1 - f and alpha = f.  lower, bias: [width], the
// heads' channels in one row.
__global__ void __launch_bounds__(256)
bounded_forget_kernel(float* __restrict__ rows, int64_t row_stride, const float* __restrict__ bias,
                      const float* __restrict__ lower, float* __restrict__ decay, int width, int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) {
        const int64_t t = i / width;
        const int c = (int)(i - t * width);
        float* row = rows + t * row_stride;
        const float q = row[c];
        row[c] = q / (1.0f + expf(-q));
        const float z = row[width + c] + bias[c];
        const float lo = lower[c];
        const float keep = 1.0f / (1.0f + expf(-z)), write = 1.0f / (1.0f + expf(z));
        decay[i] = lo + (1.0f - lo) * keep;
        row[width + c] = (1.0f - lo) * write;
    }
}

extern "C" int somi_bounded_forget(float* rows, int64_t row_stride, const float* bias, const float* lower, float* decay,
                                   int n_tokens, int width, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && width > 0 && row_stride >= 2 * (int64_t)width, "bounded_forget: bad sizes");
    const int64_t count = (int64_t)n_tokens * width;
    if (count == 0) return 0;
    const int grid = (int)(ceil_div64(count, 256) < 65536 ? ceil_div64(count, 256) : 65536);
    hipLaunchKernelGGL(bounded_forget_kernel, dim3(grid), dim3(256), 0, stream, rows, row_stride, bias, lower, decay, width,
                       count);
    SOMI_LAUNCH_CHECK("bounded_forget");
    return 0;
}
