// Mixture of experts: the router, the grouping of (token, expert) pairs by expert, the experts' products over the
// grouped rows and the weighted sum.
//
//   route      z = W_r h (float32), s = softmax(z) or, element by element, sigmoid(z); experts come in `groups` equal
//              runs of neighbours, a run scores as its best expert and only the `keep` best runs stay; of their experts
//              the `top` with the largest s are chosen, weighted by s over the chosen scores' sum (+ 1e-20) or by s as
//              it is.  Ties go to the lower index.
//   align      the N * top pairs sorted by expert: order[], the experts' offsets and a list of row tiles
//              (expert, first sorted row, rows) that the products' grids walk.
//   gate_up    act[p, :] = glu(W_gate[e] h_t, W_up[e] h_t) for the sorted pair p = (t, e); where the pair's weight is to
//              multiply the expert's input, glu(w_pair W_gate[e] h_t, w_pair W_up[e] h_t): the float32 sums are scaled
//   down       y[pair, :] = w_pair * (W_down[e] act[p, :]) (or without the weight), float32, at the pair's own place
//              t * top + j
//   combine    out[t, :] = sum_j y[t * top + j, :] (+ shared[t, :]), float32, in the order of j
//
// glu(g, u) = g' sigmoid(alpha g') (u' + shift) with g' = min(g, limit) and u' = clamp(u, -limit, limit).
// A row's sums run over K in one fixed order whatever else is in the batch.
#include "common.h"

#define MOE_MAX_EXPERTS 256
#define MOE_MAX_TOP 32
#define MOE_TILE_ROWS 16

__device__ __forceinline__ float clamped_glu(float g, float u, float limit, float alpha, float shift) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.0f + expf(-alpha * g)) * (u + shift);
}

// The router's logits for widths that are a multiple of 4: a workgroup owns ROUTE_TOKENS tokens and ROUTE_EXPERTS
// experts (2 a wavefront: few, so that a step of a few tokens still spreads over several workgroups); the tokens' x
// goes through LDS ROUTE_CHUNK channels at a time, a lane multiplies 4 channels of every 256 of a chunk (its loads of a
// chunk are all asked for before any is used), and a (token, expert) sum is the lanes' partial sums added by
// `wave_sum`: one order whatever else runs.
#define ROUTE_TOKENS 8
#define ROUTE_EXPERTS 8
#define ROUTE_CHUNK 1024
typedef __attribute__((ext_vector_type(4))) float route_f32x4;

template <typename T> struct RouteVec;
template <> struct RouteVec<float> { typedef __attribute__((ext_vector_type(4))) float type; static constexpr int N = 4; };
template <> struct RouteVec<bf16> { typedef __attribute__((ext_vector_type(8))) __bf16 type; static constexpr int N = 8; };

// WIDE: the rows of x are read 16 bytes at a time (rows aligned to 16 bytes, a width that is a multiple of the piece).
template <typename T, bool WIDE>
__global__ void __launch_bounds__(256)
moe_router_logits_kernel(const T* __restrict__ x, int64_t row_stride, const float* __restrict__ router, int n_tokens,
                         int width, int experts, float* __restrict__ logits /*[N, experts]*/) {
    __shared__ __attribute__((aligned(16))) float xs[ROUTE_TOKENS][ROUTE_CHUNK];
    constexpr int EPW = ROUTE_EXPERTS / 4, PIECES = ROUTE_CHUNK / 256;
    const int t0 = blockIdx.x * ROUTE_TOKENS;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int e0 = blockIdx.y * ROUTE_EXPERTS + wave * EPW;
    float acc[EPW][ROUTE_TOKENS];
#pragma unroll
    for (int ei = 0; ei < EPW; ++ei)
#pragma unroll
        for (int tt = 0; tt < ROUTE_TOKENS; ++tt) acc[ei][tt] = 0.f;
    for (int k0 = 0; k0 < width; k0 += ROUTE_CHUNK) {
        __syncthreads();
        if (WIDE) {
            constexpr int VN = RouteVec<T>::N, LOADS = ROUTE_TOKENS * ROUTE_CHUNK / VN / 256;
            typename RouteVec<T>::type piece[LOADS];
#pragma unroll
            for (int j = 0; j < LOADS; ++j) {
                const int i = (threadIdx.x + 256 * j) * VN, tt = i / ROUTE_CHUNK, k = k0 + (i % ROUTE_CHUNK);
                const bool in = t0 + tt < n_tokens && k < width;
                piece[j] = *reinterpret_cast<const typename RouteVec<T>::type*>(x + (int64_t)(in ? t0 + tt : 0) * row_stride + (in ? k : 0));
            }
#pragma unroll
            for (int j = 0; j < LOADS; ++j) {
                const int i = (threadIdx.x + 256 * j) * VN, tt = i / ROUTE_CHUNK, k = k0 + (i % ROUTE_CHUNK);
                const bool in = t0 + tt < n_tokens && k < width;
#pragma unroll
                for (int v = 0; v < VN; ++v) xs[tt][(i % ROUTE_CHUNK) + v] = in ? (float)piece[j][v] : 0.f;
            }
        } else {
            for (int i = threadIdx.x; i < ROUTE_TOKENS * ROUTE_CHUNK; i += 256) {
                const int tt = i / ROUTE_CHUNK, k = k0 + (i % ROUTE_CHUNK);
                xs[tt][i % ROUTE_CHUNK] = (t0 + tt < n_tokens && k < width) ? to_float(x[(int64_t)(t0 + tt) * row_stride + k]) : 0.f;
            }
        }
        route_f32x4 w[EPW][PIECES];
#pragma unroll
        for (int ei = 0; ei < EPW; ++ei)
#pragma unroll
            for (int j = 0; j < PIECES; ++j) {
                const int k = k0 + j * 256 + lane * 4;
                w[ei][j] = route_f32x4{0.f, 0.f, 0.f, 0.f};
                if (e0 + ei < experts && k < width) w[ei][j] = *reinterpret_cast<const route_f32x4*>(router + (int64_t)(e0 + ei) * width + k);
            }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < PIECES; ++j)
#pragma unroll
            for (int tt = 0; tt < ROUTE_TOKENS; ++tt) {
                const route_f32x4 xv = *reinterpret_cast<const route_f32x4*>(&xs[tt][j * 256 + lane * 4]);
#pragma unroll
                for (int ei = 0; ei < EPW; ++ei)
                    acc[ei][tt] += w[ei][j][0] * xv[0] + w[ei][j][1] * xv[1] + w[ei][j][2] * xv[2] + w[ei][j][3] * xv[3];
            }
    }
#pragma unroll
    for (int ei = 0; ei < EPW; ++ei)
#pragma unroll
        for (int tt = 0; tt < ROUTE_TOKENS; ++tt) {
            const float total = wave_sum(acc[ei][tt]);
            if (lane == 0 && e0 + ei < experts && t0 + tt < n_tokens) logits[(int64_t)(t0 + tt) * experts + e0 + ei] = total;
        }
}

// The choice, one wavefront per token: the logits (given, or computed here for widths that are no multiple of 4), the
// softmax, the best runs, the best experts of those.  A lane owns the experts lane, lane + 64, ...; the best of all
// lanes' candidates is found by exchanging (score, index) pairs, ties to the lower index.
__device__ __forceinline__ void wave_best(float& value, int& index) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float other = __shfl_xor(value, off, 64);
        const int other_index = __shfl_xor(index, off, 64);
        if (other > value || (other == value && other_index < index)) {
            value = other;
            index = other_index;
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(64)
moe_route_kernel(const T* __restrict__ x, int64_t row_stride, const float* __restrict__ router,
                 const float* __restrict__ logits, int width, int experts,
                 int top, int groups, int keep, int sigmoid_scores, int normalize, int* __restrict__ chosen,
                 float* __restrict__ weight) {
    constexpr int PER_LANE = MOE_MAX_EXPERTS / 64;
    __shared__ float score[MOE_MAX_EXPERTS];
    __shared__ int taken[MOE_MAX_EXPERTS];          // per run: kept or not
    __shared__ float pick_score[MOE_MAX_TOP];
    __shared__ int pick_index[MOE_MAX_TOP];
    const int64_t t = blockIdx.x;
    const int lane = threadIdx.x;
    if (logits != nullptr) {
        for (int e = lane; e < experts; e += 64) score[e] = logits[t * experts + e];
    } else {
        const T* row = x + t * row_stride;
        for (int e = 0; e < experts; ++e) {
            const float* w = router + (int64_t)e * width;
            float acc = 0.f;
            for (int i = lane; i < width; i += 64) acc += to_float(row[i]) * w[i];
            acc = wave_sum(acc);
            if (lane == 0) score[e] = acc;
        }
    }
    __syncthreads();
    float s[PER_LANE];
    float top_z = -INFINITY;
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
        const int e = lane + 64 * j;
        s[j] = e < experts ? score[e] : -INFINITY;
        top_z = fmaxf(top_z, s[j]);
    }
    top_z = wave_max(top_z);
    float total = 0.f;
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
        if (sigmoid_scores) s[j] = lane + 64 * j < experts ? 1.0f / (1.0f + expf(-s[j])) : 0.f;
        else s[j] = lane + 64 * j < experts ? expf(s[j] - top_z) : 0.f;
        total += s[j];
    }
    total = sigmoid_scores ? 1.0f : wave_sum(total);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
        s[j] /= total;
        if (lane + 64 * j < experts) score[lane + 64 * j] = s[j];
    }
    for (int g = lane; g < groups; g += 64) taken[g] = keep >= groups ? 1 : 0;
    __syncthreads();
    const int per = experts / groups;
    if (keep < groups) {
        // a lane owns the runs lane, lane + 64, ...: their scores, then `keep` rounds of the best run not yet kept
        float run[PER_LANE];
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j) {
            const int g = lane + 64 * j;
            run[j] = -1.f;
            if (g < groups) {
                run[j] = score[g * per];
                for (int i = 1; i < per; ++i) run[j] = fmaxf(run[j], score[g * per + i]);
            }
        }
        for (int round = 0; round < keep; ++round) {
            float best = -1.f;
            int best_run = 1 << 30;
#pragma unroll
            for (int j = 0; j < PER_LANE; ++j)
                if (run[j] > best) {
                    best = run[j];
                    best_run = lane + 64 * j;
                }
            wave_best(best, best_run);
            if (best_run >= groups) break;                 // nothing left that compares (scores that are not numbers)
#pragma unroll
            for (int j = 0; j < PER_LANE; ++j)
                if (lane + 64 * j == best_run) {
                    run[j] = -1.f;
                    taken[best_run] = 1;
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
        const int e = lane + 64 * j;
        if (e >= experts || !taken[e / per]) s[j] = -1.f;  // out of the choice
    }
    float sum = 0.f;
    for (int pick = 0; pick < top; ++pick) {
        float best = -1.f;
        int best_expert = 1 << 30;
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j)
            if (s[j] > best) {
                best = s[j];
                best_expert = lane + 64 * j;
            }
        wave_best(best, best_expert);
        if (best_expert >= experts) {                      // scores that compare with nothing: any expert, weight as it comes
            best_expert = 0;
            best = score[0];
        }
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j)
            if (lane + 64 * j == best_expert) s[j] = -1.f;
        if (lane == 0) {
            pick_score[pick] = best;
            pick_index[pick] = best_expert;
        }
        sum += best;
    }
    __syncthreads();
    for (int pick = lane; pick < top; pick += 64) {
        chosen[t * top + pick] = pick_index[pick];
        weight[t * top + pick] = normalize ? pick_score[pick] / (sum + 1e-20f) : pick_score[pick];
    }
}

extern "C" int somi_moe_route(const void* x, int dtype, int64_t row_stride, const float* router, float* logits,
                              int n_tokens, int width, int experts, int top, int groups, int keep, int sigmoid_scores,
                              int normalize, int* chosen, float* weight, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && width > 0 && experts > 0 && experts <= MOE_MAX_EXPERTS, "moe_route: %d experts, 1 to %d are supported",
                 experts, MOE_MAX_EXPERTS);
    SOMI_REQUIRE(groups >= 1 && experts % groups == 0 && keep >= 1 && keep <= groups, "moe_route: %d groups (keep %d) do not divide %d experts",
                 groups, keep, experts);
    SOMI_REQUIRE(top >= 1 && top <= MOE_MAX_TOP && top <= keep * (experts / groups), "moe_route: top %d does not fit the kept experts", top);
    if (n_tokens == 0) return 0;
    SOMI_REQUIRE(dtype == SOMI_F32 || dtype == SOMI_BF16, "moe_route: unknown dtype %d", dtype);
    // logits: a workspace [n_tokens, experts]; used where the tiled kernel applies (a width that is a multiple of 4)
    const bool tiled = logits != nullptr && width % 4 == 0 && (uintptr_t)router % 16 == 0;
    if (tiled) {
        const dim3 grid(ceil_div(n_tokens, ROUTE_TOKENS), ceil_div(experts, ROUTE_EXPERTS));
        const int piece = dtype == SOMI_F32 ? 4 : 8;
        const bool wide = width % piece == 0 && row_stride % piece == 0 && (uintptr_t)x % 16 == 0;
#define SOMI_ROUTE(T, W)                                                                                                  \
    hipLaunchKernelGGL((moe_router_logits_kernel<T, W>), grid, dim3(256), 0, stream, (const T*)x, row_stride, router, n_tokens, \
                       width, experts, logits)
        if (dtype == SOMI_F32) {
            if (wide) SOMI_ROUTE(float, true); else SOMI_ROUTE(float, false);
        } else {
            if (wide) SOMI_ROUTE(bf16, true); else SOMI_ROUTE(bf16, false);
        }
#undef SOMI_ROUTE
    }
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(moe_route_kernel<float>, dim3(n_tokens), dim3(64), 0, stream, (const float*)x, row_stride, router,
                           tiled ? logits : nullptr, width, experts, top, groups, keep, sigmoid_scores, normalize, chosen, weight);
    else
        hipLaunchKernelGGL(moe_route_kernel<bf16>, dim3(n_tokens), dim3(64), 0, stream, (const bf16*)x, row_stride, router,
                           tiled ? logits : nullptr, width, experts, top, groups, keep, sigmoid_scores, normalize, chosen, weight);
    SOMI_LAUNCH_CHECK("moe_route");
    return 0;
}

// One workgroup.  tiles: [max_tiles, 3] = (expert or -1, first sorted row, rows).
__global__ void __launch_bounds__(1024)
moe_align_kernel(const int* __restrict__ chosen, int pairs, int experts, int tile_rows, int max_tiles,
                 int* __restrict__ order, int* __restrict__ offsets, int* __restrict__ tiles) {
    __shared__ int count[MOE_MAX_EXPERTS];
    __shared__ int cursor[MOE_MAX_EXPERTS];
    for (int e = threadIdx.x; e < experts; e += 1024) count[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < pairs; p += 1024) atomicAdd(&count[chosen[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, tile = 0;
        for (int e = 0; e < experts; ++e) {
            offsets[e] = at;
            cursor[e] = at;
            for (int r = 0; r < count[e] && tile < max_tiles; r += tile_rows, ++tile) {
                tiles[tile * 3] = e;
                tiles[tile * 3 + 1] = at + r;
                tiles[tile * 3 + 2] = count[e] - r < tile_rows ? count[e] - r : tile_rows;
            }
            at += count[e];
        }
        offsets[experts] = at;
        for (; tile < max_tiles; ++tile) {
            tiles[tile * 3] = -1;
            tiles[tile * 3 + 1] = 0;
            tiles[tile * 3 + 2] = 0;
        }
    }
    __syncthreads();
    for (int p = threadIdx.x; p < pairs; p += 1024) order[atomicAdd(&cursor[chosen[p]], 1)] = p;
}

extern "C" int somi_moe_max_tiles(int pairs, int experts, int tile_rows) {
    return ceil_div(pairs, tile_rows) + experts;
}

extern "C" int somi_moe_align(const int* chosen, int pairs, int experts, int tile_rows, int max_tiles, int* order,
                              int* offsets, int* tiles, hipStream_t stream) {
    SOMI_REQUIRE(pairs >= 0 && experts > 0 && experts <= MOE_MAX_EXPERTS && tile_rows > 0, "moe_align: bad sizes");
    SOMI_REQUIRE(max_tiles >= somi_moe_max_tiles(pairs, experts, tile_rows), "moe_align: %d tiles cannot hold %d pairs of %d experts",
                 max_tiles, pairs, experts);
    hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), 0, stream, chosen, pairs, experts, tile_rows, max_tiles, order,
                       offsets, tiles);
    SOMI_LAUNCH_CHECK("moe_align");
    return 0;
}

// The experts' products over the sorted rows, plain multiply-adds with float32 sums: a workgroup owns one row tile
// (MOE_TILE_ROWS sorted rows of one expert) and 64 output columns, K goes through LDS 32 at a time.
//   GATED: rows are gathered from x by token (pair / top); W: [experts, 2 F, K] (gate rows, then up rows); the end
//          applies the gated unit and writes act[sorted row, F] in T.
//   else : rows are act's sorted rows; W: [experts, N, K]; the end multiplies by the pair's weight and writes
//          y[pair, N] in float32.
template <typename T, bool GATED>
__global__ void __launch_bounds__(256)
moe_product_kernel(const T* __restrict__ a, int64_t a_stride, const T* __restrict__ w, const int* __restrict__ tiles,
                   const int* __restrict__ order, const float* __restrict__ pair_weight, int top, int n_out, int K,
                   float limit, float alpha, float shift, void* __restrict__ out_) {
    __shared__ float As[MOE_TILE_ROWS][33];
    __shared__ float Ws[64][33];
    __shared__ float Us[GATED ? 64 : 1][33];
    __shared__ int pair_of[MOE_TILE_ROWS];
    const int expert = tiles[blockIdx.x * 3];
    if (expert < 0) return;
    const int first = tiles[blockIdx.x * 3 + 1], rows = tiles[blockIdx.x * 3 + 2];
    const int col0 = blockIdx.y * 64;
    const int tid = threadIdx.x;
    if (tid < MOE_TILE_ROWS) pair_of[tid] = tid < rows ? order[first + tid] : -1;
    __syncthreads();
    const int r = tid >> 4, cg = tid & 15;                    // the thread's row and its four columns cg * 4 ..
    const T* wg = w + (int64_t)expert * (GATED ? 2 : 1) * n_out * K;
    float acc[4] = {0.f, 0.f, 0.f, 0.f}, acu[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < K; k0 += 32) {
        for (int i = tid; i < MOE_TILE_ROWS * 32; i += 256) {
            const int rr = i >> 5, kk = i & 31;
            float v = 0.f;
            if (rr < rows && k0 + kk < K) {
                const int64_t src = GATED ? pair_of[rr] / top : first + rr;
                v = to_float(a[src * a_stride + k0 + kk]);
            }
            As[rr][kk] = v;
        }
        for (int i = tid; i < 64 * 32; i += 256) {
            const int cc = i >> 5, kk = i & 31;
            const bool in = col0 + cc < n_out && k0 + kk < K;
            Ws[cc][kk] = in ? to_float(wg[(int64_t)(col0 + cc) * K + k0 + kk]) : 0.f;
            if (GATED) Us[cc][kk] = in ? to_float(wg[(int64_t)(n_out + col0 + cc) * K + k0 + kk]) : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int kk = 0; kk < 32; ++kk) {
            const float av = As[r][kk];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[j] += av * Ws[cg * 4 + j][kk];
                if (GATED) acu[j] += av * Us[cg * 4 + j][kk];
            }
        }
        __syncthreads();
    }
    if (r >= rows) return;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int c = col0 + cg * 4 + j;
        if (c >= n_out) continue;
        const int pair = pair_of[r];
        const float pw = pair_weight != nullptr ? pair_weight[pair] : 1.0f;
        if (GATED) {
            ((T*)out_)[(int64_t)(first + r) * n_out + c] = from_float<T>(clamped_glu(pw * acc[j], pw * acu[j], limit, alpha, shift));
        } else {
            ((float*)out_)[(int64_t)pair * n_out + c] = pw * acc[j];
        }
    }
}

extern "C" int somi_moe_product(const void* a, int64_t a_stride, const void* w, int dtype, int gated, const int* tiles,
                                int max_tiles, const int* order, const float* pair_weight, int top, int n_out, int K,
                                float limit, float alpha, float shift, void* out, hipStream_t stream) {
    SOMI_REQUIRE(max_tiles >= 0 && n_out > 0 && K > 0 && top > 0 && a_stride >= K, "moe_product: bad sizes");
    if (max_tiles == 0) return 0;
    const dim3 grid(max_tiles, ceil_div(n_out, 64));
    SOMI_REQUIRE(grid.y <= 65535, "moe_product: too many columns");
#define SOMI_MOE(T, G)                                                                                                   \
    hipLaunchKernelGGL((moe_product_kernel<T, G>), grid, dim3(256), 0, stream, (const T*)a, a_stride, (const T*)w, tiles, order, \
                       pair_weight, top, n_out, K, limit, alpha, shift, out)
    if (dtype == SOMI_F32) {
        if (gated) SOMI_MOE(float, true); else SOMI_MOE(float, false);
    } else if (dtype == SOMI_BF16) {
        if (gated) SOMI_MOE(bf16, true); else SOMI_MOE(bf16, false);
    } else {
        return somi_fail("moe_product: unknown dtype %d", dtype);
    }
#undef SOMI_MOE
    SOMI_LAUNCH_CHECK("moe_product");
    return 0;
}

// The same products on the matrix cores (bfloat16, K a multiple of 8, rows aligned to 16 bytes): a workgroup owns one
// row tile of up to 64 sorted rows and 4 x 64 output columns (GATED: 4 x 32 columns of gate and the same of up), a
// wavefront up to four 16-row fragments (as many as the tile has rows for) against four 16-column fragments of `v_mfma_f32_16x16x32_bf16`.  Both operands have
// K contiguous in memory, so a lane's fragment is one 16-byte load (rows of x by token, rows of W by output column);
// the next K step's fragments are asked for before this step's products.  Sums run over K in one order per row.
typedef __attribute__((ext_vector_type(8))) __bf16 moe_bf16x8;
typedef __attribute__((ext_vector_type(4))) float moe_f32x4;
#define MOE_MFMA_ROWS 64
#define MOE_MFMA_FRAGS (MOE_MFMA_ROWS / 16)

// FRAGS: row fragments of a tile (4: up to 64 rows; 1: up to 16 rows, for steps of a few tokens, where a tile is an
// expert's one or two rows and the time is the weights' way from memory).  KS: K steps of 32 whose fragments are asked
// for together, a round ahead (1 with four row fragments; 4 with one, so that a lane has twenty loads in flight).
template <bool GATED, int FRAGS, int KS>
__global__ void __launch_bounds__(256)
moe_product_mfma_kernel(const bf16* __restrict__ a, int64_t a_stride, const bf16* __restrict__ w,
                        const int* __restrict__ tiles, const int* __restrict__ order,
                        const float* __restrict__ pair_weight, int top, int n_out, int K, float limit, float alpha,
                        float shift, void* __restrict__ out_) {
    const int expert = tiles[blockIdx.x * 3];
    if (expert < 0) return;
    const int first = tiles[blockIdx.x * 3 + 1], rows = tiles[blockIdx.x * 3 + 2];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    constexpr int WAVE_COLS = GATED ? 32 : 64;           // output columns of a wavefront
    const int col0 = (blockIdx.y * 4 + wave) * WAVE_COLS;
    if (col0 >= n_out) return;
    const bf16* wg = w + (int64_t)expert * (GATED ? 2 : 1) * n_out * K;
    // this lane's rows of the two operands
    const bf16* arow[FRAGS];
    bool alive[FRAGS];
#pragma unroll
    for (int f = 0; f < FRAGS; ++f) {
        const int row = f * 16 + r;
        alive[f] = row < rows;
        const int64_t src = alive[f] ? (GATED ? (int64_t)(order[first + row] / top) : (int64_t)(first + row)) : 0;
        arow[f] = a + src * a_stride + g * 8;
    }
    const bf16* brow[4];
    bool blive[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        // GATED: fragments 0, 1 are gate columns col0 .. col0 + 31, fragments 2, 3 the up rows of the same columns
        const int col = GATED ? col0 + (c & 1) * 16 + r : col0 + c * 16 + r;
        blive[c] = col < n_out;
        const int64_t wrow = GATED ? (int64_t)(c >> 1) * n_out + col : (int64_t)col;
        brow[c] = wg + (blive[c] ? wrow : 0) * K + g * 8;
    }
    const int frags = (rows + 15) >> 4;               // the same for the whole workgroup
    moe_f32x4 acc[FRAGS][4];
#pragma unroll
    for (int f = 0; f < FRAGS; ++f)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[f][c] = moe_f32x4{0.f, 0.f, 0.f, 0.f};
    const moe_bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    moe_bf16x8 fa[KS][FRAGS], fb[KS][4], na[KS][FRAGS], nb[KS][4];
    auto fetch = [&](moe_bf16x8 (&xa)[KS][FRAGS], moe_bf16x8 (&xb)[KS][4], int k0) {
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const bool inside = k0 + s * 32 + g * 8 < K;
#pragma unroll
            for (int f = 0; f < FRAGS; ++f)
                xa[s][f] = (inside && alive[f]) ? *reinterpret_cast<const moe_bf16x8*>(arow[f] + k0 + s * 32) : zero;
#pragma unroll
            for (int c = 0; c < 4; ++c)
                xb[s][c] = (inside && blive[c]) ? *reinterpret_cast<const moe_bf16x8*>(brow[c] + k0 + s * 32) : zero;
        }
    };
    fetch(fa, fb, 0);
    for (int k0 = 0; k0 < K; k0 += 32 * KS) {
        if (k0 + 32 * KS < K) fetch(na, nb, k0 + 32 * KS);
#pragma unroll
        for (int s = 0; s < KS; ++s)
#pragma unroll
            for (int f = 0; f < FRAGS; ++f)
                if (f < frags) {
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        acc[f][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[s][f], fb[s][c], acc[f][c], 0, 0, 0);
                }
#pragma unroll
        for (int s = 0; s < KS; ++s) {
#pragma unroll
            for (int f = 0; f < FRAGS; ++f) fa[s][f] = na[s][f];
#pragma unroll
            for (int c = 0; c < 4; ++c) fb[s][c] = nb[s][c];
        }
    }
    // a lane holds rows g * 4 + i of a fragment's 16 and column r of its 16
#pragma unroll
    for (int f = 0; f < FRAGS; ++f)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = f * 16 + g * 4 + i;
            if (row >= rows) continue;
            const int pair = order[first + row];
            const float pw = pair_weight != nullptr ? pair_weight[pair] : 1.0f;
            if (GATED) {
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    const int col = col0 + c * 16 + r;
                    if (col < n_out)
                        ((bf16*)out_)[(int64_t)(first + row) * n_out + col] =
                            (bf16)clamped_glu(pw * acc[f][c][i], pw * acc[f][c + 2][i], limit, alpha, shift);
                }
            } else {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int col = col0 + c * 16 + r;
                    if (col < n_out) ((float*)out_)[(int64_t)pair * n_out + col] = pw * acc[f][c][i];
                }
            }
        }
}

#define MOE_BIG_ROWS 128

// The same for experts with many rows (prompt portions), both operands through LDS, `32x32x16` matrix instructions:
// a workgroup owns a row tile of up to 128 sorted rows and 128 rows of the expert's matrix (GATED: 64 gate rows and the 64 up rows of the same columns), its four wavefronts a
// 64 x 64 quarter each (two row fragments x two column fragments of 32; GATED: a wavefront's column fragments are gate
// and up of the same 32 columns, so the gated unit needs no exchange).  A round is 64 values of K: every thread brings
// four 16-byte pieces of the rows and four of the matrix into registers two rounds ahead (two sets of registers) and
// stores them into the LDS buffer of the round (rows padded by 16 bytes: a fragment's 16-byte reads of 16 rows fall on different banks).
typedef __attribute__((ext_vector_type(16))) float moe_f32x16;
#define MOE_TILE_BK 64
#define MOE_TILE_ROW_BYTES (MOE_TILE_BK * 2 + 16)

template <bool GATED>
__global__ void __launch_bounds__(256)
moe_product_tile_kernel(const bf16* __restrict__ a, int64_t a_stride, const bf16* __restrict__ w,
                        const int* __restrict__ tiles, const int* __restrict__ order,
                        const float* __restrict__ pair_weight, int top, int n_out, int K, float limit, float alpha,
                        float shift, void* __restrict__ out_) {
    __shared__ __attribute__((aligned(16))) char lds_a[2][128 * MOE_TILE_ROW_BYTES];
    __shared__ __attribute__((aligned(16))) char lds_b[2][128 * MOE_TILE_ROW_BYTES];
    const int expert = tiles[blockIdx.x * 3];
    if (expert < 0) return;
    const int first = tiles[blockIdx.x * 3 + 1], rows = tiles[blockIdx.x * 3 + 2];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;
    const int frow = lane & 31, fk = lane >> 5;
    constexpr int COLS = GATED ? 64 : 128;                      // output columns of a workgroup
    const int col_base = blockIdx.y * COLS;
    const bf16* wg = w + (int64_t)expert * (GATED ? 2 : 1) * n_out * K;
    // the pieces a thread stages: piece p = tid + 256 j is the 16 bytes p % 8 of row p / 8 (of the rows and of the matrix)
    const bf16* arow[4];
    const bf16* brow[4];
    bool alive[4], blive[4];
    int soff[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int p = tid + 256 * j, row = p >> 3, piece = p & 7;
        soff[j] = row * MOE_TILE_ROW_BYTES + piece * 16;
        alive[j] = row < rows;
        const int64_t src = alive[j] ? (GATED ? (int64_t)(order[first + row] / top) : (int64_t)(first + row)) : 0;
        arow[j] = a + src * a_stride + piece * 8;
        // LDS row of the matrix: wavefront column wn' = row / 64, its fragment f = (row / 32) % 2, column c = row % 32
        const int wq = row >> 6, f = (row >> 5) & 1, c = row & 31;
        const int col = GATED ? col_base + wq * 32 + c : col_base + wq * 64 + f * 32 + c;
        blive[j] = col < n_out;
        const int64_t wrow = GATED ? (int64_t)f * n_out + col : (int64_t)col;
        brow[j] = wg + (blive[j] ? wrow : 0) * K + piece * 8;
    }
    const int mfrags = min(2, (rows - wm * 64 + 31) >> 5);     // row fragments of this wavefront that hold rows (<= 0: none)
    moe_f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    const moe_bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    // two sets of staging registers: a round's pieces are asked of memory two rounds before they go into LDS
    moe_bf16x8 sa0[4], sb0[4], sa1[4], sb1[4];
    auto fetch = [&](moe_bf16x8 (&sa)[4], moe_bf16x8 (&sb)[4], int k0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool inside = k0 + ((tid + 256 * j) & 7) * 8 < K;
            sa[j] = (inside && alive[j]) ? *reinterpret_cast<const moe_bf16x8*>(arow[j] + k0) : zero;
            sb[j] = (inside && blive[j]) ? *reinterpret_cast<const moe_bf16x8*>(brow[j] + k0) : zero;
        }
    };
    auto round = [&](moe_bf16x8 (&sa)[4], moe_bf16x8 (&sb)[4], int buf, int k_next) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            *reinterpret_cast<moe_bf16x8*>(lds_a[buf] + soff[j]) = sa[j];
            *reinterpret_cast<moe_bf16x8*>(lds_b[buf] + soff[j]) = sb[j];
        }
        __syncthreads();
        if (k_next < K) fetch(sa, sb, k_next);
        if (mfrags > 0) {
#pragma unroll
            for (int ks = 0; ks < MOE_TILE_BK / 16; ++ks) {
                moe_bf16x8 fa[2], fb[2];
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    fa[i] = *reinterpret_cast<const moe_bf16x8*>(lds_a[buf] + (wm * 64 + i * 32 + frow) * MOE_TILE_ROW_BYTES + ks * 32 + fk * 16);
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    fb[j] = *reinterpret_cast<const moe_bf16x8*>(lds_b[buf] + (wn * 64 + j * 32 + frow) * MOE_TILE_ROW_BYTES + ks * 32 + fk * 16);
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    if (i < mfrags) {
#pragma unroll
                        for (int j = 0; j < 2; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);   // D[row][column]
                    }
            }
        }
    };
    fetch(sa0, sb0, 0);
    if (MOE_TILE_BK < K) fetch(sa1, sb1, MOE_TILE_BK);
    for (int k0 = 0; k0 < K; k0 += 2 * MOE_TILE_BK) {
        round(sa0, sb0, 0, k0 + 2 * MOE_TILE_BK);
        if (k0 + MOE_TILE_BK >= K) break;
        round(sa1, sb1, 1, k0 + 3 * MOE_TILE_BK);
    }
    // D[row][column]: lane l has column l % 32 of a fragment and, in registers 4 g .. 4 g + 3, the rows 8 g + 4 (l / 32) + 0..3
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = wm * 64 + i * 32 + 8 * g + 4 * fk + e;
                if (row >= rows) continue;
                const int pair = order[first + row];
                const float pw = pair_weight != nullptr ? pair_weight[pair] : 1.0f;
                if (GATED) {
                    const int col = col_base + wn * 32 + frow;
                    if (col < n_out)
                        ((bf16*)out_)[(int64_t)(first + row) * n_out + col] =
                            (bf16)clamped_glu(pw * acc[i][0][4 * g + e], pw * acc[i][1][4 * g + e], limit, alpha, shift);
                } else {
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const int col = col_base + wn * 64 + j * 32 + frow;
                        if (col < n_out) ((float*)out_)[(int64_t)pair * n_out + col] = pw * acc[i][j][4 * g + e];
                    }
                }
            }
}

extern "C" int somi_moe_product_mfma(const void* a, int64_t a_stride, const void* w, int gated, const int* tiles,
                                     int max_tiles, int tile_rows, const int* order, const float* pair_weight, int top,
                                     int n_out, int K, float limit, float alpha, float shift, void* out,
                                     hipStream_t stream) {
    SOMI_REQUIRE(tile_rows == 16 || tile_rows == MOE_MFMA_ROWS || tile_rows == MOE_BIG_ROWS,
                 "moe_product_mfma: tiles of %d rows (16, %d or %d)", tile_rows, MOE_MFMA_ROWS, MOE_BIG_ROWS);
    SOMI_REQUIRE(max_tiles >= 0 && n_out > 0 && K > 0 && top > 0 && a_stride >= K, "moe_product_mfma: bad sizes");
    SOMI_REQUIRE(K % 8 == 0 && a_stride % 8 == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0,
                 "moe_product_mfma: K of %d or rows that are not aligned to 16 bytes", K);
    if (max_tiles == 0) return 0;
    const dim3 grid(max_tiles, ceil_div(n_out, gated ? 128 : 256));
    SOMI_REQUIRE(grid.y <= 65535, "moe_product_mfma: too many columns");
    if (tile_rows == MOE_BIG_ROWS) {
        const dim3 tgrid(max_tiles, ceil_div(n_out, gated ? 64 : 128));
        SOMI_REQUIRE(tgrid.y <= 65535, "moe_product_mfma: too many columns");
        if (gated)
            hipLaunchKernelGGL(moe_product_tile_kernel<true>, tgrid, dim3(256), 0, stream, (const bf16*)a, a_stride,
                               (const bf16*)w, tiles, order, pair_weight, top, n_out, K, limit, alpha, shift, out);
        else
            hipLaunchKernelGGL(moe_product_tile_kernel<false>, tgrid, dim3(256), 0, stream, (const bf16*)a, a_stride,
                               (const bf16*)w, tiles, order, pair_weight, top, n_out, K, limit, alpha, shift, out);
    } else if (tile_rows == 16) {
        if (gated)
            hipLaunchKernelGGL((moe_product_mfma_kernel<true, 1, 4>), grid, dim3(256), 0, stream, (const bf16*)a, a_stride,
                               (const bf16*)w, tiles, order, pair_weight, top, n_out, K, limit, alpha, shift, out);
        else
            hipLaunchKernelGGL((moe_product_mfma_kernel<false, 1, 4>), grid, dim3(256), 0, stream, (const bf16*)a, a_stride,
                               (const bf16*)w, tiles, order, pair_weight, top, n_out, K, limit, alpha, shift, out);
    } else if (gated)
        hipLaunchKernelGGL((moe_product_mfma_kernel<true, MOE_MFMA_FRAGS, 1>), grid, dim3(256), 0, stream, (const bf16*)a, a_stride,
                           (const bf16*)w, tiles, order, pair_weight, top, n_out, K, limit, alpha, shift, out);
    else
        hipLaunchKernelGGL((moe_product_mfma_kernel<false, MOE_MFMA_FRAGS, 1>), grid, dim3(256), 0, stream, (const bf16*)a, a_stride,
                           (const bf16*)w, tiles, order, pair_weight, top, n_out, K, limit, alpha, shift, out);
    SOMI_LAUNCH_CHECK("moe_product_mfma");
    return 0;
}

// out[t, :] = sum_j y[t * top + j, :] (+ shared[t, :]).
template <typename T>
__global__ void __launch_bounds__(256)
moe_combine_kernel(const float* __restrict__ y, const T* __restrict__ shared_rows, int top, int width,
                   float* __restrict__ out) {
    const int64_t t = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= width) return;
    float acc = 0.f;
    for (int j = 0; j < top; ++j) acc += y[(t * top + j) * width + c];
    if (shared_rows != nullptr) acc += to_float(shared_rows[t * width + c]);
    out[t * width + c] = acc;
}

extern "C" int somi_moe_combine(const float* y, const void* shared_rows, int shared_dtype, int n_tokens, int top, int width,
                                float* out, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && top > 0 && width > 0, "moe_combine: bad sizes");
    if (n_tokens == 0) return 0;
    const dim3 grid(n_tokens, ceil_div(width, 256));
    SOMI_REQUIRE(grid.y <= 65535, "moe_combine: rows too wide");
    if (shared_rows == nullptr || shared_dtype == SOMI_F32)
        hipLaunchKernelGGL(moe_combine_kernel<float>, grid, dim3(256), 0, stream, y, (const float*)shared_rows, top,
                           width, out);
    else if (shared_dtype == SOMI_BF16)
        hipLaunchKernelGGL(moe_combine_kernel<bf16>, grid, dim3(256), 0, stream, y, (const bf16*)shared_rows, top,
                           width, out);
    else
        return somi_fail("moe_combine: unknown dtype %d", shared_dtype);
    SOMI_LAUNCH_CHECK("moe_combine");
    return 0;
}

// The gated unit on a dense product's rows [gate (F) | up (F)] -> [F].
template <typename T>
__global__ void __launch_bounds__(256)
clamped_glu_kernel(const T* __restrict__ gate_up, int F, float limit, float alpha, float shift, T* __restrict__ out,
                   int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) {
        const int64_t t = i / F;
        const int c = (int)(i - t * F);
        out[i] = from_float<T>(clamped_glu(to_float(gate_up[t * 2 * F + c]), to_float(gate_up[t * 2 * F + F + c]), limit,
                                           alpha, shift));
    }
}

extern "C" int somi_clamped_glu(const void* gate_up, int dtype, int n_tokens, int F, float limit, float alpha, float shift,
                                void* out, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && F > 0, "clamped_glu: bad sizes");
    if (n_tokens == 0) return 0;
    const int64_t count = (int64_t)n_tokens * F;
    const int grid = (int)(ceil_div64(count, 256) < 65536 ? ceil_div64(count, 256) : 65536);
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(clamped_glu_kernel<float>, dim3(grid), dim3(256), 0, stream, (const float*)gate_up, F, limit, alpha,
                           shift, (float*)out, count);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(clamped_glu_kernel<bf16>, dim3(grid), dim3(256), 0, stream, (const bf16*)gate_up, F, limit, alpha,
                           shift, (bf16*)out, count);
    else
        return somi_fail("clamped_glu: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("clamped_glu");
    return 0;
}
