// Grouped-query attention whose heads' softmax weights are mixed by a matrix before they meet the values.
//
//     s_g(i, j) = cap * tanh(scale * q_g(i) . k_kv(g)(j) / cap)            (cap = 0: scale * q . k as it is)
//     p_g(i, j) = exp(s_g(i, j)) / (extra + sum_j' exp(s_g(i, j')))         (extra = 1: as if one more key of score 0 and value 0 were seen)
//     w_h(i, j) = sum_g T[h, g] p_g(i, j)
//     o_h(i)    = sum_j w_h(i, j) v_kv(h)(j)
//
// over the keys j with max(0, i - window + 1) <= j <= i (window = 0: every j <= i).  Keys are rotated by their
// position on their first `rot_dims` channels; values may be rotated by their position over all their channels with
// frequencies of their own, and a head's output is then turned back by the query's position, which leaves the values
// rotated by j - i.  Because the mixed weights need every head's finished softmax, the kernel walks a token's keys
// twice: first the running maximum and the sum of every head, then the weights themselves, their mix and the sum over
// the values.  Scores, softmax, mix, the weighted sum and both rotations are float32.
//
//   store    one workgroup a token: q rotated into the rows the attention reads, k rotated and v (rotated or not) into
//            the token's slot of the pages.  k: [pages, kv_heads, page, dim]; v is transposed inside a page, [pages,
//            kv_heads, vdim, page]: consecutive positions of one channel are adjacent, the operand layout of the
//            weights-times-values product on the matrix cores
//   plain    one workgroup a token, all heads: a wavefront takes a head at a time and its 64 lanes the keys of a
//            64-key tile (tiles aligned to absolute positions), so a head's maximum and sum are wave reductions
#include "common.h"

#define MXA_NT 256
#define MXA_TILE 64
#define MXA_ACC 32            // (head, value channel) sums a thread holds: heads * vdim <= 32 * 256

// pairing 0: channel m turns with m + dims / 2; 1: channel 2m with 2m + 1.  Returns the partner's index and whether
// `ch` is the pair's first channel; `pair` is the index of its frequency.
__device__ __forceinline__ int mxa_partner(int ch, int dims, int pairing, int* pair, bool* first) {
    if (pairing == 0) {
        const int half = dims >> 1;
        *first = ch < half;
        *pair = *first ? ch : ch - half;
        return *first ? ch + half : ch - half;
    }
    *first = (ch & 1) == 0;
    *pair = ch >> 1;
    return ch ^ 1;
}

// rows: [n, heads * dim + kv * dim + kv * vdim] float32 as projected (a layer that reads another's cache: heads * dim
// only, k_cache null).  q_out: [n, heads * dim].
template <typename T>
__global__ void __launch_bounds__(MXA_NT)
mixed_store_kernel(const float* __restrict__ rows, int64_t row_stride, const int* __restrict__ positions,
                   const int* __restrict__ slots, const float* __restrict__ inv_freq, int rot_dims, int pairing,
                   const float* __restrict__ v_freq, int v_pairing, int heads, int kv, int dim, int vdim,
                   T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int page_size) {
    const int64_t t = blockIdx.x;
    const float* row = rows + t * row_stride;
    const float p = (float)positions[t];
    const int q_width = heads * dim, k_width = kv * dim, v_width = kv * vdim;
    const int slot = k_cache != nullptr ? slots[t] : -1;          // a padding token keeps nothing
    const int total = q_width + (slot >= 0 ? k_width + v_width : 0);
    for (int i = threadIdx.x; i < total; i += MXA_NT) {
        if (i < q_width + k_width) {
            const bool is_q = i < q_width;
            const int at = is_q ? i : i - q_width;
            const int h = at / dim, ch = at % dim;
            const float* head = row + (is_q ? 0 : q_width) + h * dim;
            float v = head[ch];
            if (ch < rot_dims) {
                int pair;
                bool first;
                const float other = head[mxa_partner(ch, rot_dims, pairing, &pair, &first)];
                const float angle = p * inv_freq[pair];
                const float c = cosf(angle), s = sinf(angle);
                v = first ? v * c - other * s : v * c + other * s;
            }
            if (is_q) {
                q_out[t * q_width + at] = from_float<T>(v);
            } else {
                const int64_t page = slot / page_size, off = slot % page_size;
                k_cache[((page * kv + h) * page_size + off) * dim + ch] = from_float<T>(v);
            }
        } else {
            const int at = i - q_width - k_width;
            const int h = at / vdim, ch = at % vdim;
            const float* head = row + q_width + k_width + h * vdim;
            float v = head[ch];
            if (v_freq != nullptr) {
                int pair;
                bool first;
                const float other = head[mxa_partner(ch, vdim, v_pairing, &pair, &first)];
                const float angle = p * v_freq[pair];
                const float c = cosf(angle), s = sinf(angle);
                v = first ? v * c - other * s : v * c + other * s;
            }
            const int64_t page = slot / page_size, off = slot % page_size;
            v_cache[((page * kv + h) * vdim + ch) * page_size + off] = from_float<T>(v);
        }
    }
}

extern "C" int somi_mixed_attention_store(const float* rows, int64_t row_stride, int n_tokens, const int* positions,
                                          const int* slots, const float* inv_freq, int rot_dims, int pairing,
                                          const float* v_freq, int v_pairing, int heads, int kv, int dim, int vdim,
                                          void* q_out, void* k_cache, void* v_cache, int page_size, int dtype,
                                          hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && heads > 0 && kv > 0 && dim > 0 && vdim > 0, "mixed_attention_store: bad sizes");
    SOMI_REQUIRE(rot_dims >= 0 && rot_dims <= dim && rot_dims % 2 == 0, "mixed_attention_store: %d rotated channels of %d", rot_dims, dim);
    SOMI_REQUIRE(rot_dims == 0 || inv_freq != nullptr, "mixed_attention_store: a rotation needs its frequencies");
    SOMI_REQUIRE(v_freq == nullptr || vdim % 2 == 0, "mixed_attention_store: rotated values need an even size, got %d", vdim);
    SOMI_REQUIRE((pairing == 0 || pairing == 1) && (v_pairing == 0 || v_pairing == 1), "mixed_attention_store: unknown pairing");
    SOMI_REQUIRE((k_cache == nullptr) == (v_cache == nullptr), "mixed_attention_store: keys and values come together");
    SOMI_REQUIRE(k_cache == nullptr || (slots != nullptr && page_size > 0), "mixed_attention_store: pages need slots and a page size");
    SOMI_REQUIRE(row_stride >= heads * dim + (k_cache ? kv * (dim + vdim) : 0), "mixed_attention_store: rows too narrow");
    if (n_tokens == 0) return 0;
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(mixed_store_kernel<float>, dim3(n_tokens), dim3(MXA_NT), 0, stream, rows, row_stride, positions,
                           slots, inv_freq, rot_dims, pairing, v_freq, v_pairing, heads, kv, dim, vdim, (float*)q_out,
                           (float*)k_cache, (float*)v_cache, page_size);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(mixed_store_kernel<bf16>, dim3(n_tokens), dim3(MXA_NT), 0, stream, rows, row_stride, positions,
                           slots, inv_freq, rot_dims, pairing, v_freq, v_pairing, heads, kv, dim, vdim, (bf16*)q_out,
                           (bf16*)k_cache, (bf16*)v_cache, page_size);
    else
        return somi_fail("mixed_attention_store: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("mixed_attention_store");
    return 0;
}

// ------------------------------------------------------------------------------------------------ plain attention
template <typename T>
__device__ __forceinline__ float mxa_dot(const float* __restrict__ q, const T* __restrict__ k, int dim) {
    float dot = 0.f;
    for (int d = 0; d < dim; ++d) dot = fmaf(q[d], to_float(k[d]), dot);
    return dot;
}

// LDS (floats): q [heads * dim] | talk [heads * heads] | ml [2 * heads] | P [heads * TILE] | W [heads * TILE] |
// O [heads * vdim]; then int64 rowbase [TILE]: page * kv * page_size + offset of each key of the tile (what a key's
// row of kv head 0 starts at, in rows of k; the transposed values are addressed from its two parts).
template <typename T>
__global__ void __launch_bounds__(MXA_NT)
mixed_attention_plain_kernel(const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                             const int* __restrict__ block_table, int max_blocks, const int* __restrict__ token_entry,
                             const int* __restrict__ positions, int heads, int kv, int dim, int vdim, int page_size,
                             int window, float scale, float cap, float extra, const float* __restrict__ talk,
                             const float* __restrict__ v_freq, int v_pairing, T* __restrict__ out) {
    extern __shared__ __attribute__((aligned(16))) float mxa_lds[];
    float* q_s = mxa_lds;
    float* talk_s = q_s + heads * dim;
    float* ml = talk_s + heads * heads;
    float* P = ml + 2 * heads;
    float* W = P + heads * MXA_TILE;
    float* O = W + heads * MXA_TILE;
    int64_t* rowbase = reinterpret_cast<int64_t*>(O + ((heads * vdim + 1) & ~1));
    const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int p = positions[t];
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const int* table = block_table + (int64_t)token_entry[t] * max_blocks;
    const int group = heads / kv;
    for (int i = tid; i < heads * dim; i += MXA_NT) q_s[i] = to_float(q[(int64_t)t * heads * dim + i]);
    for (int i = tid; i < heads * heads; i += MXA_NT)
        talk_s[i] = talk != nullptr ? talk[i] : (i / heads == i % heads ? 1.f : 0.f);
    __syncthreads();
    const int tile0 = lo / MXA_TILE, tile1 = p / MXA_TILE;
    const float inv_cap = cap > 0.f ? 1.0f / cap : 0.f;

    auto key_base = [&](int key) -> int64_t {
        const int64_t page = table[key / page_size];
        return page * kv * page_size + key % page_size;
    };
    auto score = [&](int g, int64_t base) -> float {
        const T* kr = k_cache + (base + (int64_t)(g / group) * page_size) * dim;
        float s = mxa_dot(q_s + g * dim, kr, dim) * scale;
        if (cap > 0.f) s = cap * tanhf(s * inv_cap);
        return s;
    };

    // ---- first walk: every head's maximum and sum
    for (int g = wave; g < heads; g += MXA_NT / 64) {
        float m = extra > 0.f ? 0.f : -INFINITY, l = extra;
        for (int tile = tile0; tile <= tile1; ++tile) {
            const int key = tile * MXA_TILE + lane;
            const bool seen = key >= lo && key <= p;
            const float s = seen ? score(g, key_base(key)) : -INFINITY;
            const float m_new = fmaxf(m, wave_max(s));          // finite: a walked tile holds a key that is seen
            const float e = seen ? expf(s - m_new) : 0.f;
            l = l * expf(m - m_new) + wave_sum(e);
            m = m_new;
        }
        if (lane == 0) {
            ml[2 * g] = m;
            ml[2 * g + 1] = l;
        }
    }
    float acc[MXA_ACC];
#pragma unroll
    for (int r = 0; r < MXA_ACC; ++r) acc[r] = 0.f;
    // ---- second walk: the weights, their mix, the sum over the values
    for (int tile = tile0; tile <= tile1; ++tile) {
        __syncthreads();                       // ml written; the previous tile's P, W and rowbase no longer read
        const int key = tile * MXA_TILE + lane;
        const bool seen = key >= lo && key <= p;
        const int64_t base = seen ? key_base(key) : 0;
        if (wave == 0) rowbase[lane] = base;
        for (int g = wave; g < heads; g += MXA_NT / 64)
            P[g * MXA_TILE + lane] = seen ? expf(score(g, base) - ml[2 * g]) / ml[2 * g + 1] : 0.f;
        __syncthreads();
        for (int i = tid; i < heads * MXA_TILE; i += MXA_NT) {
            const int h = i / MXA_TILE, j = i % MXA_TILE;
            float w = 0.f;
            for (int g = 0; g < heads; ++g) w = fmaf(talk_s[h * heads + g], P[g * MXA_TILE + j], w);
            W[i] = w;
        }
        __syncthreads();
        const int j0 = max(lo, tile * MXA_TILE) - tile * MXA_TILE;
        const int j1 = min(p, tile * MXA_TILE + MXA_TILE - 1) - tile * MXA_TILE;
#pragma unroll
        for (int r = 0; r < MXA_ACC; ++r) {
            const int i = tid + r * MXA_NT;
            if (i < heads * vdim) {
                const int h = i / vdim, d = i % vdim;
                const int c = h / group;
                float a = acc[r];
                for (int j = j0; j <= j1; ++j) {
                    // rowbase = page * kv * page_size + offset with offset < page_size
                    const int64_t page = rowbase[j] / ((int64_t)kv * page_size), off = rowbase[j] % page_size;
                    a = fmaf(W[h * MXA_TILE + j], to_float(v_cache[((page * kv + c) * vdim + d) * page_size + off]), a);
                }
                acc[r] = a;
            }
        }
    }
    // ---- the heads' outputs, turned back by the query's position where the values were turned by theirs
#pragma unroll
    for (int r = 0; r < MXA_ACC; ++r) {
        const int i = tid + r * MXA_NT;
        if (i < heads * vdim) O[i] = acc[r];
    }
    __syncthreads();
    for (int i = tid; i < heads * vdim; i += MXA_NT) {
        float v = O[i];
        if (v_freq != nullptr) {
            const int h = i / vdim, d = i % vdim;
            int pair;
            bool first;
            const float other = O[h * vdim + mxa_partner(d, vdim, v_pairing, &pair, &first)];
            const float angle = (float)p * v_freq[pair];
            const float c = cosf(angle), s = sinf(angle);          // by -angle: the sine changes its sign
            v = first ? v * c + other * s : v * c - other * s;
        }
        out[(int64_t)t * heads * vdim + i] = from_float<T>(v);
    }
}

// q: [n_tokens, heads * dim] rotated; k_cache: [pages, kv, page, dim]; v_cache: [pages, kv, vdim, page]; block_table:
// [entries, max_blocks]; talk: [heads, heads] float32 (to, from) or null for no mix; v_freq: [vdim / 2] float32 or null
// for values that are not rotated; extra: what is added to the softmax's denominator (0 or 1); out: [n_tokens, heads *
// vdim].
extern "C" int somi_mixed_attention_plain(const void* q, int dtype, const void* k_cache, const void* v_cache,
                                          const int* block_table, int max_blocks, const int* token_entry,
                                          const int* positions, int n_tokens, int heads, int kv, int dim, int vdim,
                                          int page_size, int window, float scale, float cap, float extra,
                                          const float* talk, const float* v_freq, int v_pairing, void* out,
                                          hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && heads > 0 && kv > 0 && heads % kv == 0 && dim > 0 && vdim > 0 && page_size > 0 &&
                 max_blocks > 0 && window >= 0, "mixed_attention: bad sizes");
    SOMI_REQUIRE(extra == 0.f || extra == 1.f, "mixed_attention: the denominator takes 0 or 1 more, got %g", (double)extra);
    SOMI_REQUIRE(heads * vdim <= MXA_ACC * MXA_NT, "mixed_attention: %d heads of %d value channels are more than the supported %d",
                 heads, vdim, MXA_ACC * MXA_NT);
    SOMI_REQUIRE(v_freq == nullptr || vdim % 2 == 0, "mixed_attention: rotated values need an even size, got %d", vdim);
    if (n_tokens == 0) return 0;
    const size_t floats = (size_t)heads * dim + (size_t)heads * heads + 2 * heads + 2 * (size_t)heads * MXA_TILE +
                          (((size_t)heads * vdim + 1) & ~(size_t)1);
    const size_t smem = floats * sizeof(float) + MXA_TILE * sizeof(int64_t);
    SOMI_REQUIRE(smem <= 160 * 1024, "mixed_attention: %d heads of %d + %d channels need %zu bytes of LDS, more than 160 KiB",
                 heads, dim, vdim, smem);
    const dim3 grid(n_tokens);
    if (smem > 48 * 1024) {
        // more LDS than a workgroup gets unasked
        const void* kernel = dtype == SOMI_F32 ? (const void*)mixed_attention_plain_kernel<float>
                                               : (const void*)mixed_attention_plain_kernel<bf16>;
        hipError_t err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (err != hipSuccess) return somi_fail("mixed_attention: %s", hipGetErrorString(err));
    }
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(mixed_attention_plain_kernel<float>, grid, dim3(MXA_NT), smem, stream, (const float*)q,
                           (const float*)k_cache, (const float*)v_cache, block_table, max_blocks, token_entry, positions,
                           heads, kv, dim, vdim, page_size, window, scale, cap, extra, talk, v_freq, v_pairing, (float*)out);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(mixed_attention_plain_kernel<bf16>, grid, dim3(MXA_NT), smem, stream, (const bf16*)q,
                           (const bf16*)k_cache, (const bf16*)v_cache, block_table, max_blocks, token_entry, positions,
                           heads, kv, dim, vdim, page_size, window, scale, cap, extra, talk, v_freq, v_pairing, (bf16*)out);
    else
        return somi_fail("mixed_attention: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("mixed_attention_plain");
    return 0;
}
