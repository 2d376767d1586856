// Attention over a shared low-rank latent: every past token keeps one vector [c (rank) | r (rot)] for all heads, c
// the normed latent from which a head's keys and values are linear maps (k_h = U_h c, v_h = V_h c), r one rotated key
// part that all heads share.  Because the maps are linear they move to the query's side: with a_h = U_h^T q_h,
//
//     score(i, j, h) = scale * (a_h(i) . c(j) + qr_h(i) . r(j)),      ctx_h(i) = sum_j p(i, j, h) c(j),
//
// and the head's output is V_h ctx_h, computed by the caller.  So the kernels here see one key/value "head" of
// rank + rot key channels whose first rank channels are also the values, and H query heads per token.
//
// The softmax has a sink: a learned number per head stands in the denominator beside the keys' terms, with no key
// and no value; it is not scaled.  Causal: position i sees every j <= i of its request.
//
//   prepare   RMS norm of the query latent (rows out in the compute dtype), RMS norm of c and rotation of r into the
//             request's pages (and c once more, transposed inside its page, where the matrix-core kernel wants it)
//   place     a head's rotated query part goes behind its a_h in the query rows that the attention reads
//   plain     one workgroup per (token, head), float32 online softmax over 128-key tiles aligned to absolute
//             positions, which starts from the sink (running maximum = sink, running sum = 1, output 0)
#include "common.h"

// One workgroup per token.  rows: [n, row_stride] float32 = [query latent (q_rank) | c as projected (rank) | r (rot)]
// (the last two only if latent != null).  Without q_weight the first q_rank values are the queries themselves and
// pass unnormed.  inv_freq: [rot_dims / 2]; channel i of r turns with channel i + rot_dims/2 (pairing 0) or channel 2i
// with 2i + 1 (pairing 1) by the angle position * inv_freq[i], both cosine and sine times `amplitude`; channels from
// rot_dims on pass.
template <typename T>
__global__ void __launch_bounds__(256)
latent_prepare_kernel(const float* __restrict__ rows, int64_t row_stride, int q_rank, int rank, int rot,
                      const float* __restrict__ q_weight, const float* __restrict__ c_weight, float eps,
                      const float* __restrict__ inv_freq, int rot_dims, float amplitude, int pairing,
                      const int* __restrict__ positions, const int* __restrict__ slots, T* __restrict__ q_latent,
                      T* __restrict__ latent, T* __restrict__ latent_t, int page_size) {
    __shared__ float red[16];
    const int64_t t = blockIdx.x;
    const float* row = rows + t * row_stride;
    float ss = 0.f;
    if (q_weight != nullptr) {
        for (int i = threadIdx.x; i < q_rank; i += 256) ss = fmaf(row[i], row[i], ss);
        ss = block_sum<256>(ss, red);
        const float inv_q = 1.0f / sqrtf(ss / (float)q_rank + eps);
        for (int i = threadIdx.x; i < q_rank; i += 256) q_latent[t * q_rank + i] = from_float<T>(row[i] * inv_q * q_weight[i]);
    } else {
        for (int i = threadIdx.x; i < q_rank; i += 256) q_latent[t * q_rank + i] = from_float<T>(row[i]);
    }
    if (latent == nullptr) return;
    const int slot = slots[t];
    if (slot < 0) return;                                  // a padding token keeps nothing
    const float* kv = row + q_rank;
    ss = 0.f;
    for (int i = threadIdx.x; i < rank; i += 256) ss = fmaf(kv[i], kv[i], ss);
    ss = block_sum<256>(ss, red);
    const float inv_c = 1.0f / sqrtf(ss / (float)rank + eps);
    T* kept = latent + (int64_t)slot * (rank + rot);
    // the same latent once more, transposed inside its page ([pages, rank, page]), for kernels that read it by channel
    T* kept_t = latent_t != nullptr ? latent_t + (int64_t)(slot / page_size) * rank * page_size + slot % page_size : nullptr;
    for (int i = threadIdx.x; i < rank; i += 256) {
        const T v = from_float<T>(kv[i] * inv_c * c_weight[i]);
        kept[i] = v;
        if (kept_t != nullptr) kept_t[(int64_t)i * page_size] = v;
    }
    const float p = (float)positions[t];
    const int half = rot_dims / 2;
    for (int i = threadIdx.x; i < rot; i += 256) {
        float v = kv[rank + i];
        if (i < rot_dims) {
            const bool first = pairing == 0 ? i < half : (i & 1) == 0;
            const int f = pairing == 0 ? (first ? i : i - half) : i >> 1;
            const float angle = p * inv_freq[f];
            const float c = cosf(angle) * amplitude, s = sinf(angle) * amplitude;
            const float other = kv[rank + (pairing == 0 ? (first ? i + half : i - half) : (i ^ 1))];
            v = first ? v * c - other * s : v * c + other * s;
        }
        kept[rank + i] = from_float<T>(v);
    }
}

extern "C" int somi_latent_prepare(const float* rows, int64_t row_stride, int n_tokens, int q_rank, int rank, int rot,
                                   const float* q_weight, const float* c_weight, float eps, const float* inv_freq,
                                   int rot_dims, float amplitude, int pairing, const int* positions, const int* slots,
                                   void* q_latent, void* latent, void* latent_t, int page_size, int dtype,
                                   hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && q_rank > 0 && rank > 0 && rot >= 0, "latent_prepare: bad sizes");
    SOMI_REQUIRE(pairing == 0 || pairing == 1, "latent_prepare: unknown pairing %d", pairing);
    SOMI_REQUIRE(rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0, "latent_prepare: %d rotated channels of %d", rot_dims, rot);
    SOMI_REQUIRE(row_stride >= q_rank + (latent ? rank + rot : 0), "latent_prepare: rows too narrow");
    SOMI_REQUIRE(latent_t == nullptr || (latent != nullptr && page_size > 0), "latent_prepare: transposed pages need the pages and their size");
    if (n_tokens == 0) return 0;
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(latent_prepare_kernel<float>, dim3(n_tokens), dim3(256), 0, stream, rows, row_stride, q_rank,
                           rank, rot, q_weight, c_weight, eps, inv_freq, rot_dims, amplitude, pairing, positions, slots,
                           (float*)q_latent, (float*)latent, (float*)latent_t, page_size);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(latent_prepare_kernel<bf16>, dim3(n_tokens), dim3(256), 0, stream, rows, row_stride, q_rank,
                           rank, rot, q_weight, c_weight, eps, inv_freq, rot_dims, amplitude, pairing, positions, slots,
                           (bf16*)q_latent, (bf16*)latent, (bf16*)latent_t, page_size);
    else
        return somi_fail("latent_prepare: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("latent_prepare");
    return 0;
}

// q: [n, heads * (dim + rot)] as projected (rows q_stride apart, in the queries' type or float32), head by head [dim
// plain | rot to be rotated]; the rotated part of head h goes to queries[t, h, rank .. rank + rot).  A thread per
// (token, head, channel).
template <typename TS, typename T>
__global__ void __launch_bounds__(256)
latent_place_kernel(const TS* __restrict__ q, int64_t q_stride, int heads, int dim, int rot, int rank, const float* __restrict__ inv_freq,
                    int rot_dims, float amplitude, int pairing, const int* __restrict__ positions,
                    T* __restrict__ queries, int64_t count) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    const int ch = (int)(i % rot);
    const int64_t th = i / rot;
    const int h = (int)(th % heads);
    const int64_t t = th / heads;
    const TS* src = q + t * q_stride + h * (int64_t)(dim + rot) + dim;
    float v = to_float(src[ch]);
    if (ch < rot_dims) {
        const int half = rot_dims / 2;
        const bool first = pairing == 0 ? ch < half : (ch & 1) == 0;
        const int f = pairing == 0 ? (first ? ch : ch - half) : ch >> 1;
        const float angle = (float)positions[t] * inv_freq[f];
        const float c = cosf(angle) * amplitude, s = sinf(angle) * amplitude;
        const float other = to_float(src[pairing == 0 ? (first ? ch + half : ch - half) : (ch ^ 1)]);
        v = first ? v * c - other * s : v * c + other * s;
    }
    queries[(t * heads + h) * (int64_t)(rank + rot) + rank + ch] = from_float<T>(v);
}

extern "C" int somi_latent_place(const void* q, int q_dtype, int64_t q_stride, int dtype, int n_tokens, int heads, int dim, int rot, int rank,
                                 const float* inv_freq, int rot_dims, float amplitude, int pairing, const int* positions,
                                 void* queries, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && heads > 0 && dim > 0 && rot >= 0 && rank > 0, "latent_place: bad sizes");
    SOMI_REQUIRE(pairing == 0 || pairing == 1, "latent_place: unknown pairing %d", pairing);
    SOMI_REQUIRE(rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0, "latent_place: %d rotated channels of %d", rot_dims, rot);
    const int64_t count = (int64_t)n_tokens * heads * rot;
    if (count == 0) return 0;
    const dim3 grid((unsigned)ceil_div64(count, 256));
    SOMI_REQUIRE(q_dtype == SOMI_F32 || q_dtype == dtype, "latent_place: the projected queries are float32 or of the queries' type");
    SOMI_REQUIRE(q_stride >= (int64_t)heads * (dim + rot), "latent_place: rows too narrow");
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL((latent_place_kernel<float, float>), grid, dim3(256), 0, stream, (const float*)q, q_stride, heads,
                           dim, rot, rank, inv_freq, rot_dims, amplitude, pairing, positions, (float*)queries, count);
    else if (dtype == SOMI_BF16 && q_dtype == SOMI_F32)
        hipLaunchKernelGGL((latent_place_kernel<float, bf16>), grid, dim3(256), 0, stream, (const float*)q, q_stride, heads,
                           dim, rot, rank, inv_freq, rot_dims, amplitude, pairing, positions, (bf16*)queries, count);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL((latent_place_kernel<bf16, bf16>), grid, dim3(256), 0, stream, (const bf16*)q, q_stride, heads,
                           dim, rot, rank, inv_freq, rot_dims, amplitude, pairing, positions, (bf16*)queries, count);
    else
        return somi_fail("latent_place: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("latent_place");
    return 0;
}

// ------------------------------------------------------------------------------------------------ plain attention
#define LATENT_PLAIN_NT 128
#define LATENT_PLAIN_ACC 8            // value channels a thread sums: rank <= 8 * 128

template <typename T>
__global__ void __launch_bounds__(LATENT_PLAIN_NT)
latent_attention_plain_kernel(const T* __restrict__ queries, const T* __restrict__ latent,
                              const int* __restrict__ block_table, int max_blocks, const int* __restrict__ token_entry,
                              const int* __restrict__ positions, int heads, int rank, int rot, int page_size,
                              int window, float scale, const float* __restrict__ sink, T* __restrict__ out) {
    constexpr int NT = LATENT_PLAIN_NT;
    extern __shared__ float smem[];
    const int D = rank + rot;
    float* qs = smem;                          // [D]
    float* ps = qs + ((D + 1) & ~1);           // [NT] softmax weights of the tile
    float* red = ps + NT;                      // [16]
    int64_t* rowoff = (int64_t*)(red + 16);    // [NT] element offset of each key row of the tile

    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int e = token_entry[t];
    const int p = positions[t];
    const int* table = block_table + (int64_t)e * max_blocks;
    for (int d = tid; d < D; d += NT) qs[d] = to_float(queries[((int64_t)t * heads + h) * D + d]);

    // the sink: a term exp(sink - m) with no value; without one the first walked tile, which holds a key that is
    // seen, sets the maximum
    float m = sink != nullptr ? sink[h] : -INFINITY, l = sink != nullptr ? 1.f : 0.f;
    const int lo = window > 0 ? max(0, p - window + 1) : 0;     // the first key the token sees
    float acc[LATENT_PLAIN_ACC];
#pragma unroll
    for (int r = 0; r < LATENT_PLAIN_ACC; ++r) acc[r] = 0.f;
    for (int tile = lo / NT; tile <= p / NT; ++tile) {
        const int pos = tile * NT + tid;
        const bool valid = pos >= lo && pos <= p;
        __syncthreads();                        // qs ready; the previous tile's ps and rowoff no longer read
        float s = -INFINITY;
        if (valid) {
            const int64_t page = table[pos / page_size];
            const int64_t off = (page * page_size + pos % page_size) * (int64_t)D;
            rowoff[tid] = off;
            const T* kr = latent + off;
            float dot = 0.f;
            for (int d = 0; d < D; ++d) dot = fmaf(qs[d], to_float(kr[d]), dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, block_max<NT>(s, red));
        const float corr = expf(m - m_new);
        const float w = valid ? expf(s - m_new) : 0.f;
        ps[tid] = w;
        l = l * corr + block_sum<NT>(w, red);
        m = m_new;
        __syncthreads();                        // ps and rowoff visible
        const int j0 = (lo > tile * NT ? lo : tile * NT) - tile * NT;
        const int j1 = (p < tile * NT + NT - 1 ? p : tile * NT + NT - 1) - tile * NT;
#pragma unroll
        for (int r = 0; r < LATENT_PLAIN_ACC; ++r) {
            const int d = tid + r * NT;
            if (d < rank) {
                float a = acc[r] * corr;
                for (int j = j0; j <= j1; ++j) a = fmaf(ps[j], to_float(latent[rowoff[j] + d]), a);
                acc[r] = a;
            }
        }
    }
#pragma unroll
    for (int r = 0; r < LATENT_PLAIN_ACC; ++r) {
        const int d = tid + r * NT;
        if (d < rank) out[((int64_t)t * heads + h) * rank + d] = from_float<T>(acc[r] / l);
    }
}

// queries: [n_tokens, heads, rank + rot]; latent: [pages, page_size, rank + rot]; block_table: [entries, max_blocks];
// sink: [heads] float32 or null for a softmax over the keys alone; window: the keys a token sees, itself included
// (0: all); out: [n_tokens, heads, rank], the weighted sums of the latents.
extern "C" int somi_latent_attention_plain(const void* queries, int dtype, const void* latent, const int* block_table,
                                           int max_blocks, const int* token_entry, const int* positions, int n_tokens,
                                           int heads, int rank, int rot, int page_size, int window, float scale,
                                           const float* sink, void* out, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && heads > 0 && rank > 0 && rot >= 0 && page_size > 0 && max_blocks > 0 && window >= 0,
                 "latent_attention: bad sizes");
    SOMI_REQUIRE(rank <= LATENT_PLAIN_ACC * LATENT_PLAIN_NT, "latent_attention: a latent of %d is more than the supported %d",
                 rank, LATENT_PLAIN_ACC * LATENT_PLAIN_NT);
    SOMI_REQUIRE(heads <= 65535, "latent_attention: too many heads");
    if (n_tokens == 0) return 0;
    const int D = rank + rot;
    const dim3 grid(n_tokens, heads);
    const size_t smem = (size_t)(((D + 1) & ~1) + LATENT_PLAIN_NT + 16) * sizeof(float) + LATENT_PLAIN_NT * sizeof(int64_t);
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(latent_attention_plain_kernel<float>, grid, dim3(LATENT_PLAIN_NT), smem, stream,
                           (const float*)queries, (const float*)latent, block_table, max_blocks, token_entry, positions,
                           heads, rank, rot, page_size, window, scale, sink, (float*)out);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(latent_attention_plain_kernel<bf16>, grid, dim3(LATENT_PLAIN_NT), smem, stream,
                           (const bf16*)queries, (const bf16*)latent, block_table, max_blocks, token_entry, positions,
                           heads, rank, rot, page_size, window, scale, sink, (bf16*)out);
    else
        return somi_fail("latent_attention: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("latent_attention_plain");
    return 0;
}
