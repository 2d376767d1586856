// Attention with mixed heads on the matrix cores (bfloat16): see mixed_attention.hip for what is computed.
//
// A workgroup (eight wavefronts) serves `tq` consecutive tokens of the step and ALL their heads, because the mix needs
// every head's weights of a (token, key) pair in one place.  For each key/value head c there is one tile of 16 query
// slots: slot = token * rp + r holds head c * group + r of that token (rp: the power of two >= group; slots with r >=
// group, or of tokens of another request, are dead).  Tokens of one request stand side by side with rising positions;
// where the workgroup's tokens belong to several requests it takes them run by run.
//
//   first walk   a wavefront takes a (key/value head, parity of the 16-key tile) at a time; 16 keys at a time, S^T = K Q^T by `16x16x32`
//                products (K fragments straight from the pages, Q fragments from LDS); a lane holds 4 keys of one slot
//                and keeps a running maximum and sum of its own, joined over the lanes at the end: (m, l) of every slot
//   second walk  32 keys at a time: the same scores again, p = exp(s - m) / l in float32, which goes to LDS by (token,
//                key) and head as two bfloat16 halves (p = hi + lo, so no weight is rounded to eight bits); the mix W^T =
//                P^T T^T as matrix products too (T in two halves as well: hi hi + lo hi + hi lo), whose results go to LDS
//                by key/value head and slot, again in two halves; then O^T = V^T W^T, the V^T fragments straight from
//                the pages (values are stored transposed inside a page), each wavefront owning some (key/value head, 16
//                channels) tiles of the output
//   end          the sums go through LDS, are turned back by the query's position where values were turned by theirs,
//                and are written out
//
// Keys below a token's window may lie in pages the request has given back: they are read (finite values of whoever
// holds the page now) and weigh exactly 0.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 mxm_bf16x8;
typedef __attribute__((ext_vector_type(4))) float mxm_f32x4;

#define MXM_PAGES 2048         // page ids of a run's keys that are kept in LDS (the walk reads the table itself beyond them)
#define MXM_NW 8               // wavefronts of a workgroup
#define MXM_NT (64 * MXM_NW)
#define MXM_WROW 40            // bfloat16 a row of 32 weights takes in LDS (rows stay 16-byte aligned)

// A barrier for data that went through LDS: waits for this wavefront's LDS traffic only, so that loads from memory
// that were asked for ahead of their use stay in flight across it (the language's barrier waits for those as well).
__device__ __forceinline__ void mxm_lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
}

// cap * tanh(s / cap) with tanh(x) = 1 - 2 / (1 + exp(2 x)): float32, a handful of instructions
__device__ __forceinline__ float mxm_cap(float s, float cap, float inv_cap) {
    return cap > 0.f ? cap * (1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __expf(2.0f * s * inv_cap))) : s;
}

// mode 0: a workgroup walks all keys of its tokens and writes their outputs.  Modes 1 and 2 split a token's keys over
// `gridDim.y` workgroups (one token a workgroup): mode 1 leaves every head's (maximum, sum) over the split's keys in
// `stats` [tokens, splits, heads, 2]; mode 2 joins the splits' statistics itself (with the sink's share), forms the
// weights of its keys against the joined maximum and sum, and leaves its unnormed share of the output, which is simply a
// term of the sum over the splits, in `part` [tokens, splits, heads * vdim] (not yet turned back).
template <int STEPS, int ACC>
__global__ void __launch_bounds__(MXM_NT)
mixed_attention_mfma_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
                            const int* __restrict__ block_table, int max_blocks, const int* __restrict__ token_entry,
                            const int* __restrict__ positions, int n_tokens, int heads, int kv, int dim, int vdim,
                            int page_size, int window, float scale, float cap, float extra,
                            const float* __restrict__ talk, const float* __restrict__ v_freq, int v_pairing, int rp,
                            int tq, int mode, float* __restrict__ stats, float* __restrict__ part,
                            bf16* __restrict__ out) {
    constexpr int QROW = STEPS * 32 + 8;
    const int hp = (heads + 31) & ~31, trow = hp + 8;       // heads padded to the products' K, and a row of them in LDS
    extern __shared__ __attribute__((aligned(16))) char mxm_lds[];
    bf16* q_s = reinterpret_cast<bf16*>(mxm_lds);                                  // [kv][16][QROW]
    bf16* t_hi = q_s + (size_t)kv * 16 * QROW;                                     // [hp (to)][trow (from)]
    bf16* t_lo = t_hi + (size_t)hp * trow;
    bf16* p_hi = t_lo + (size_t)hp * trow;                                         // [tq * 32 (token, key)][trow (head)]
    bf16* p_lo = p_hi + (size_t)tq * 32 * trow;
    bf16* w_hi = p_lo + (size_t)tq * 32 * trow;                                    // [kv][16][WROW]
    bf16* w_lo = w_hi + (size_t)kv * 16 * MXM_WROW;
    float* ml = reinterpret_cast<float*>(w_lo + (size_t)kv * 16 * MXM_WROW);       // [kv][16][2]
    float* ml_half = ml + (size_t)kv * 32;                                         // [kv][2 (tile parity)][16][2]
    float* o_s = reinterpret_cast<float*>(mxm_lds);                                // [kv][16][vdim], over all of the above
    __shared__ int pages_s[MXM_PAGES];         // the run's pages from its first key's page on: one lookup a run, not one a load

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, col = lane & 15, quad = lane >> 4;
    const int group = heads / kv, dts = vdim >> 4;
    const int t0 = (int)blockIdx.x * tq;
    const int count = min(tq, n_tokens - t0);
    const int split = blockIdx.y, splits = gridDim.y;
    const float inv_cap = cap > 0.f ? 1.0f / cap : 0.f;
    const int my_u = col / rp, my_r = col % rp;          // the token and head-in-group of the slot this lane serves
    // pages of a power of two of tokens (the usual case) are found by a shift, others by a division
    const int page_shift = (page_size & (page_size - 1)) == 0 ? __ffs(page_size) - 1 : -1;
    auto page_index = [&](int key) { return page_shift >= 0 ? key >> page_shift : key / page_size; };
    auto page_offset = [&](int key) { return page_shift >= 0 ? key & (page_size - 1) : key % page_size; };

    for (int r0 = 0; r0 < count;) {
        const int entry = token_entry[t0 + r0];
        int r1 = r0 + 1;
        while (r1 < count && token_entry[t0 + r1] == entry) ++r1;
        const int* table = block_table + (int64_t)entry * max_blocks;
        const int p_first = positions[t0 + r0], p_last = positions[t0 + r1 - 1];
        const int k_lo = window > 0 ? max(0, p_first - window + 1) : 0;
        // this workgroup's keys: whole 32-key chunks (aligned to absolute positions) of k_lo .. p_last
        const int chunks = ((p_last - (k_lo & ~31)) >> 5) + 1, per = (chunks + splits - 1) / splits;
        const int kb0 = (k_lo & ~31) + split * per * 32;
        const int k_hi = min(p_last, kb0 + per * 32 - 1);
        const bool live = my_u >= r0 && my_u < r1 && my_r < group;
        const int my_pos = live ? positions[t0 + my_u] : -1;
        const int my_first = window > 0 ? max(0, my_pos - window + 1) : 0;

        const int page0 = page_index(kb0);
        for (int i = tid; i < MXM_PAGES && (int64_t)(page0 + i) * page_size <= p_last; i += MXM_NT) pages_s[i] = table[page0 + i];
        auto page_of = [&](int key) -> int64_t {
            const int at = page_index(key) - page0;
            return at < MXM_PAGES ? pages_s[at] : table[page0 + at];
        };
        // ---- into LDS (the end of a run writes over all of it): the mix in two bfloat16 halves, zeros where weights
        //      of dead slots and padded heads would stand, and the queries of the run's tokens, slot by slot
        for (int i = tid; i < hp * trow; i += MXM_NT) {
            const int h = i / trow, g = i % trow;
            float t = 0.f;
            if (h < heads && g < heads) t = talk != nullptr ? talk[h * heads + g] : (h == g ? 1.f : 0.f);
            const bf16 hi = (bf16)t;
            t_hi[i] = hi;
            t_lo[i] = (bf16)(t - (float)hi);
        }
        for (int i = tid; i < tq * 32 * trow; i += MXM_NT) p_hi[i] = p_lo[i] = (bf16)0.f;
        for (int i = tid; i < kv * 16 * MXM_WROW; i += MXM_NT) w_hi[i] = w_lo[i] = (bf16)0.f;
        for (int i = tid; i < kv * 16 * STEPS * 4; i += MXM_NT) {
            const int ch = (i % (STEPS * 4)) * 8, slot = (i / (STEPS * 4)) % 16, c = i / (STEPS * 4 * 16);
            const int u = slot / rp, r = slot % rp;
            mxm_bf16x8 v;
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = (__bf16)0.f;
            if (u >= r0 && u < r1 && r < group && ch < dim)
                v = *reinterpret_cast<const mxm_bf16x8*>(q + ((int64_t)(t0 + u) * heads + c * group + r) * dim + ch);
            *reinterpret_cast<mxm_bf16x8*>(q_s + ((size_t)c * 16 + slot) * QROW + ch) = v;
        }
        __syncthreads();

        // scores of 16 keys from kb on against the 16 slots of key/value head c: the lane's 4 keys of its slot
        // the K fragments of 16 keys from kb on of key/value head c (the lane's key row), as they are stored: nothing
        // touches them until the products that read them, so two tiles' loads are under way at once
        auto load_keys = [&](int c, int kb, mxm_bf16x8 (&kf)[STEPS]) {
            const int key_row = min(kb + col, p_last);
            const int64_t page = page_of(key_row);
            const bf16* krow = k_cache + ((page * kv + c) * page_size + page_offset(key_row)) * dim;
#pragma unroll
            for (int s = 0; s < STEPS; ++s) {
                const int ch = s * 32 + quad * 8;
#pragma unroll
                for (int e = 0; e < 8; ++e) kf[s][e] = (__bf16)0.f;
                if (ch < dim) kf[s] = *reinterpret_cast<const mxm_bf16x8*>(krow + ch);
            }
        };
        auto scores = [&](int c, int kb, const mxm_bf16x8 (&kf)[STEPS], float (&s4)[4]) {
            const bf16* q_lane = q_s + ((size_t)c * 16 + col) * QROW + quad * 8;
            mxm_f32x4 sc = mxm_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < STEPS; ++s)
                sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[s], *reinterpret_cast<const mxm_bf16x8*>(q_lane + s * 32), sc, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = kb + quad * 4 + i;
                s4[i] = live && key >= my_first && key <= my_pos && key <= k_hi ? mxm_cap(sc[i] * scale, cap, inv_cap) : -INFINITY;
            }
        };

        // ---- first walk: every slot's maximum and sum.  A unit of work is (key/value head, parity of the 16-key tile);
        //      the two parities' results are joined afterwards (mode 2: the splits' results are joined instead)
        if (mode != 2) {
            for (int unit = w; unit < kv * 2; unit += MXM_NW) {
                const int c = unit >> 1, parity = unit & 1;
                float m = -INFINITY, l = 0.f;
                // four tiles of this parity a round: all their fragments are asked for before the first is used
                for (int kb = kb0 + 16 * parity; kb <= k_hi; kb += 128) {
                    mxm_bf16x8 kf[4][STEPS];
#pragma unroll
                    for (int x = 0; x < 4; ++x) load_keys(c, kb + 32 * x, kf[x]);
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        float s4[4];
                        scores(c, kb + 32 * x, kf[x], s4);
                        const float mx = fmaxf(fmaxf(s4[0], s4[1]), fmaxf(s4[2], s4[3]));
                        const float m_new = fmaxf(m, mx);
                        if (m_new > -INFINITY) {
                            l = l * __expf(m - m_new) + ((__expf(s4[0] - m_new) + __expf(s4[1] - m_new)) +
                                                        (__expf(s4[2] - m_new) + __expf(s4[3] - m_new)));
                            m = m_new;
                        }
                    }
                }
                // the four lanes of a slot
                float top = fmaxf(m, __shfl_xor(m, 16, 64));
                top = fmaxf(top, __shfl_xor(top, 32, 64));
                float sum = top > -INFINITY ? l * __expf(m - top) : 0.f;
                sum += __shfl_xor(sum, 16, 64);
                sum += __shfl_xor(sum, 32, 64);
                if (quad == 0) {
                    ml_half[(unit * 16 + col) * 2] = top;
                    ml_half[(unit * 16 + col) * 2 + 1] = sum;
                }
            }
            __syncthreads();
        }
        // a thread a (key/value head, slot): the parities (or the splits) joined, then the sink's share
        for (int i = tid; i < kv * 16; i += MXM_NT) {
            const int c = i >> 4, slot = i & 15, u = slot / rp, r = slot % rp;
            const bool mine = u >= r0 && u < r1 && r < group;
            float m = -INFINITY, l = 0.f;
            auto join = [&](float m_s, float l_s) {
                const float m_new = fmaxf(m, m_s);
                if (m_new > -INFINITY) {
                    l = l * __expf(m - m_new) + l_s * __expf(m_s - m_new);
                    m = m_new;
                }
            };
            if (mode != 2) {
                join(ml_half[((c * 2) * 16 + slot) * 2], ml_half[((c * 2) * 16 + slot) * 2 + 1]);
                join(ml_half[((c * 2 + 1) * 16 + slot) * 2], ml_half[((c * 2 + 1) * 16 + slot) * 2 + 1]);
            } else if (mine) {
                const float* from = stats + (((int64_t)(t0 + u) * splits) * heads + c * group + r) * 2;
                for (int sp = 0; sp < splits; ++sp) join(from[(int64_t)sp * heads * 2], from[(int64_t)sp * heads * 2 + 1]);
            }
            if (mode == 1) {
                if (mine) {
                    float* to = stats + ((((int64_t)(t0 + u) * splits + split) * heads) + c * group + r) * 2;
                    to[0] = m;
                    to[1] = l;
                }
                continue;
            }
            if (extra > 0.f) join(0.f, extra);
            ml[i * 2] = m;
            ml[i * 2 + 1] = l;
        }
        if (mode == 1) {
            __syncthreads();
            r0 = r1;
            continue;
        }
        __syncthreads();

        // ---- second walk: the weights, their mix, the sum over the values
        mxm_f32x4 acc[ACC];
#pragma unroll
        for (int a = 0; a < ACC; ++a) acc[a] = mxm_f32x4{0.f, 0.f, 0.f, 0.f};
        // the K fragments of the wavefront's first unit are asked for a chunk ahead, a chunk's V^T fragments at its top:
        // both are under way while the chunk's weights go through LDS (whose barriers wait for LDS only)
        mxm_bf16x8 kf_ahead[STEPS];
        if (w < kv * 2 && kb0 <= k_hi) load_keys(w >> 1, kb0 + (w & 1) * 16, kf_ahead);
        for (int kb = kb0; kb <= k_hi; kb += 32) {
            mxm_bf16x8 vf[ACC];
            {
                // the lane's 8 keys lie in one page (pages hold a multiple of 8 tokens, the walk is aligned to 32)
                const int key8 = min(kb + quad * 8, p_last & ~7);
                const int64_t page = page_of(key8);
                const int off = page_offset(key8);
#pragma unroll
                for (int a = 0; a < ACC; ++a) {
                    const int pair = w + MXM_NW * a;
                    if (pair < kv * dts)
                        vf[a] = *reinterpret_cast<const mxm_bf16x8*>(
                            v_cache + (((page * kv + pair / dts) * vdim + (pair % dts) * 16 + col) * page_size + off));
                }
            }
            // the weights p = exp(s - m) / l, by (token, key) and head, in two bfloat16 halves
            for (int unit = w; unit < kv * 2; unit += MXM_NW) {
                const int c = unit >> 1, half = unit & 1;
                const float m = ml[(c * 16 + col) * 2], inv_l = live ? 1.0f / ml[(c * 16 + col) * 2 + 1] : 0.f;
                mxm_bf16x8 kf[STEPS];
                if (unit == w) {
#pragma unroll
                    for (int st = 0; st < STEPS; ++st) kf[st] = kf_ahead[st];
                } else {
                    load_keys(c, kb + half * 16, kf);
                }
                // every lane takes part in the scores (its key row is one of the tile's 16, whatever its slot is)
                {
                    float s4[4];
                    scores(c, kb + half * 16, kf, s4);
                    if (live) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const float pv = __expf(s4[i] - m) * inv_l;
                            const bf16 hi = (bf16)pv;
                            const size_t at = ((size_t)my_u * 32 + half * 16 + quad * 4 + i) * trow + c * group + my_r;
                            p_hi[at] = hi;
                            p_lo[at] = (bf16)(pv - (float)hi);
                        }
                    }
                }
            }
            if (w < kv * 2 && kb + 32 <= k_hi) load_keys(w >> 1, kb + 32 + (w & 1) * 16, kf_ahead);
            mxm_lds_barrier();
            // the mix: W^T [(token, key) x head] = P^T [(token, key) x head] T^T, tiles of 16 x 16 over the wavefronts
            {
                const int n_tiles = tq * 2, h_tiles = (heads + 15) >> 4;
                for (int tile = w; tile < n_tiles * h_tiles; tile += MXM_NW) {
                    const int nt = tile / h_tiles, ht = tile % h_tiles;
                    mxm_f32x4 mixed = mxm_f32x4{0.f, 0.f, 0.f, 0.f};
                    for (int ks = 0; ks < hp; ks += 32) {
                        const size_t pa = ((size_t)nt * 16 + col) * trow + ks + quad * 8;
                        const size_t ta = ((size_t)ht * 16 + col) * trow + ks + quad * 8;
                        const mxm_bf16x8 ph = *reinterpret_cast<const mxm_bf16x8*>(p_hi + pa);
                        const mxm_bf16x8 pl = *reinterpret_cast<const mxm_bf16x8*>(p_lo + pa);
                        const mxm_bf16x8 th = *reinterpret_cast<const mxm_bf16x8*>(t_hi + ta);
                        const mxm_bf16x8 tl = *reinterpret_cast<const mxm_bf16x8*>(t_lo + ta);
                        mixed = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ph, th, mixed, 0, 0, 0);
                        mixed = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pl, th, mixed, 0, 0, 0);
                        mixed = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ph, tl, mixed, 0, 0, 0);
                    }
                    // the lane holds head ht * 16 + col for the (token, key) pairs nt * 16 + quad * 4 + i
                    const int h = ht * 16 + col;
                    if (h < heads) {
                        const int u = nt >> 1, c = h / group, r = h % group;
                        const size_t at = ((size_t)c * 16 + u * rp + r) * MXM_WROW + (nt & 1) * 16 + quad * 4;
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const bf16 hi = (bf16)mixed[i];
                            w_hi[at + i] = hi;
                            w_lo[at + i] = (bf16)(mixed[i] - (float)hi);
                        }
                    }
                }
            }
            mxm_lds_barrier();
#pragma unroll
            for (int a = 0; a < ACC; ++a) {
                const int pair = w + MXM_NW * a;
                if (pair < kv * dts) {
                    const size_t at = ((size_t)(pair / dts) * 16 + col) * MXM_WROW + quad * 8;
                    acc[a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[a], *reinterpret_cast<const mxm_bf16x8*>(w_hi + at), acc[a], 0, 0, 0);
                    acc[a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[a], *reinterpret_cast<const mxm_bf16x8*>(w_lo + at), acc[a], 0, 0, 0);
                }
            }
        }
        // ---- the heads' outputs through LDS, turned back by the query's position (mode 2: the split's share as it is)
        __syncthreads();
#pragma unroll
        for (int a = 0; a < ACC; ++a) {
            const int pair = w + MXM_NW * a;
            if (pair < kv * dts) {
                const int c = pair / dts, dt = pair % dts;
#pragma unroll
                for (int i = 0; i < 4; ++i) o_s[((size_t)c * 16 + col) * vdim + dt * 16 + quad * 4 + i] = acc[a][i];
            }
        }
        __syncthreads();
        for (int i = tid; i < kv * 16 * vdim; i += MXM_NT) {
            const int d = i % vdim, slot = (i / vdim) % 16, c = i / (vdim * 16);
            const int u = slot / rp, r = slot % rp;
            if (u < r0 || u >= r1 || r >= group) continue;
            const float* row = o_s + ((size_t)c * 16 + slot) * vdim;
            float v = row[d];
            if (mode == 2) {
                part[(((int64_t)(t0 + u) * splits + split) * heads + c * group + r) * vdim + d] = v;
                continue;
            }
            if (v_freq != nullptr) {
                const int half = vdim >> 1;
                const bool first = v_pairing == 0 ? d < half : (d & 1) == 0;
                const int pair = v_pairing == 0 ? (first ? d : d - half) : d >> 1;
                const float other = row[v_pairing == 0 ? (first ? d + half : d - half) : (d ^ 1)];
                const float angle = (float)positions[t0 + u] * v_freq[pair];
                const float cs = cosf(angle), sn = sinf(angle);            // by -angle: the sine changes its sign
                v = first ? v * cs + other * sn : v * cs - other * sn;
            }
            out[((int64_t)(t0 + u) * heads + c * group + r) * vdim + d] = (bf16)v;
        }
        __syncthreads();
        r0 = r1;
    }
}

// out[t, h, :] = the sum of the splits' shares, turned back by the token's position.  A thread per (token, head, channel).
__global__ void __launch_bounds__(256)
mixed_attention_join_kernel(const float* __restrict__ part, int splits, int heads, int vdim, const int* __restrict__ positions,
                            const float* __restrict__ v_freq, int v_pairing, bf16* __restrict__ out, int64_t count) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    const int d = (int)(i % vdim);
    const int64_t th = i / vdim;
    const int h = (int)(th % heads);
    const int64_t t = th / heads;
    const float* mine = part + ((t * splits) * heads + h) * vdim;
    auto total = [&](int ch) {
        float sum = 0.f;
        for (int s = 0; s < splits; ++s) sum += mine[(int64_t)s * heads * vdim + ch];
        return sum;
    };
    float v = total(d);
    if (v_freq != nullptr) {
        const int half = vdim >> 1;
        const bool first = v_pairing == 0 ? d < half : (d & 1) == 0;
        const int pair = v_pairing == 0 ? (first ? d : d - half) : d >> 1;
        const float other = total(v_pairing == 0 ? (first ? d + half : d - half) : (d ^ 1));
        const float angle = (float)positions[t] * v_freq[pair];
        const float cs = cosf(angle), sn = sinf(angle);
        v = first ? v * cs + other * sn : v * cs - other * sn;
    }
    out[i] = (bf16)v;
}

static size_t mxm_lds_bytes(int steps, int heads, int kv, int vdim, int tq) {
    const size_t hp = (size_t)((heads + 31) & ~31), trow = hp + 8;
    const size_t walk = (size_t)kv * 16 * (steps * 32 + 8) * 2 + 2 * hp * trow * 2 + 2 * (size_t)tq * 32 * trow * 2 +
                        2 * (size_t)kv * 16 * MXM_WROW * 2 + (size_t)kv * 32 * 4 + (size_t)kv * 64 * 4;
    const size_t end = (size_t)kv * 16 * vdim * 4;
    return walk > end ? walk : end;
}

static int mxm_steps(int dim) { return dim <= 32 ? 1 : dim <= 64 ? 2 : dim <= 128 ? 4 : 8; }
static int mxm_acc(int kv, int vdim) {
    const int need = ceil_div(kv * (vdim / 16), MXM_NW);
    return need <= 1 ? 1 : need <= 2 ? 2 : need <= 4 ? 4 : 8;
}

extern "C" int somi_mixed_attention_mfma_supported(int heads, int kv, int dim, int vdim, int page_size) {
    if (heads <= 0 || kv <= 0 || heads % kv || heads / kv > 16 || dim <= 0 || dim % 8 || dim > 256 || vdim <= 0 ||
        vdim % 16 || page_size <= 0 || page_size % 8)
        return 0;
    if (ceil_div(kv * (vdim / 16), MXM_NW) > 8) return 0;
    int rp = 1;
    while (rp < heads / kv) rp <<= 1;
    return mxm_lds_bytes(mxm_steps(dim), heads, kv, vdim, 16 / rp) <= 160 * 1024 ? 1 : 0;
}

// As somi_mixed_attention_plain, bfloat16 only.  portions != 0: the step holds prompt portions, and as many consecutive
// tokens share a workgroup as their heads fill 16 query slots a key/value head; otherwise a workgroup serves one token,
// and with splits > 1 a token's keys are dealt out to that many workgroups (three launches: the splits' statistics,
// their shares of the output, the join; group_tokens must be 0 then), for which `stats` holds n_tokens * splits * heads * 2 floats and `part`
// n_tokens * splits * heads * vdim.
extern "C" int somi_mixed_attention_mfma(const void* q, const void* k_cache, const void* v_cache, const int* block_table,
                                         int max_blocks, const int* token_entry, const int* positions, int n_tokens,
                                         int heads, int kv, int dim, int vdim, int page_size, int window, float scale,
                                         float cap, float extra, const float* talk, const float* v_freq, int v_pairing,
                                         int portions, int splits, float* stats, float* part, void* out,
                                         int group_tokens, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && max_blocks > 0 && window >= 0 && splits >= 1 && splits <= 65535, "mixed_attention_mfma: bad sizes");
    SOMI_REQUIRE(somi_mixed_attention_mfma_supported(heads, kv, dim, vdim, page_size),
                 "mixed_attention_mfma: %d heads over %d of %d + %d channels in pages of %d are not what the kernel is built for",
                 heads, kv, dim, vdim, page_size);
    SOMI_REQUIRE(extra == 0.f || extra == 1.f, "mixed_attention_mfma: the denominator takes 0 or 1 more, got %g", (double)extra);
    SOMI_REQUIRE(v_pairing == 0 || v_pairing == 1, "mixed_attention_mfma: unknown pairing");
    SOMI_REQUIRE(splits == 1 || (!portions && stats != nullptr && part != nullptr),
                 "mixed_attention_mfma: key splits are for steps of single tokens and need their workspaces");
    if (n_tokens == 0) return 0;
    const int group = heads / kv;
    int rp = 1;
    while (rp < group) rp <<= 1;
    // tokens a workgroup: at most what fills the 16 slots; fewer tokens make more workgroups, whose waits for memory
    // overlap (group_tokens: the caller's choice, 0 = the default)
    int tq = portions ? 16 / rp : 1;
    if (portions && group_tokens > 0 && group_tokens < tq) tq = group_tokens;
    const int steps = mxm_steps(dim), accs = mxm_acc(kv, vdim);
    const size_t lds = mxm_lds_bytes(steps, heads, kv, vdim, tq);
#define MXM_LAUNCH(STEPS, ACC, MODE, GRID)                                                                              \
    do {                                                                                                                \
        hipError_t err = hipFuncSetAttribute((const void*)mixed_attention_mfma_kernel<STEPS, ACC>,                      \
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                     \
        if (err != hipSuccess) return somi_fail("mixed_attention_mfma: %s", hipGetErrorString(err));                    \
        hipLaunchKernelGGL((mixed_attention_mfma_kernel<STEPS, ACC>), GRID, dim3(MXM_NT), lds, stream, (const bf16*)q,  \
                           (const bf16*)k_cache, (const bf16*)v_cache, block_table, max_blocks, token_entry, positions, \
                           n_tokens, heads, kv, dim, vdim, page_size, window, scale, cap, extra, talk, v_freq,          \
                           v_pairing, rp, tq, MODE, stats, part, (bf16*)out);                                           \
    } while (0)
#define MXM_BY_ACC(STEPS, MODE, GRID)                            \
    do {                                                         \
        if (accs == 1) MXM_LAUNCH(STEPS, 1, MODE, GRID);         \
        else if (accs == 2) MXM_LAUNCH(STEPS, 2, MODE, GRID);    \
        else if (accs == 4) MXM_LAUNCH(STEPS, 4, MODE, GRID);    \
        else MXM_LAUNCH(STEPS, 8, MODE, GRID);                   \
    } while (0)
#define MXM_BY_STEPS(MODE, GRID)                         \
    do {                                                 \
        if (steps == 1) MXM_BY_ACC(1, MODE, GRID);       \
        else if (steps == 2) MXM_BY_ACC(2, MODE, GRID);  \
        else if (steps == 4) MXM_BY_ACC(4, MODE, GRID);  \
        else MXM_BY_ACC(8, MODE, GRID);                  \
    } while (0)
    if (splits == 1) {
        const dim3 grid(ceil_div(n_tokens, tq));
        MXM_BY_STEPS(0, grid);
        SOMI_LAUNCH_CHECK("mixed_attention_mfma");
        return 0;
    }
    const dim3 grid(n_tokens, splits);
    MXM_BY_STEPS(1, grid);
    SOMI_LAUNCH_CHECK("mixed_attention_mfma (statistics)");
    MXM_BY_STEPS(2, grid);
    SOMI_LAUNCH_CHECK("mixed_attention_mfma (shares)");
    const int64_t count = (int64_t)n_tokens * heads * vdim;
    hipLaunchKernelGGL(mixed_attention_join_kernel, dim3((unsigned)ceil_div64(count, 256)), dim3(256), 0, stream, part, splits,
                       heads, vdim, positions, v_freq, v_pairing, (bf16*)out, count);
    SOMI_LAUNCH_CHECK("mixed_attention_join");
#undef MXM_BY_STEPS
#undef MXM_BY_ACC
#undef MXM_LAUNCH
    return 0;
}
