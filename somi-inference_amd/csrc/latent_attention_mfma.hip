// Attention over kept latents on the matrix cores (bfloat16).
//
// Every past token keeps one row [c (rank) | r (rot)] for all heads, and the same c once more transposed inside its
// page (pages of a power of two of tokens; [pages, rank, page]: consecutive positions of one channel are adjacent, the operand layout of the
// weights-times-values product).  A workgroup serves ONE token and up to 16 of its heads (its query slots), which all
// see the same keys, over one part of the token's keys (a key split); its four wavefronts walk 64-key tiles:
//
//   scores   wavefront w owns keys 16 w .. 16 w + 15 of the tile: S^T = K Q^T by `16x16x32` products over the rank + rot
//            channels, K fragments straight from the rows (16 bytes a lane), the slots' Q fragments from LDS, where they
//            stay for the whole walk; a lane then holds 4 keys of one slot
//   softmax  float32, online: the running maximum of a slot starts at the head's sink and its running sum at 1 (the
//            sink's own term, in the first key split only), the tile's maximum is exchanged through LDS
//   values   the weights go to LDS as two bfloat16 halves (p = hi + lo, so no weight is rounded to eight bits) and
//            come back as B operands; wavefront w owns the channel tiles w, w + 4, ... of the output, O^T = C^T P^T with
//            the C^T fragments straight from the transposed pages
//
// The loads run ahead of their use: a tile's transposed latents are asked for a whole tile earlier (two sets of
// registers), the next tile's K fragments as soon as this tile's score products have read the registers they go to.
// A token's key splits leave (maximum, sum, unnormed output) in a workspace and a second kernel joins them.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 lam_bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 lam_bf16x4;
typedef __attribute__((ext_vector_type(4))) float lam_f32x4;

#define LAM_KEYS 64

// A barrier for data that went through LDS: waits for this wavefront's LDS traffic only, so that loads from memory
// that were asked for ahead of their use stay in flight across it (the language's barrier waits for those as well).
__device__ __forceinline__ void lam_lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
}

template <int STEPS, int CT>
__global__ void __launch_bounds__(256)
latent_attention_mfma_kernel(const bf16* __restrict__ queries, const bf16* __restrict__ latent,
                             const bf16* __restrict__ latent_t, const int* __restrict__ block_table, int max_blocks,
                             const int* __restrict__ token_entry, const int* __restrict__ positions, int n_tokens,
                             int heads, int rank, int D, int page_shift, int window, float scale,
                             const float* __restrict__ sink, int splits, bf16* __restrict__ out, float* __restrict__ part) {
    const int page_mask = (1 << page_shift) - 1;
    __shared__ float wmax[4][16];
    __shared__ float wsum[4][16];
    __shared__ __attribute__((aligned(16))) bf16 p_hi[16][LAM_KEYS + 8];
    __shared__ __attribute__((aligned(16))) bf16 p_lo[16][LAM_KEYS + 8];
    __shared__ __attribute__((aligned(16))) bf16 q_s[16][STEPS * 32 + 8];
    const int t = n_tokens - 1 - (int)blockIdx.x;               // the longest walks first
    const int hg = blockIdx.y, split = blockIdx.z;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const int head = hg * 16 + col;
    const bool live = head < heads;
    const int p = positions[t];
    const int* table = block_table + (int64_t)token_entry[t] * max_blocks;
    const int steps = (D + 31) >> 5, tiles_c = rank >> 4;
    // this split's keys: whole 64-key tiles (aligned to absolute positions) of the keys lo .. p that the token sees
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const int first_tile = lo / LAM_KEYS;
    const int tiles_all = (p + LAM_KEYS) / LAM_KEYS - first_tile;
    const int per = (tiles_all + splits - 1) / splits;
    const int k_begin = (first_tile + split * per) * LAM_KEYS;
    const int k_end = min(p + 1, (first_tile + (split + 1) * per) * LAM_KEYS);

    // the slots' queries go to LDS once (rows padded by 16 bytes, so that the 16 rows of a fragment fall on different
    // banks): held in registers they would leave no room for loads that run ahead
    for (int i = threadIdx.x; i < 16 * STEPS * 4; i += 256) {
        const int slot = i / (STEPS * 4), ch = (i % (STEPS * 4)) * 8;
        lam_bf16x8 v;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (__bf16)0.f;
        if (hg * 16 + slot < heads && ch < D)
            v = *reinterpret_cast<const lam_bf16x8*>(queries + ((int64_t)t * heads + hg * 16 + slot) * D + ch);
        *reinterpret_cast<lam_bf16x8*>(&q_s[slot][ch]) = v;
    }
    __syncthreads();
    lam_f32x4 acc[CT];
#pragma unroll
    for (int j = 0; j < CT; ++j) acc[j] = lam_f32x4{0.f, 0.f, 0.f, 0.f};
    // without a sink the first tile, which holds a key that is seen, sets the maximum
    float m = split == 0 ? (live ? (sink != nullptr ? sink[head] : -INFINITY) : 0.f) : -INFINITY;
    float lsum = (split == 0 && sink != nullptr && w == 0 && quad == 0) ? 1.f : 0.f;

    // A tile's K fragments (this wavefront's 16 keys) and the transposed latents of the channel tiles it owns, as they
    // are stored: nothing touches them until the products that read them.
    auto load_keys = [&](int kb, lam_bf16x8 (&kf)[STEPS]) {
        const int key_row = min(kb + 16 * w + col, p);
        const bf16* krow = latent + ((((int64_t)table[key_row >> page_shift]) << page_shift) + (key_row & page_mask)) * D;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const int ch = s * 32 + quad * 8;
            if (s < steps && ch < D) kf[s] = *reinterpret_cast<const lam_bf16x8*>(krow + ch);
        }
    };
    auto load_values = [&](int kb, lam_bf16x8 (&vf)[CT][2]) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            // the lane's 8 keys lie in one page: its channel rows there, one page lookup for all channel tiles
            const int key8 = min(kb + half * 32 + quad * 8, p & ~7);
            const bf16* rows = latent_t + ((((int64_t)table[key8 >> page_shift] * rank + col) << page_shift) + (key8 & page_mask));
#pragma unroll
            for (int j = 0; j < CT; ++j) {
                const int ct = w + 4 * j;
                if (ct < tiles_c) vf[j][half] = *reinterpret_cast<const lam_bf16x8*>(rows + ((int64_t)(ct * 16) << page_shift));
            }
        }
    };
    // One tile: the next tile's transposed latents are asked for first (they are used a whole tile later), the next
    // tile's K fragments right after this tile's score products have read the registers they go to.
    auto tile = [&](int kb, lam_bf16x8 (&kf)[STEPS], lam_bf16x8 (&vf)[CT][2], lam_bf16x8 (&vnext)[CT][2]) {
        const bool more = kb + LAM_KEYS < k_end;
        if (more) load_values(kb + LAM_KEYS, vnext);
        lam_f32x4 sc = lam_f32x4{0.f, 0.f, 0.f, 0.f};
        int q_at = col * (STEPS * 32 + 8) + quad * 8;        // opaque once a tile: the Q fragments are read at every use
        asm volatile("" : "+v"(q_at));
        const bf16* q_lane = &q_s[0][0] + q_at;
#pragma unroll
        for (int s = 0; s < STEPS; ++s)
            if (s < steps)
                sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[s], *reinterpret_cast<const lam_bf16x8*>(q_lane + s * 32), sc, 0, 0, 0);
        if (more) load_keys(kb + LAM_KEYS, kf);
        // ---- softmax over the tile, float32
        float s4[4], mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = kb + 16 * w + quad * 4 + i;
            s4[i] = key >= lo && key < k_end ? sc[i] * scale : -INFINITY;
            mx = fmaxf(mx, s4[i]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        if (quad == 0) wmax[w][col] = mx;
        lam_lds_barrier();
        const float m_new = fmaxf(fmaxf(m, fmaxf(wmax[0][col], wmax[1][col])), fmaxf(wmax[2][col], wmax[3][col]));
        const float m_ref = m_new == -INFINITY ? 0.f : m_new;   // nothing seen yet: every weight below is exp(-inf) = 0
        const float corr = __expf(m - m_ref);
        m = m_new;
        float psum = 0.f;
        lam_bf16x4 hi, low;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float pv = __expf(s4[i] - m_ref);              // exp(-inf) = 0 for keys that are not seen
            psum += pv;
            hi[i] = (__bf16)pv;
            low[i] = (__bf16)(pv - (float)hi[i]);
        }
        lsum = lsum * corr + psum;
        *reinterpret_cast<lam_bf16x4*>(&p_hi[col][16 * w + quad * 4]) = hi;
        *reinterpret_cast<lam_bf16x4*>(&p_lo[col][16 * w + quad * 4]) = low;
        if (__any(corr != 1.0f)) {                               // only where some slot's maximum moved
#pragma unroll
            for (int j = 0; j < CT; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[j][i] *= corr;
        }
        lam_lds_barrier();
        // ---- weights times latents
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const lam_bf16x8 ph = *reinterpret_cast<const lam_bf16x8*>(&p_hi[col][half * 32 + quad * 8]);
            const lam_bf16x8 pl = *reinterpret_cast<const lam_bf16x8*>(&p_lo[col][half * 32 + quad * 8]);
#pragma unroll
            for (int j = 0; j < CT; ++j)
                if (w + 4 * j < tiles_c) {
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[j][half], ph, acc[j], 0, 0, 0);
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[j][half], pl, acc[j], 0, 0, 0);
                }
        }
    };
    lam_bf16x8 kf[STEPS], va[CT][2], vb[CT][2];
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
#pragma unroll
        for (int i = 0; i < 8; ++i) kf[s][i] = (__bf16)0.f;        // the half step past the row's end stays zero
#pragma unroll
    for (int j = 0; j < CT; ++j)
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int i = 0; i < 8; ++i) va[j][half][i] = vb[j][half][i] = (__bf16)0.f;
    if (k_begin < k_end) {
        load_keys(k_begin, kf);
        load_values(k_begin, va);
    }
    for (int kb = k_begin; kb < k_end; kb += 2 * LAM_KEYS) {
        tile(kb, kf, va, vb);
        if (kb + LAM_KEYS < k_end) tile(kb + LAM_KEYS, kf, vb, va);
    }
    // ---- the slots' sums: the lane groups of a wavefront, then the wavefronts
    lsum += __shfl_xor(lsum, 16, 64);
    lsum += __shfl_xor(lsum, 32, 64);
    __syncthreads();
    if (quad == 0) wsum[w][col] = lsum;
    __syncthreads();
    const float l = (wsum[0][col] + wsum[1][col]) + (wsum[2][col] + wsum[3][col]);
    if (!live) return;
    if (splits == 1) {
        const float inv = 1.0f / l;
#pragma unroll
        for (int j = 0; j < CT; ++j) {
            const int ct = w + 4 * j;
            if (ct >= tiles_c) continue;
            lam_bf16x4 o;
#pragma unroll
            for (int i = 0; i < 4; ++i) o[i] = (__bf16)(acc[j][i] * inv);
            *reinterpret_cast<lam_bf16x4*>(out + ((int64_t)t * heads + head) * rank + ct * 16 + quad * 4) = o;
        }
        return;
    }
    float* mine = part + (((int64_t)t * heads + head) * splits + split) * (rank + 2);
#pragma unroll
    for (int j = 0; j < CT; ++j) {
        const int ct = w + 4 * j;
        if (ct >= tiles_c) continue;
        *reinterpret_cast<lam_f32x4*>(mine + ct * 16 + quad * 4) = acc[j];
    }
    if (w == 0 && quad == 0) {
        mine[rank] = m;
        mine[rank + 1] = l;
    }
}

// The same for prompt portions: a workgroup serves TT consecutive tokens of the step (and up to 16 heads of each:
// 16 TT query slots), so that a tile of kept rows is read once for all of them.  Tokens of one request stand side
// by side with rising positions; where a group of tokens holds several requests (a portion's end beside the next
// entry) the workgroup takes them run by run.  A wavefront again owns 16 keys of a tile for the scores (one K fragment
// against the TT tokens' Q fragments from LDS) and a quarter of the channel tiles for the output (every token's).
// The transposed latents of a tile are asked for before its scores, the next tile's K fragments after them.
// TT: tokens of a workgroup; PW: its wavefronts (a tile is 16 PW keys); WPS: wavefronts a SIMD is to hold (2 = two
// workgroups of four wavefronts a compute unit, so that one's softmax runs under the other's matrix instructions).

template <int STEPS, int CT, int TT, int PW, int WPS>
__global__ void __launch_bounds__(64 * PW, WPS)
latent_attention_portion_kernel(const bf16* __restrict__ queries, const bf16* __restrict__ latent,
                                const bf16* __restrict__ latent_t, const int* __restrict__ block_table, int max_blocks,
                                const int* __restrict__ token_entry, const int* __restrict__ positions, int n_tokens,
                                int heads, int rank, int D, int page_shift, int window, float scale,
                                const float* __restrict__ sink, bf16* __restrict__ out) {
    const int page_mask = (1 << page_shift) - 1;
    constexpr int VH = CT >= 8 ? 1 : 2;          // 32-key steps whose transposed latents are in registers at a time
    constexpr int SLOTS = 16 * TT, QROW = STEPS * 32 + 8, PROW = (16 * PW) + 8, NT = 64 * PW;
    extern __shared__ __attribute__((aligned(16))) char lam_lds[];
    bf16 (*q_s)[QROW] = reinterpret_cast<bf16 (*)[QROW]>(lam_lds);
    bf16 (*p_hi)[PROW] = reinterpret_cast<bf16 (*)[PROW]>(lam_lds + (size_t)SLOTS * QROW * 2);
    bf16 (*p_lo)[PROW] = reinterpret_cast<bf16 (*)[PROW]>(lam_lds + (size_t)SLOTS * QROW * 2 + (size_t)SLOTS * PROW * 2);
    float (*wmax)[SLOTS] = reinterpret_cast<float (*)[SLOTS]>(lam_lds + (size_t)SLOTS * QROW * 2 + (size_t)SLOTS * PROW * 4);
    const int groups = (n_tokens + TT - 1) / TT;
    const int t0 = (groups - 1 - (int)blockIdx.x) * TT;      // the longest walks first
    const int count = min(TT, n_tokens - t0);
    const int hg = blockIdx.y;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const int head = hg * 16 + col;
    const int steps = (D + 31) >> 5, tiles_c = rank >> 4;

    for (int r0 = 0; r0 < count;) {
        const int entry = token_entry[t0 + r0];
        int r1 = r0 + 1;
        while (r1 < count && token_entry[t0 + r1] == entry) ++r1;
        const int* table = block_table + (int64_t)entry * max_blocks;
        const int p_last = positions[t0 + r1 - 1];
        int pos[TT], first[TT];              // a token sees the keys first[u] .. pos[u]
        bool live[TT];
#pragma unroll
        for (int u = 0; u < TT; ++u) {
            live[u] = u >= r0 && u < r1;
            pos[u] = live[u] ? positions[t0 + u] : -1;
            first[u] = window > 0 ? max(0, pos[u] - window + 1) : 0;
        }
        // the walk starts at the tile (aligned to absolute positions) of the first key the run's first token sees
        const int p_first = positions[t0 + r0];
        const int kb0 = ((window > 0 ? max(0, p_first - window + 1) : 0) / (16 * PW)) * (16 * PW);
        for (int i = threadIdx.x; i < SLOTS * STEPS * 4; i += NT) {
            const int slot = i / (STEPS * 4), ch = (i % (STEPS * 4)) * 8;
            const int u = slot >> 4, h = hg * 16 + (slot & 15);
            lam_bf16x8 v;
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = (__bf16)0.f;
            if (u >= r0 && u < r1 && h < heads && ch < D)
                v = *reinterpret_cast<const lam_bf16x8*>(queries + ((int64_t)(t0 + u) * heads + h) * D + ch);
            *reinterpret_cast<lam_bf16x8*>(&q_s[slot][ch]) = v;
        }
        __syncthreads();
        lam_f32x4 acc[TT][CT];
        float m[TT], lsum[TT];
#pragma unroll
        for (int u = 0; u < TT; ++u) {
#pragma unroll
            for (int j = 0; j < CT; ++j) acc[u][j] = lam_f32x4{0.f, 0.f, 0.f, 0.f};
            m[u] = live[u] && head < heads ? (sink != nullptr ? sink[head] : -INFINITY) : 0.f;
            lsum[u] = (live[u] && sink != nullptr && w == 0 && quad == 0) ? 1.f : 0.f;
        }
        lam_bf16x8 kf[STEPS], vf[CT][VH];
#pragma unroll
        for (int s = 0; s < STEPS; ++s)
#pragma unroll
            for (int i = 0; i < 8; ++i) kf[s][i] = (__bf16)0.f;        // the half step past the row's end stays zero
        auto load_keys = [&](int kb) {
            const int key_row = min(kb + 16 * w + col, p_last);
            const bf16* krow = latent + ((((int64_t)table[key_row >> page_shift]) << page_shift) + (key_row & page_mask)) * D;
#pragma unroll
            for (int s = 0; s < STEPS; ++s) {
                const int ch = s * 32 + quad * 8;
                if (s < steps && ch < D) kf[s] = *reinterpret_cast<const lam_bf16x8*>(krow + ch);
            }
        };
        // the transposed latents of VH 32-key steps of a tile at a time (a tile has PW / 2 of them)
        auto load_values = [&](int kb, int pair) {
#pragma unroll
            for (int half = 0; half < VH; ++half) {
                // the lane's 8 keys lie in one page: its channel rows there, one page lookup for all channel tiles
                const int key8 = min(kb + (VH * pair + half) * 32 + quad * 8, p_last & ~7);
                const bf16* rows = latent_t + ((((int64_t)table[key8 >> page_shift] * rank + col) << page_shift) + (key8 & page_mask));
#pragma unroll
                for (int j = 0; j < CT; ++j) {
                    const int ct = w + PW * j;
                    if (ct < tiles_c) vf[j][half] = *reinterpret_cast<const lam_bf16x8*>(rows + ((int64_t)(ct * 16) << page_shift));
                }
            }
        };
        load_keys(kb0);
        for (int kb = kb0; kb <= p_last; kb += (16 * PW)) {
            load_values(kb, 0);
            lam_f32x4 sc[TT];
#pragma unroll
            for (int u = 0; u < TT; ++u) sc[u] = lam_f32x4{0.f, 0.f, 0.f, 0.f};
            // the offset of the lane's Q fragments is made opaque once a tile: the fragments are read from LDS at every
            // use instead of being kept in registers across the walk, which they would fill
            int q_at = col * QROW + quad * 8;
            asm volatile("" : "+v"(q_at));
            const bf16* q_lane = &q_s[0][0] + q_at;
#pragma unroll
            for (int s = 0; s < STEPS; ++s)
                if (s < steps) {
#pragma unroll
                    for (int u = 0; u < TT; ++u)
                        if (live[u])
                            sc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                                kf[s], *reinterpret_cast<const lam_bf16x8*>(q_lane + u * 16 * QROW + s * 32), sc[u], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);       // a step's Q fragments are read when the step comes, not ahead
                }
            if (kb + (16 * PW) <= p_last) load_keys(kb + (16 * PW));
            // ---- softmax over the tile, float32, slot by slot
            float s4[TT][4];
#pragma unroll
            for (int u = 0; u < TT; ++u) {
                float mx = -INFINITY;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = kb + 16 * w + quad * 4 + i;
                    s4[u][i] = key <= pos[u] && key >= first[u] ? sc[u][i] * scale : -INFINITY;
                    mx = fmaxf(mx, s4[u][i]);
                }
                mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
                mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
                if (quad == 0) wmax[w][u * 16 + col] = mx;
            }
            lam_lds_barrier();
#pragma unroll
            for (int u = 0; u < TT; ++u) {
                const int slot = u * 16 + col;
                float m_new = m[u];
#pragma unroll
                for (int x = 0; x < PW; ++x) m_new = fmaxf(m_new, wmax[x][slot]);
                const float m_ref = m_new == -INFINITY ? 0.f : m_new;    // nothing seen yet: the weights below are 0
                const float corr = __expf(m[u] - m_ref);
                m[u] = m_new;
                float psum = 0.f;
                lam_bf16x4 hi, lo;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float pv = __expf(s4[u][i] - m_ref);          // exp(-inf) = 0 for keys that are not seen
                    psum += pv;
                    hi[i] = (__bf16)pv;
                    lo[i] = (__bf16)(pv - (float)hi[i]);
                }
                lsum[u] = lsum[u] * corr + psum;
                *reinterpret_cast<lam_bf16x4*>(&p_hi[slot][16 * w + quad * 4]) = hi;
                *reinterpret_cast<lam_bf16x4*>(&p_lo[slot][16 * w + quad * 4]) = lo;
#pragma unroll
                for (int j = 0; j < CT; ++j)
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[u][j][i] *= corr;
            }
            lam_lds_barrier();
            // ---- weights times latents, VH 32-key steps at a time; the next are asked for as soon as these have
            //      been read
#pragma unroll
            for (int pair = 0; pair < PW / 2 / VH; ++pair) {
#pragma unroll
                for (int half = 0; half < VH; ++half)
#pragma unroll
                    for (int u = 0; u < TT; ++u) {
                        if (!live[u]) continue;
                        const int at = (VH * pair + half) * 32 + quad * 8;
                        const lam_bf16x8 ph = *reinterpret_cast<const lam_bf16x8*>(&p_hi[u * 16 + col][at]);
                        const lam_bf16x8 pl = *reinterpret_cast<const lam_bf16x8*>(&p_lo[u * 16 + col][at]);
#pragma unroll
                        for (int j = 0; j < CT; ++j)
                            if (w + PW * j < tiles_c) {
                                acc[u][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[j][half], ph, acc[u][j], 0, 0, 0);
                                acc[u][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[j][half], pl, acc[u][j], 0, 0, 0);
                            }
                    }
                if (pair + 1 < PW / 2 / VH) load_values(kb, pair + 1);
            }
        }
        // ---- the slots' sums (the lane groups of a wavefront, then the wavefronts; wmax is free again) and the output
        __syncthreads();
#pragma unroll
        for (int u = 0; u < TT; ++u) {
            float v = lsum[u];
            v += __shfl_xor(v, 16, 64);
            v += __shfl_xor(v, 32, 64);
            if (quad == 0) wmax[w][u * 16 + col] = v;
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < TT; ++u) {
            if (!live[u] || head >= heads) continue;
            const int slot = u * 16 + col;
            float total = 0.f;
#pragma unroll
            for (int x = 0; x < PW; ++x) total += wmax[x][slot];
            const float inv = 1.0f / total;
#pragma unroll
            for (int j = 0; j < CT; ++j) {
                const int ct = w + PW * j;
                if (ct >= tiles_c) continue;
                lam_bf16x4 o;
#pragma unroll
                for (int i = 0; i < 4; ++i) o[i] = (__bf16)(acc[u][j][i] * inv);
                *reinterpret_cast<lam_bf16x4*>(out + ((int64_t)(t0 + u) * heads + head) * rank + ct * 16 + quad * 4) = o;
            }
        }
        __syncthreads();
        r0 = r1;
    }
}

// out[t, h, :] = sum_s exp(m_s - M) O_s / sum_s exp(m_s - M) l_s over a token's key splits (a split without keys has
// m = -inf and weighs nothing).  One workgroup per (token, head): the splits' weights go to LDS first, then a thread sums
// its channels over the splits, neighbouring threads reading neighbouring channels.
#define LAM_MAX_SPLITS 64
__global__ void __launch_bounds__(128)
latent_attention_join_kernel(const float* __restrict__ part, int splits, int rank, bf16* __restrict__ out) {
    __shared__ float weight[LAM_MAX_SPLITS];
    __shared__ float red[16];
    const int64_t slot = blockIdx.x;
    const float* mine = part + slot * splits * (rank + 2);
    const int s_mine = threadIdx.x;
    const float m_s = s_mine < splits ? mine[s_mine * (rank + 2) + rank] : -INFINITY;
    const float l_s = s_mine < splits ? mine[s_mine * (rank + 2) + rank + 1] : 0.f;
    const float top = block_max<128>(m_s, red);
    const float e = __expf(m_s - top);
    const float total = block_sum<128>(e * l_s, red);
    if (s_mine < splits) weight[s_mine] = e / total;
    __syncthreads();
    for (int c = threadIdx.x; c < rank; c += 128) {
        float sum = 0.f;
#pragma unroll 8
        for (int s = 0; s < splits; ++s) sum = fmaf(weight[s], mine[s * (rank + 2) + c], sum);
        out[slot * rank + c] = (bf16)sum;
    }
}

extern "C" int somi_latent_attention_mfma_supported(int rank, int rot, int page_size) {
    const int D = rank + rot;
    return rank > 0 && rank % 16 == 0 && D % 16 == 0 && D <= 576 && rank <= 512 && page_size >= 8
           && (page_size & (page_size - 1)) == 0;
}

// queries: [n_tokens, heads, rank + rot] bfloat16; latent: [pages, page, rank + rot]; latent_t: [pages, rank, page];
// block_table: [entries, max_blocks]; sink: [heads] float32 or null for a softmax over the keys alone; window: the keys
// a token sees, itself included (0: all); out: [n_tokens, heads, rank] bfloat16; part: a workspace of n_tokens * heads *
// splits * (rank + 2) floats where splits > 1.
extern "C" int somi_latent_attention_mfma(const void* queries, const void* latent, const void* latent_t,
                                          const int* block_table, int max_blocks, const int* token_entry,
                                          const int* positions, int n_tokens, int heads, int rank, int rot, int page_size,
                                          int window, float scale, const float* sink, int splits, int portions, void* out,
                                          float* part, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && heads > 0 && max_blocks > 0 && splits >= 1 && window >= 0, "latent_attention_mfma: bad sizes");
    SOMI_REQUIRE(somi_latent_attention_mfma_supported(rank, rot, page_size),
                 "latent_attention_mfma: a latent of %d + %d in pages of %d is not what the kernel is built for", rank, rot,
                 page_size);
    SOMI_REQUIRE(splits == 1 || part != nullptr, "latent_attention_mfma: key splits need a workspace");
    SOMI_REQUIRE(ceil_div(heads, 16) <= 65535 && splits <= LAM_MAX_SPLITS, "latent_attention_mfma: too many heads or splits");
    if (n_tokens == 0) return 0;
    const int D = rank + rot;
    int page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
    if (portions) {
        // prompt portions: several tokens a workgroup, no key splits
        SOMI_REQUIRE(splits == 1, "latent_attention_mfma: prompt portions take no key splits");
#define LAM_PORTION(STEPS, CT, TT, PW, WPS)                                                                            \
    do {                                                                                                                \
        const dim3 groups(ceil_div(n_tokens, TT), ceil_div(heads, 16));                                                 \
        const size_t lds = (size_t)16 * TT * ((STEPS * 32 + 8) * 2 + (16 * PW + 8) * 4 + PW * 4);                       \
        hipError_t err = hipFuncSetAttribute((const void*)latent_attention_portion_kernel<STEPS, CT, TT, PW, WPS>,      \
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                     \
        if (err != hipSuccess) return somi_fail("latent_attention_mfma: %s", hipGetErrorString(err));                   \
        hipLaunchKernelGGL((latent_attention_portion_kernel<STEPS, CT, TT, PW, WPS>), groups, dim3(64 * PW), lds,       \
                           stream, (const bf16*)queries, (const bf16*)latent, (const bf16*)latent_t, block_table,       \
                           max_blocks, token_entry, positions, n_tokens, heads, rank, D, page_shift, window, scale,    \
                           sink, (bf16*)out);                                                                               \
    } while (0)
        // the widest rows: two tokens and four wavefronts a workgroup, two workgroups a compute unit (four tokens and
        // eight wavefronts would not fit a wavefront's sums, fragments in flight and scores into its registers)
        if (D <= 128 && rank <= 128) LAM_PORTION(4, 2, 2, 4, 2);
        else if (D <= 256 && rank <= 256) LAM_PORTION(8, 4, 2, 4, 2);
        else LAM_PORTION(18, 8, 2, 4, 2);
#undef LAM_PORTION
        SOMI_LAUNCH_CHECK("latent_attention_portion");
        return 0;
    }
    const dim3 grid(n_tokens, ceil_div(heads, 16), splits);
#define LAM_LAUNCH(STEPS, CT)                                                                                          \
    hipLaunchKernelGGL((latent_attention_mfma_kernel<STEPS, CT>), grid, dim3(256), 0, stream, (const bf16*)queries,     \
                       (const bf16*)latent, (const bf16*)latent_t, block_table, max_blocks, token_entry, positions,    \
                       n_tokens, heads, rank, D, page_shift, window, scale, sink, splits, (bf16*)out, part)
    if (D <= 128 && rank <= 128) LAM_LAUNCH(4, 2);
    else if (D <= 256 && rank <= 256) LAM_LAUNCH(8, 4);
    else LAM_LAUNCH(18, 8);
#undef LAM_LAUNCH
    SOMI_LAUNCH_CHECK("latent_attention_mfma");
    if (splits > 1) {
        hipLaunchKernelGGL(latent_attention_join_kernel, dim3((unsigned)((int64_t)n_tokens * heads)), dim3(128), 0, stream,
                           part, splits, rank, (bf16*)out);
        SOMI_LAUNCH_CHECK("latent_attention_join");
    }
    return 0;
}
