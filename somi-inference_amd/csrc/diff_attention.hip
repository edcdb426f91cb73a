// Differential attention over cache pages: two softmax maps per head over the same values, joined and normed.
//
//   a_m[t, h] = softmax_j(q_m[t, h] . k_m[j, g] * scale) v[j, g]      m = 1, 2;  g = h / (nq / nkv)
//   o         = a_1 - lambda * a_2
//   out[t, h] = o / sqrt(mean(o^2) + eps) * out_scale                  (mean over the head's value channels)
//
// A token at position p of its request sees the keys j <= p of the same request with p - j < window (window == 0: no
// bound) or j < keep_first: a sliding window that also keeps the first tokens of the sequence, at their true
// positions.  Keys are walked in tiles aligned to absolute positions (first the kept tokens below the window, then
// the window), so the arithmetic for a (request, position) is the same whatever portion or batch the token arrives
// in.  Scores, weights, sums, the join and the norm are float32 whatever the storage type.
//
// Cache layout: K [pages, 2 nkv, page_size, dk] with the two maps of key/value head g at heads 2 g and 2 g + 1;
// V [pages, nkv, dv, page_size] (transposed inside a page).  q: token t's map m of head h starts at
// q + t * q_stride + (2 h + m) * dk.
#include "common.h"

template <typename T, int NT>
__global__ void __launch_bounds__(NT)
diff_attention_plain_kernel(const T* __restrict__ q, int64_t q_stride, const T* __restrict__ kc,
                            const T* __restrict__ vc, const int* __restrict__ block_table, int max_blocks,
                            const int* __restrict__ token_list, const int* __restrict__ token_entry,
                            const int* __restrict__ positions, int nq, int nkv, int dk, int dv, int page_size,
                            int window, int keep_first, float scale, float lambda, float eps, float out_scale,
                            T* __restrict__ out) {
    extern __shared__ float smem[];
    float* qs = smem;                          // [2][dk] the two maps' queries
    float* ps = qs + 2 * ((dk + 1) & ~1);      // [2][NT] the tile's weights of the two maps
    float* red = ps + 2 * NT;                  // [16]
    int64_t* coloff = (int64_t*)(red + 16);    // [NT] element offset of each key's value column

    const int t = token_list ? token_list[blockIdx.x] : blockIdx.x;
    const int h = blockIdx.y, tid = threadIdx.x;
    const int e = token_entry[t];
    const int p = positions[t];
    const int g = h / (nq / nkv);
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;     // first key of the window
    const int kept = keep_first < lo ? keep_first : lo;                          // keys 0 .. kept-1 lie below the window
    const int* table = block_table + (int64_t)e * max_blocks;
    const int dkp = (dk + 1) & ~1;

    for (int d = tid; d < 2 * dk; d += NT)
        qs[(d / dk) * dkp + d % dk] = to_float(q[(int64_t)t * q_stride + (int64_t)(2 * h) * dk + d]);

    float m[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};
    float acc[2][2] = {{0.f, 0.f}, {0.f, 0.f}};      // [map][r]: value channels tid and tid + NT (dv <= 2 NT)

    // two ranges of keys: [0, kept) and [lo, p]; tiles are aligned to absolute positions in both
    for (int range = 0; range < 2; ++range) {
        const int r0 = range == 0 ? 0 : lo, r1 = range == 0 ? kept - 1 : p;       // inclusive
        if (r1 < r0) continue;
        for (int tile = r0 / NT; tile <= r1 / NT; ++tile) {
            const int pos = tile * NT + tid;
            const bool valid = pos >= r0 && pos <= r1;
            __syncthreads();                    // qs ready; the previous tile's ps and coloff no longer read
            float s[2] = {-INFINITY, -INFINITY};
            if (valid) {
                const int64_t page = table[pos / page_size];
                const int64_t in_page = pos % page_size;
                coloff[tid] = (page * nkv + g) * (int64_t)dv * page_size + in_page;
#pragma unroll
                for (int map = 0; map < 2; ++map) {
                    const T* kr = kc + ((page * (2 * nkv) + (2 * g + map)) * page_size + in_page) * (int64_t)dk;
                    const float* qm = qs + map * dkp;
                    float dot = 0.f;
                    for (int d = 0; d < dk; ++d) dot = fmaf(qm[d], to_float(kr[d]), dot);
                    s[map] = dot * scale;
                }
            }
            float corr[2];
#pragma unroll
            for (int map = 0; map < 2; ++map) {
                const float tile_max = block_max<NT>(s[map], red);
                const float m_new = fmaxf(m[map], tile_max);
                corr[map] = expf(m[map] - m_new);          // exp(-inf) = 0 on the first tile
                const float w = valid ? expf(s[map] - m_new) : 0.f;
                ps[map * NT + tid] = w;
                const float tile_sum = block_sum<NT>(w, red);
                l[map] = l[map] * corr[map] + tile_sum;
                m[map] = m_new;
            }
            __syncthreads();                    // ps and coloff visible
            const int j0 = (r0 > tile * NT ? r0 : tile * NT) - tile * NT;
            const int j1 = (r1 < tile * NT + NT - 1 ? r1 : tile * NT + NT - 1) - tile * NT;
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const int d = tid + r * NT;
                if (d < dv) {
                    float a0 = acc[0][r] * corr[0], a1 = acc[1][r] * corr[1];
                    for (int j = j0; j <= j1; ++j) {
                        const float value = to_float(vc[coloff[j] + (int64_t)d * page_size]);
                        a0 = fmaf(ps[j], value, a0);
                        a1 = fmaf(ps[NT + j], value, a1);
                    }
                    acc[0][r] = a0;
                    acc[1][r] = a1;
                }
            }
        }
    }
    // join the maps, norm over the head's value channels
    float o[2], ss = 0.f;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const int d = tid + r * NT;
        o[r] = d < dv ? acc[0][r] / l[0] - lambda * (acc[1][r] / l[1]) : 0.f;
        ss = fmaf(o[r], o[r], ss);
    }
    ss = block_sum<NT>(ss, red);
    const float inv = out_scale / sqrtf(ss / (float)dv + eps);
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const int d = tid + r * NT;
        if (d < dv) out[((int64_t)t * nq + h) * dv + d] = from_float<T>(o[r] * inv);
    }
}

// token_list (or null: every token): [n_list] int32 indices of the tokens to run; block_table: [entries, max_blocks]
// int32 pages of each entry's request (pages that hold no visible key are never read); token_entry, positions:
// [n_tokens] int32.  out: [n_tokens, nq * dv].
extern "C" int somi_diff_attention_plain(const void* q, int dtype, int64_t q_stride, const void* k_cache,
                                         const void* v_cache, const int* block_table, int max_blocks,
                                         const int* token_list, const int* token_entry, const int* positions,
                                         int n_list, int nq, int nkv, int dk, int dv, int page_size, int window,
                                         int keep_first, float scale, float lambda, float eps, float out_scale,
                                         void* out, hipStream_t stream) {
    constexpr int NT = 128;
    SOMI_REQUIRE(n_list >= 0 && nq > 0 && nkv > 0 && dk > 0 && dv > 0 && page_size > 0 && max_blocks > 0,
                 "diff_attention: bad sizes");
    SOMI_REQUIRE(nq % nkv == 0, "diff_attention: heads (%d) must be divisible by kv_heads (%d)", nq, nkv);
    SOMI_REQUIRE(dv <= 2 * NT, "diff_attention: a value size of %d is larger than the supported %d", dv, 2 * NT);
    SOMI_REQUIRE(window >= 0 && keep_first >= 0, "diff_attention: window and keep_first must be >= 0");
    SOMI_REQUIRE(nq <= 65535, "diff_attention: too many heads");
    if (n_list == 0) return 0;
    const dim3 grid(n_list, nq);
    const size_t smem = (size_t)(2 * ((dk + 1) & ~1) + 2 * NT + 16) * sizeof(float) + NT * sizeof(int64_t);
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL((diff_attention_plain_kernel<float, NT>), grid, dim3(NT), smem, stream, (const float*)q,
                           q_stride, (const float*)k_cache, (const float*)v_cache, block_table, max_blocks, token_list,
                           token_entry, positions, nq, nkv, dk, dv, page_size, window, keep_first, scale, lambda, eps,
                           out_scale, (float*)out);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL((diff_attention_plain_kernel<bf16, NT>), grid, dim3(NT), smem, stream, (const bf16*)q,
                           q_stride, (const bf16*)k_cache, (const bf16*)v_cache, block_table, max_blocks, token_list,
                           token_entry, positions, nq, nkv, dk, dv, page_size, window, keep_first, scale, lambda, eps,
                           out_scale, (bf16*)out);
    else
        return somi_fail("diff_attention: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("diff_attention_plain");
    return 0;
}
