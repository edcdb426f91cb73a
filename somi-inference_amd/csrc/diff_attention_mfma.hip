// Differential attention over cache pages on the matrix cores, bfloat16: prompt portions and decoded tokens.
//
// What diff_attention.hip computes (two softmax maps per head over shared values, o = a1 - lambda a2, o divided by
// its root mean square over the head's value channels, times out_scale; a token sees the keys within `window`
// positions and the first `keep_first` of its request), for key sizes and value sizes that are multiples of 16.
//
// A workgroup serves one query tile: 16 (token, head) slots that share a key/value head, HT heads (a power of two
// that divides heads / kv_heads) of 16 / HT consecutive tokens of one portion, or of one listed token.  Its four
// wavefronts (eight for a listed token) take the tile's 16-key tiles in turn (the kept first tokens below the window, then the window; tiles are
// aligned to absolute positions) and are merged through LDS.  Per key tile and map, in a wavefront:
//   S^T[key, slot] = K[key, :] . Q^T      v_mfma_f32_16x16x16_bf16 (16x16x32 where a quarter of a key row is a multiple
//                                         of eight channels); K rows are the A operand.  The sum over the key
//                                         channels has no order, so lane group g takes the g-th quarter of a row:
//                                         one contiguous read of dk / 4 channels per lane
//   mask by the slot's own position (tiles that every slot sees whole skip it), online softmax per slot in float32
//                                         in powers of two (a lane holds four keys of its slot) against a reference
//                                         point that follows the slot's maximum lazily
//   O^T[channel, slot] += V^T[channel, key] . P^T     S^T leaves the first product in the B-operand layout of the
//                                         second, and V is stored transposed inside a page, so a lane reads four
//                                         consecutive keys of a channel with one 8-byte load, once for both maps.
// The weights stay 32-bit in effect: P is split into a bfloat16 head and a bfloat16 rest (p = hi + lo, |lo| <= 2^-9 hi)
// and both go through the product, so no weight is rounded to eight bits.  Scores, maxima, sums, the join of the two
// maps and the norm are float32.
#include "common.h"

typedef __attribute__((ext_vector_type(4))) __bf16 dmf_bf16x4;
typedef __attribute__((ext_vector_type(4))) short dmf_short4;
typedef __attribute__((ext_vector_type(4))) float dmf_f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 dmf_bf16x8;

#define DMF_WAVES 4               // wavefronts of a workgroup for portions of prompts
#define DMF_LISTED_WAVES 8        // and for listed tokens
#define DMF_SLACK 8.0f            // powers of two a score may pass its slot's reference point by before the point moves

struct DiffArgs {
    const bf16* q; int64_t q_stride;
    const bf16* kc; const bf16* vc;
    const int* block_table; int max_blocks;
    const int* entry_start; const int* entry_first; const int* entry_len;    // portions
    const int* token_list; const int* token_entry; const int* positions;     // listed tokens
    int listed;                    // 1: a workgroup per listed token; 0: per block of tokens of a portion
    int nq, nkv, page_size, window, keep_first;
    int heads_per_tile, tokens_per_tile, subgroups;
    float scale, lambda, eps, out_scale;
    bf16* out;
};

__device__ __forceinline__ dmf_short4 dmf_ld4(const bf16* p) { return *reinterpret_cast<const dmf_short4*>(p); }
__device__ __forceinline__ dmf_bf16x8 dmf_ld8(const bf16* p) { return *reinterpret_cast<const dmf_bf16x8*>(p); }

// WAVES: wavefronts of a workgroup, which take the query tile's key tiles in turn: four for portions of prompts (two
// workgroups fit a compute unit), eight for listed tokens (decoding), whose few query tiles each walk a whole window.
template <int DKT, int DVT, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
diff_attention_mfma_kernel(const DiffArgs a) {
    constexpr int DK = 16 * DKT, DV = 16 * DVT;
    extern __shared__ float lds[];
    float* lds_acc = lds;                                          // [waves][2][DVT][64][4]
    float* lds_m = lds_acc + WAVES * 2 * DVT * 256;            // [waves][2][16]
    float* lds_l = lds_m + WAVES * 32;                         // [waves][2][16]
    float* lds_ss = lds_l + WAVES * 32;                        // [waves][16]

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    // ---- which tokens and heads
    int t0, count, e, p0;
    if (a.listed) {
        t0 = a.token_list ? a.token_list[blockIdx.x] : blockIdx.x;
        count = 1;
        e = a.token_entry[t0];
        p0 = a.positions[t0];
    } else {
        e = blockIdx.y;
        const int start = a.entry_start[e];
        const int len = a.entry_len ? a.entry_len[e] : a.entry_start[e + 1] - start;
        const int first = blockIdx.x * a.tokens_per_tile;
        if (first >= len) return;                                  // the whole workgroup: no barrier was passed yet
        t0 = start + first;
        count = min(a.tokens_per_tile, len - first);
        p0 = a.entry_first[e] + first;
    }
    const int kvh = blockIdx.z / a.subgroups, sub = blockIdx.z % a.subgroups;
    const int group = a.nq / a.nkv;
    const int slot_token = r / a.heads_per_tile, slot_head = r % a.heads_per_tile;
    const bool live = slot_token < count;
    const int head = kvh * group + sub * a.heads_per_tile + slot_head;
    const int pq = live ? p0 + slot_token : -1;                    // the slot's position; -1 sees nothing
    const int* table = a.block_table + (int64_t)e * a.max_blocks;

    // ---- the slot's two queries: lane group g holds channels g * DK/4 .. + DK/4 - 1; a product step takes four of
    // them (v_mfma_f32_16x16x16_bf16), or eight where a quarter of a row is a multiple of eight
    // (v_mfma_f32_16x16x32_bf16: half the instructions, 16-byte reads)
    constexpr bool WIDE = DKT % 2 == 0;
    constexpr int QSTEPS = WIDE ? DKT / 2 : DKT;
    dmf_short4 qf[2][WIDE ? 1 : DKT];
    dmf_bf16x8 qw[2][WIDE ? QSTEPS : 1];
#pragma unroll
    for (int map = 0; map < 2; ++map) {
        const bf16* qrow = a.q + (int64_t)(t0 + (live ? slot_token : 0)) * a.q_stride + (int64_t)(2 * head + map) * DK + g * (DK / 4);
#pragma unroll
        for (int kk = 0; kk < QSTEPS; ++kk) {
            if (WIDE) {
                qw[map][kk] = dmf_bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
                if (live) qw[map][kk] = dmf_ld8(qrow + 8 * kk);
            } else {
                qf[map][kk] = dmf_short4{0, 0, 0, 0};
                if (live) qf[map][kk] = dmf_ld4(qrow + 4 * kk);
            }
        }
    }

    // ---- the key tiles of the query tile: kept first tokens below its window, then the window
    const int pmin = p0, pmax = p0 + count - 1;
    const int wlo = (a.window > 0 && pmin - a.window + 1 > 0) ? pmin - a.window + 1 : 0;
    const int kept = a.keep_first < wlo ? a.keep_first : wlo;
    const int sink_tiles = (kept + 15) >> 4;
    const int w0 = max(wlo >> 4, sink_tiles);
    const int window_tiles = max(0, (pmax >> 4) - w0 + 1);
    const int tiles = sink_tiles + window_tiles;

    float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};
    dmf_f32x4 acc[2][DVT];
#pragma unroll
    for (int map = 0; map < 2; ++map)
#pragma unroll
        for (int c = 0; c < DVT; ++c) acc[map][c] = dmf_f32x4{0.f, 0.f, 0.f, 0.f};

    const int last_block = a.max_blocks - 1;
    const float scale2 = a.scale * 1.4426950408889634f;            // scores in units of log 2
    for (int idx = wave; idx < tiles; idx += WAVES) {
        const int tile = idx < sink_tiles ? idx : w0 + (idx - sink_tiles);
        const int j0 = tile << 4;
        // keys: lane reads row j0 + r of both maps (a row of the request's pages also where the key is masked)
        const int kpos = min(j0 + r, pmax);
        const int64_t kpage = table[min(kpos / a.page_size, last_block)];
        const bf16* krow = a.kc + ((kpage * (2 * a.nkv) + 2 * kvh) * a.page_size + kpos % a.page_size) * (int64_t)DK +
                           g * (DK / 4);
        // values: lane reads channel c * 16 + r at keys j0 + 4 g .. + 3 (one page: page_size % 4 == 0)
        const int vpos = min(j0 + 4 * g, pmax & ~3);
        const int64_t vpage = table[min(vpos / a.page_size, last_block)];
        const bf16* vbase = a.vc + (vpage * a.nkv + kvh) * (int64_t)DV * a.page_size + vpos % a.page_size;
        dmf_short4 kf[2][WIDE ? 1 : DKT], vf[DVT];
        dmf_bf16x8 kw[2][WIDE ? QSTEPS : 1];
#pragma unroll
        for (int map = 0; map < 2; ++map)
#pragma unroll
            for (int kk = 0; kk < QSTEPS; ++kk) {
                if (WIDE) kw[map][kk] = dmf_ld8(krow + (int64_t)map * a.page_size * DK + 8 * kk);
                else kf[map][kk] = dmf_ld4(krow + (int64_t)map * a.page_size * DK + 4 * kk);
            }
#pragma unroll
        for (int c = 0; c < DVT; ++c) vf[c] = dmf_ld4(vbase + (int64_t)(c * 16 + r) * a.page_size);
        // A tile whose every key every slot of the query tile sees (it ends at or before the first slot's position,
        // and begins inside the last slot's window or lies among the kept tokens) needs no mask: most tiles of a
        // long window.
        const bool full = j0 + 15 <= pmin && (a.window == 0 || pmax - j0 < a.window || j0 + 15 < a.keep_first);
        if (!full) {
            // a key that no slot of the tile sees (past the last written position, or below the window in a page that
            // was given back) may hold anything: its weight is 0, but 0 x NaN is NaN
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = j0 + 4 * g + i;
                if (j > pmax || (j < wlo && j >= a.keep_first)) {
#pragma unroll
                    for (int c = 0; c < DVT; ++c) vf[c][i] = 0;
                }
            }
        }

        dmf_short4 p_hi[2], p_lo[2];
        dmf_f32x4 s[2];
        float mx[2];
#pragma unroll
        for (int map = 0; map < 2; ++map) {
            s[map] = dmf_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < QSTEPS; ++kk) {
                if (WIDE) s[map] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kw[map][kk], qw[map][kk], s[map], 0, 0, 0);
                else s[map] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kf[map][kk], qf[map][kk], s[map], 0, 0, 0);
            }
            // s[i] = S[key j0 + 4 g + i][slot r], from here on in units of log 2: the weights are powers of two
            mx[map] = -INFINITY;
            if (full) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    s[map][i] *= scale2;
                    mx[map] = fmaxf(mx[map], s[map][i]);
                }
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int j = j0 + 4 * g + i;
                    const bool sees = j <= pq && (a.window == 0 || pq - j < a.window || j < a.keep_first);
                    s[map][i] = sees ? s[map][i] * scale2 : -INFINITY;
                    mx[map] = fmaxf(mx[map], s[map][i]);
                }
            }
        }
        // The weights are taken against a reference point per slot and map that follows the maximum lazily: it moves
        // (and the sums so far are rescaled) only when a score passes it by more than DMF_SLACK powers of two, which
        // the whole wavefront decides together; until then no lane looks at another lane's scores.
        if (__any(mx[0] > m_run[0] + DMF_SLACK || mx[1] > m_run[1] + DMF_SLACK)) {
#pragma unroll
            for (int map = 0; map < 2; ++map) {
                float top = mx[map];
                top = fmaxf(top, __shfl_xor(top, 16, 64));
                top = fmaxf(top, __shfl_xor(top, 32, 64));
                if (top > m_run[map] + DMF_SLACK) {                   // the slot's four lanes agree: top is theirs together
                    const float corr = m_run[map] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_run[map] - top);
                    l_run[map] *= corr;
#pragma unroll
                    for (int c = 0; c < DVT; ++c) acc[map][c] *= corr;
                    m_run[map] = top;
                }
            }
        }
#pragma unroll
        for (int map = 0; map < 2; ++map) {
            const float m_safe = m_run[map] == -INFINITY ? 0.f : m_run[map];      // a slot that has seen no key yet
            float sum = 0.f;
            dmf_bf16x4 hi, lo;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float p = __builtin_amdgcn_exp2f(s[map][i] - m_safe);
                sum += p;
                hi[i] = (bf16)p;
                lo[i] = (bf16)(p - (float)hi[i]);
            }
            l_run[map] += sum;                                          // the lane's own keys; lane groups are added at the end
            p_hi[map] = *reinterpret_cast<dmf_short4*>(&hi);
            p_lo[map] = *reinterpret_cast<dmf_short4*>(&lo);
        }
#pragma unroll
        for (int map = 0; map < 2; ++map)
#pragma unroll
            for (int c = 0; c < DVT; ++c) {
                acc[map][c] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf[c], p_hi[map], acc[map][c], 0, 0, 0);
                acc[map][c] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf[c], p_lo[map], acc[map][c], 0, 0, 0);
            }
    }

    // ---- merge the wavefronts: acc[map][c][i] = O^T[channel c * 16 + 4 g + i][slot r]
#pragma unroll
    for (int map = 0; map < 2; ++map) {
        float l = l_run[map];
        l += __shfl_xor(l, 16, 64);
        l += __shfl_xor(l, 32, 64);
        if (g == 0) {
            lds_m[(wave * 2 + map) * 16 + r] = m_run[map];
            lds_l[(wave * 2 + map) * 16 + r] = l;
        }
#pragma unroll
        for (int c = 0; c < DVT; ++c)
            *reinterpret_cast<dmf_f32x4*>(lds_acc + (((wave * 2 + map) * DVT + c) * 64 + lane) * 4) = acc[map][c];
    }
    __syncthreads();
    float factor[2][WAVES], l_all[2];
    bool any = true;
#pragma unroll
    for (int map = 0; map < 2; ++map) {
        float m_all = -INFINITY;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) m_all = fmaxf(m_all, lds_m[(w * 2 + map) * 16 + r]);
        any = any && m_all > -INFINITY;
        l_all[map] = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float mw = lds_m[(w * 2 + map) * 16 + r];
            factor[map][w] = (m_all > -INFINITY && mw > -INFINITY) ? exp2f(mw - m_all) : 0.f;
            l_all[map] += lds_l[(w * 2 + map) * 16 + r] * factor[map][w];
        }
    }
    // wavefront w joins the maps on the channel tiles w, w + 4, ...
    constexpr int MINE = (DVT + WAVES - 1) / WAVES;
    dmf_f32x4 o[MINE];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < MINE; ++k) {
        const int c = wave + k * WAVES;
        o[k] = dmf_f32x4{0.f, 0.f, 0.f, 0.f};
        if (c < DVT && any) {
            dmf_f32x4 sum[2] = {dmf_f32x4{0.f, 0.f, 0.f, 0.f}, dmf_f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int map = 0; map < 2; ++map)
#pragma unroll
                for (int w = 0; w < WAVES; ++w)
                    sum[map] += *reinterpret_cast<const dmf_f32x4*>(lds_acc + (((w * 2 + map) * DVT + c) * 64 + lane) * 4) *
                                factor[map][w];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                o[k][i] = sum[0][i] / l_all[0] - a.lambda * (sum[1][i] / l_all[1]);
                ss = fmaf(o[k][i], o[k][i], ss);
            }
        }
    }
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    if (g == 0) lds_ss[wave * 16 + r] = ss;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) total += lds_ss[w * 16 + r];
    const float inv = a.out_scale / sqrtf(total / (float)DV + a.eps);
    if (live) {
        bf16* row = a.out + ((int64_t)(t0 + slot_token) * a.nq + head) * DV;
#pragma unroll
        for (int k = 0; k < MINE; ++k) {
            const int c = wave + k * WAVES;
            if (c < DVT) {
                dmf_bf16x4 v = {(bf16)(o[k][0] * inv), (bf16)(o[k][1] * inv), (bf16)(o[k][2] * inv), (bf16)(o[k][3] * inv)};
                *reinterpret_cast<dmf_bf16x4*>(row + c * 16 + 4 * g) = v;
            }
        }
    }
}

template <int DKT, int DVT, int WAVES>
static int diff_mfma_launch_waves(const DiffArgs& args, dim3 grid, hipStream_t stream) {
    const size_t smem = ((size_t)WAVES * 2 * DVT * 256 + WAVES * 32 * 2 + WAVES * 16) * sizeof(float);
    static_assert(((size_t)WAVES * 2 * DVT * 256 + WAVES * 32 * 2 + WAVES * 16) * sizeof(float) <= 160 * 1024, "LDS of a compute unit");
    if (smem > 64 * 1024)
        (void)hipFuncSetAttribute((const void*)diff_attention_mfma_kernel<DKT, DVT, WAVES>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL((diff_attention_mfma_kernel<DKT, DVT, WAVES>), grid, dim3(WAVES * 64), smem, stream, args);
    SOMI_LAUNCH_CHECK("diff_attention_mfma");
    return 0;
}

template <int DKT, int DVT>
static int diff_mfma_launch(const DiffArgs& args, dim3 grid, hipStream_t stream) {
    if (args.listed) return diff_mfma_launch_waves<DKT, DVT, DMF_LISTED_WAVES>(args, grid, stream);
    return diff_mfma_launch_waves<DKT, DVT, DMF_WAVES>(args, grid, stream);
}

template <int DKT>
static int diff_mfma_by_values(int dvt, const DiffArgs& args, dim3 grid, hipStream_t stream) {
    switch (dvt) {
        case 1: return diff_mfma_launch<DKT, 1>(args, grid, stream);
        case 2: return diff_mfma_launch<DKT, 2>(args, grid, stream);
        case 3: return diff_mfma_launch<DKT, 3>(args, grid, stream);
        case 4: return diff_mfma_launch<DKT, 4>(args, grid, stream);
        case 8: return diff_mfma_launch<DKT, 8>(args, grid, stream);
    }
    return somi_fail("diff_attention_mfma: a value size of %d is not built (16, 32, 48, 64, 128)", 16 * dvt);
}

// Whether the kernel is built for these sizes (key sizes 16, 32, 48, 64, 128; value sizes 16, 32, 48, 64, 128; pages
// of a multiple of 4 keys).
extern "C" int somi_diff_attention_mfma_supported(int dk, int dv, int page_size) {
    const bool key_ok = dk == 16 || dk == 32 || dk == 48 || dk == 64 || dk == 128;
    const bool value_ok = dv == 16 || dv == 32 || dv == 48 || dv == 64 || dv == 128;
    return key_ok && value_ok && page_size > 0 && page_size % 4 == 0;
}

// The largest power of two, at most 16, that divides the query heads of a key/value head: the heads of a query tile.
extern "C" int somi_diff_attention_tile_heads(int nq, int nkv) {
    if (nq <= 0 || nkv <= 0 || nq % nkv) return 0;
    int heads = 1;
    while (heads < 16 && (nq / nkv) % (heads * 2) == 0) heads *= 2;
    return heads;
}

// Portions (token_list == null and listed == 0): the tokens of entry e are entry_start[e] .. entry_start[e + 1] - 1 at
// positions entry_first[e] ..; entry_len (or null) stands for the offsets' own lengths, 0 leaves an entry out;
// max_entry_len bounds the lengths.  Listed tokens (listed == 1): token_list (or null: all n_list tokens) names them,
// token_entry and positions give each token's entry and position.  q: token t's map m of head h starts at
// q + t * q_stride + (2 h + m) * dk.  k cache: [pages, 2 nkv, page, dk]; v cache: [pages, nkv, dv, page];
// out: [n_tokens, nq * dv] bfloat16.
extern "C" int somi_diff_attention_mfma(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                                        const int* block_table, int max_blocks, int listed, const int* entry_start,
                                        const int* entry_first, const int* entry_len, int n_entries, int max_entry_len,
                                        const int* token_list, const int* token_entry, const int* positions, int n_list,
                                        int nq, int nkv, int dk, int dv, int page_size, int window, int keep_first,
                                        float scale, float lambda, float eps, float out_scale, void* out,
                                        hipStream_t stream) {
    SOMI_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0 && max_blocks > 0, "diff_attention_mfma: bad sizes");
    SOMI_REQUIRE(somi_diff_attention_mfma_supported(dk, dv, page_size),
                 "diff_attention_mfma: key size %d, value size %d or page size %d is not built", dk, dv, page_size);
    SOMI_REQUIRE(window >= 0 && keep_first >= 0, "diff_attention_mfma: window and keep_first must be >= 0");
    SOMI_REQUIRE(q_stride % 4 == 0 && (uintptr_t)q % 8 == 0 && (uintptr_t)k_cache % 8 == 0 && (uintptr_t)v_cache % 8 == 0 &&
                 (uintptr_t)out % 8 == 0, "diff_attention_mfma: operands must be aligned to 8 bytes");
    // key sizes of a multiple of 32 read a quarter of a row sixteen bytes at a time
    SOMI_REQUIRE(dk % 32 != 0 || (q_stride % 8 == 0 && (uintptr_t)q % 16 == 0 && (uintptr_t)k_cache % 16 == 0),
                 "diff_attention_mfma: with a key size of %d the queries and the key cache must be aligned to 16 bytes", dk);
    DiffArgs args;
    args.q = (const bf16*)q; args.q_stride = q_stride; args.kc = (const bf16*)k_cache; args.vc = (const bf16*)v_cache;
    args.block_table = block_table; args.max_blocks = max_blocks;
    args.entry_start = entry_start; args.entry_first = entry_first; args.entry_len = entry_len;
    args.token_list = token_list; args.token_entry = token_entry; args.positions = positions;
    args.listed = listed ? 1 : 0;
    args.nq = nq; args.nkv = nkv; args.page_size = page_size; args.window = window; args.keep_first = keep_first;
    args.heads_per_tile = somi_diff_attention_tile_heads(nq, nkv);
    args.tokens_per_tile = listed ? 1 : 16 / args.heads_per_tile;
    args.subgroups = (nq / nkv) / args.heads_per_tile;
    args.scale = scale; args.lambda = lambda; args.eps = eps; args.out_scale = out_scale; args.out = (bf16*)out;
    dim3 grid;
    if (listed) {
        SOMI_REQUIRE(n_list >= 0 && token_entry && positions, "diff_attention_mfma: listed tokens need their entries and positions");
        if (n_list == 0) return 0;
        grid = dim3(n_list, 1, nkv * args.subgroups);
    } else {
        SOMI_REQUIRE(n_entries >= 0 && max_entry_len >= 0 && entry_start && entry_first,
                     "diff_attention_mfma: portions need their offsets and first positions");
        if (n_entries == 0 || max_entry_len == 0) return 0;
        SOMI_REQUIRE(n_entries <= 65535, "diff_attention_mfma: too many entries");
        grid = dim3(ceil_div(max_entry_len, args.tokens_per_tile), n_entries, nkv * args.subgroups);
    }
    SOMI_REQUIRE(grid.z <= 65535, "diff_attention_mfma: too many heads");
    switch (dk / 16) {
        case 1: return diff_mfma_by_values<1>(dv / 16, args, grid, stream);
        case 2: return diff_mfma_by_values<2>(dv / 16, args, grid, stream);
        case 3: return diff_mfma_by_values<3>(dv / 16, args, grid, stream);
        case 4: return diff_mfma_by_values<4>(dv / 16, args, grid, stream);
        case 8: return diff_mfma_by_values<8>(dv / 16, args, grid, stream);
    }
    return somi_fail("diff_attention_mfma: a key size of %d is not built", dk);
}
