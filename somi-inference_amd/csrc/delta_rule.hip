// The gated delta rule: a recurrent mixer with a float32 matrix state per request and head.
//
// Per head (state S: dim x vdim, from zero), with unit-length k, unit-length q times dim^-1/2, a write strength beta
// in (0, 1) and a decay g in (0, 1):
//
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q          (o sees the token's own write)
//
// q and k have `groups` heads that the `heads` value heads share (head h reads group h / (heads / groups)).
// Before that q, k and v pass a short causal convolution over time per channel (taps[c, last] weighs the current
// token, zeros before a sequence's start) and SiLU; the last taps - 1 inputs of a request are state as well.
//
// Four kernels: `conv` (convolution and SiLU) and `unit` (unit norms, beta, decay), which together leave everything
// the recurrence reads in float32; `conv_state` (the convolution's inputs that the next step needs); `scan` (the
// recurrence).
#include "common.h"

#define DELTA_MAX_TAPS 9        // conv_state keeps taps - 1 <= 8 values a channel in registers

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// The convolution: a thread per (token, channel).  x: the token's row [q (G dim) | k (G dim) | v (H vdim) | ...] as
// projected; taps: [C, taps] float32 for the C = 2 G dim + H vdim channels in that order; conv_state: [slots,
// taps - 1, C] float32, the inputs before the entry's first token, oldest first.
template <typename T>
__global__ void __launch_bounds__(256)
delta_conv_kernel(const T* __restrict__ x, int64_t row_stride, const float* __restrict__ taps_w, int taps,
                  const float* __restrict__ conv_state, const int* __restrict__ token_entry,
                  const int* __restrict__ entry_start, const int* __restrict__ state_slots, int C,
                  float* __restrict__ qkv_out /*[N, C]*/) {
    const int64_t t = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int e = token_entry[t];
    const int i = (int)t - entry_start[e];
    const int64_t slot = state_slots[e];
    float acc = 0.f;
#pragma unroll
    for (int d = 0; d < DELTA_MAX_TAPS; ++d) {
        if (d >= taps) break;
        const float w = taps_w[c * taps + taps - 1 - d];
        const float xv = i - d >= 0 ? to_float(x[(t - d) * row_stride + c])
                                    : conv_state[(slot * (taps - 1) + (taps - 1 + i - d)) * C + c];
        acc += w * xv;
    }
    qkv_out[t * C + c] = silu_f(acc);
}

// One workgroup per token, after the convolution: unit vectors per q and k head (2 G heads of dim channels, q heads
// first; q also times dim^-1/2), and beta and the decay from ab: [N, 2 H] float32, the projections behind beta (first
// H) and the decay (last H).
__global__ void __launch_bounds__(256)
delta_unit_kernel(const float* __restrict__ ab, const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                  int G, int H, int dim, int vdim, float* __restrict__ qkv_out /*[N, C]*/, float* __restrict__ beta,
                  float* __restrict__ decay) {
    const int64_t t = blockIdx.x;
    const int C = 2 * G * dim + H * vdim;
    float* out = qkv_out + t * C;
    for (int h = threadIdx.x; h < H; h += 256) {
        beta[t * H + h] = 1.0f / (1.0f + expf(-ab[t * 2 * H + h]));
        decay[t * H + h] = expf(-expf(a_log[h]) * softplus_f(ab[t * 2 * H + H + h] + dt_bias[h]));
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const float q_scale = 1.0f / sqrtf((float)dim);
    for (int head = wave; head < 2 * G; head += 4) {
        float* p = out + head * dim;
        float ss = 0.f;
        for (int d = lane; d < dim; d += 64) ss += p[d] * p[d];
        ss = wave_sum(ss);
        const float inv = (head < G ? q_scale : 1.0f) / sqrtf(ss + 1e-6f);
        for (int d = lane; d < dim; d += 64) p[d] *= inv;
    }
}

// After `conv`: the last taps - 1 inputs of every entry's request, from the step's rows and, where the entry is
// shorter than that, from what the state held.  A thread reads all of a channel's values before it writes any.
template <typename T>
__global__ void __launch_bounds__(256)
delta_conv_state_kernel(const T* __restrict__ x, int64_t row_stride, int taps, float* __restrict__ conv_state,
                        const int* __restrict__ entry_start, const int* __restrict__ state_slots, int C) {
    const int e = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int start = entry_start[e], len = entry_start[e + 1] - start;
    float* st = conv_state + (int64_t)state_slots[e] * (taps - 1) * C;
    float vals[DELTA_MAX_TAPS - 1];
#pragma unroll
    for (int s = 0; s < DELTA_MAX_TAPS - 1; ++s) {
        if (s >= taps - 1) break;
        const int j = len - (taps - 1) + s;          // index among the entry's tokens; negative: before the entry
        vals[s] = j >= 0 ? to_float(x[(int64_t)(start + j) * row_stride + c]) : st[(taps - 1 + j) * C + c];
    }
#pragma unroll
    for (int s = 0; s < DELTA_MAX_TAPS - 1; ++s) {
        if (s >= taps - 1) break;
        st[s * C + c] = vals[s];
    }
}

// The recurrence.  A wavefront (a workgroup of its own) owns 64 / LPC columns of one (entry, head): lane = LPC *
// column + row group, and row group r of the LPC (4 or 16) holds the rows r * RPL .. r * RPL + RPL - 1 of its column in
// registers (rows past dim are padding that stays zero).  A column evolves on its own: with a = (g S)^T k and
// b = (g S)^T q of the column, u = beta (v - a), the new column is g S + k u and o = b + u (k . q).  The tokens' k, q,
// v, beta and g go through LDS CH tokens at a time; the next CH tokens are asked of memory before this chunk's
// arithmetic and not touched until they are staged, so that their way from memory hides behind a whole chunk.  The
// order of the operations does not depend on how a prompt is cut, so float32 results are the same for every cut.
// The value of another lane by a data-parallel move (no LDS, no wait): a quad permutation or a rotation of a row of 16.
template <int PATTERN> __device__ __forceinline__ float delta_dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), PATTERN, 0xF, 0xF, true));
}
// The sum over the LPC (4 or 16) neighbouring lanes that share a column, left in all of them.
template <int LPC> __device__ __forceinline__ float delta_group_sum(float v) {
    v += delta_dpp<0xB1>(v);                 // the neighbour in the quad
    v += delta_dpp<0x4E>(v);                 // the other pair of the quad
    if (LPC == 16) {
        v += delta_dpp<0x124>(v);            // the quad four lanes on in the row of 16
        v += delta_dpp<0x128>(v);            // the pair of quads eight lanes on
    }
    return v;
}

template <int LPC, int RPL, int CH>
__global__ void __launch_bounds__(64)
delta_scan_kernel(const float* __restrict__ qkv /*[N, C]*/, const float* __restrict__ beta,
                  const float* __restrict__ decay, const int* __restrict__ entry_start,
                  const int* __restrict__ state_slots, float* __restrict__ state /*[slots, H, dim, vdim]*/, int G, int H,
                  int dim, int vdim, float* __restrict__ o /*[N, H, vdim]*/) {
    constexpr int DELTA_COLS = 64 / LPC;                // columns of a wavefront
    constexpr int PAD = LPC * RPL;            // rows of a column with the padding
    constexpr int PJ = (PAD + 63) / 64;                // elements of k (or q) of one token a lane stages
    constexpr int VJ = (CH * DELTA_COLS + 63) / 64;    // elements of v of a chunk a lane stages
    __shared__ __attribute__((aligned(16))) float ks[CH][PAD];
    __shared__ __attribute__((aligned(16))) float qs[CH][PAD];
    __shared__ float vs[CH][DELTA_COLS];
    __shared__ float bg[2][CH];
    const int e = blockIdx.x, h = blockIdx.y;
    const int lane = threadIdx.x, col = blockIdx.z * DELTA_COLS + lane / LPC, rg = lane % LPC;
    const int g = h / (H / G);
    const int C = 2 * G * dim + H * vdim;
    const int start = entry_start[e], end = entry_start[e + 1];
    if (start >= end) return;
    const bool live = col < vdim;
    float* S_mem = state + (((int64_t)state_slots[e] * H + h) * dim) * vdim;
    float S[RPL];
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
        const int d = rg * RPL + r;
        S[r] = (live && d < dim) ? S_mem[(int64_t)d * vdim + col] : 0.f;
    }
    // what a lane asks of memory for a chunk: addresses are clamped into the entry's rows and the row's channels
    // (what they bring for padding is dropped when it is staged), so no loaded value is looked at before its time
    float nk[CH][PJ], nq[CH][PJ], nv[VJ], nbg = 0.f;
    const int vcols = min(DELTA_COLS, vdim - blockIdx.z * DELTA_COLS);
    auto fetch = [&](int t0) {
#pragma unroll
        for (int tt = 0; tt < CH; ++tt) {
            const float* row = qkv + (int64_t)min(t0 + tt, end - 1) * C;
#pragma unroll
            for (int j = 0; j < PJ; ++j) {
                const int d = min(lane + 64 * j, dim - 1);
                nq[tt][j] = row[g * dim + d];
                nk[tt][j] = row[G * dim + g * dim + d];
            }
        }
#pragma unroll
        for (int j = 0; j < VJ; ++j) {
            const int idx = lane + 64 * j, tt = min(idx / DELTA_COLS, CH - 1), c = min(idx % DELTA_COLS, vcols - 1);
            nv[j] = qkv[(int64_t)min(t0 + tt, end - 1) * C + 2 * G * dim + h * vdim + blockIdx.z * DELTA_COLS + c];
        }
        const int tb = min(t0 + (lane & (CH - 1)), end - 1);
        nbg = (lane < CH ? beta : decay)[(int64_t)tb * H + h];
    };
    auto stage = [&]() {
#pragma unroll
        for (int tt = 0; tt < CH; ++tt)
#pragma unroll
            for (int j = 0; j < PJ; ++j) {
                const int d = lane + 64 * j;
                if (d < PAD) {
                    ks[tt][d] = d < dim ? nk[tt][j] : 0.f;
                    qs[tt][d] = d < dim ? nq[tt][j] : 0.f;
                }
            }
#pragma unroll
        for (int j = 0; j < VJ; ++j) {
            const int idx = lane + 64 * j;
            if (idx < CH * DELTA_COLS) vs[idx / DELTA_COLS][idx % DELTA_COLS] = nv[j];
        }
        if (lane < 2 * CH) bg[lane / CH][lane & (CH - 1)] = nbg;
    };
    fetch(start);
    for (int t0 = start; t0 < end; t0 += CH) {
        stage();
        __syncthreads();
        if (t0 + CH < end) fetch(t0 + CH);
        const int count = min(CH, end - t0);
        for (int tt = 0; tt < count; ++tt) {
            const float* kt = ks[tt] + rg * RPL;
            const float* qt = qs[tt] + rg * RPL;
            const float v = vs[tt][lane / LPC], b_t = bg[0][tt], g_t = bg[1][tt];
            float a = 0.f, b = 0.f, kdq = 0.f;
#pragma unroll
            for (int r = 0; r < RPL; ++r) {
                S[r] *= g_t;
                a += S[r] * kt[r];
                b += S[r] * qt[r];
                kdq += kt[r] * qt[r];
            }
            a = delta_group_sum<LPC>(a);
            b = delta_group_sum<LPC>(b);
            kdq = delta_group_sum<LPC>(kdq);
            const float u = b_t * (v - a);
#pragma unroll
            for (int r = 0; r < RPL; ++r) S[r] += kt[r] * u;
            if (live && rg == 0) o[((int64_t)(t0 + tt) * H + h) * vdim + col] = b + u * kdq;
        }
        __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
        const int d = rg * RPL + r;
        if (live && d < dim) S_mem[(int64_t)d * vdim + col] = S[r];
    }
}

extern "C" int somi_delta_prepare(const void* x, int dtype, int64_t row_stride, const float* ab, const float* taps_w,
                                  int taps, float* conv_state, const int* token_entry, const int* entry_start,
                                  const int* state_slots, const float* a_log, const float* dt_bias, int n_tokens,
                                  int n_entries, int groups, int heads, int dim, int vdim, float* qkv_out, float* beta,
                                  float* decay, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && n_entries >= 0 && groups > 0 && heads > 0 && heads % groups == 0 && dim > 0 && vdim > 0,
                 "delta_prepare: bad sizes");
    SOMI_REQUIRE(taps >= 1 && taps <= DELTA_MAX_TAPS, "delta_prepare: %d taps, at most %d are supported", taps, DELTA_MAX_TAPS);
    SOMI_REQUIRE(ceil_div(2 * groups * dim + heads * vdim, 256) <= 65535, "delta_prepare: too many channels");
    const int C = 2 * groups * dim + heads * vdim;
    SOMI_REQUIRE(row_stride >= C, "delta_prepare: rows too narrow");
    if (n_tokens == 0) return 0;
    const dim3 cgrid(n_entries, ceil_div(C, 256));
    const dim3 tgrid(n_tokens, ceil_div(C, 256));
    if (dtype == SOMI_F32) {
        hipLaunchKernelGGL(delta_conv_kernel<float>, tgrid, dim3(256), 0, stream, (const float*)x, row_stride, taps_w, taps,
                           conv_state, token_entry, entry_start, state_slots, C, qkv_out);
        if (taps > 1)
            hipLaunchKernelGGL(delta_conv_state_kernel<float>, cgrid, dim3(256), 0, stream, (const float*)x, row_stride, taps,
                               conv_state, entry_start, state_slots, C);
    } else if (dtype == SOMI_BF16) {
        hipLaunchKernelGGL(delta_conv_kernel<bf16>, tgrid, dim3(256), 0, stream, (const bf16*)x, row_stride, taps_w, taps,
                           conv_state, token_entry, entry_start, state_slots, C, qkv_out);
        if (taps > 1)
            hipLaunchKernelGGL(delta_conv_state_kernel<bf16>, cgrid, dim3(256), 0, stream, (const bf16*)x, row_stride, taps,
                               conv_state, entry_start, state_slots, C);
    } else {
        return somi_fail("delta_prepare: unknown dtype %d", dtype);
    }
    hipLaunchKernelGGL(delta_unit_kernel, dim3(n_tokens), dim3(256), 0, stream, ab, a_log, dt_bias, groups, heads, dim, vdim,
                       qkv_out, beta, decay);
    SOMI_LAUNCH_CHECK("delta_prepare");
    return 0;
}

extern "C" int somi_delta_scan(const float* qkv, const float* beta, const float* decay, const int* entry_start,
                               const int* state_slots, float* state, int n_entries, int groups, int heads, int dim,
                               int vdim, int lanes, float* o, hipStream_t stream) {
    SOMI_REQUIRE(n_entries >= 0 && groups > 0 && heads > 0 && heads % groups == 0 && dim > 0 && vdim > 0,
                 "delta_scan: bad sizes");
    SOMI_REQUIRE(lanes == 0 || lanes == 4 || lanes == 16, "delta_scan: %d lanes a column (0 for the launcher's choice, 4 or 16)", lanes);
    SOMI_REQUIRE(dim <= 256, "delta_scan: a key size of %d is more than the supported 256", dim);
    if (n_entries == 0) return 0;
    // Lanes a column: 16 where 4 would leave the device short of wavefronts.  The choice looks at the model's sizes and
    // the device only, never at the step, so a request's sums run in one order whatever else is in the batch.
    const bool wide = lanes == 0 ? heads * ceil_div(vdim, 16) < 2 * somi_units() : lanes == 16;
    const int lpc = wide ? 16 : 4, cols = 64 / lpc;
    SOMI_REQUIRE(heads <= 65535 && ceil_div(vdim, cols) <= 65535, "delta_scan: too many heads or columns");
    const dim3 grid(n_entries, heads, ceil_div(vdim, cols));
    const int rpl = ceil_div(dim, lpc);
#define SOMI_DELTA(L, R, CH)                                                                                               \
    hipLaunchKernelGGL((delta_scan_kernel<L, R, CH>), grid, dim3(64), 0, stream, qkv, beta, decay, entry_start, state_slots, \
                       state, groups, heads, dim, vdim, o)
    if (wide) {
        if (rpl <= 4) SOMI_DELTA(16, 4, 16);
        else if (rpl <= 8) SOMI_DELTA(16, 8, 16);
        else SOMI_DELTA(16, 16, 8);
    } else {
        if (rpl <= 8) SOMI_DELTA(4, 8, 16);
        else if (rpl <= 16) SOMI_DELTA(4, 16, 16);
        else if (rpl <= 32) SOMI_DELTA(4, 32, 16);
        else SOMI_DELTA(4, 64, 8);
    }
#undef SOMI_DELTA
    SOMI_LAUNCH_CHECK("delta_scan");
    return 0;
}
