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
// Three kernels: `prepare` (convolution, SiLU, unit norms, beta, decay: everything the recurrence reads, float32),
// `conv_state` (the convolution's inputs that the next step needs) and `scan` (the recurrence).
#include "common.h"

#define DELTA_MAX_TAPS 9        // conv_state keeps taps - 1 <= 8 values a channel in registers

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// One workgroup per token.  x: the token's row [q (G dim) | k (G dim) | v (H vdim) | ...] as projected; taps: [C,
// taps] float32 for the C = 2 G dim + H vdim channels in that order; conv_state: [slots, taps - 1, C] float32, the
// inputs before the entry's first token, oldest first; ab: [N, 2 H] float32, the projections behind beta (first H)
// and the decay (last H).
template <typename T>
__global__ void __launch_bounds__(256)
delta_prepare_kernel(const T* __restrict__ x, int64_t row_stride, const float* __restrict__ ab,
                     const float* __restrict__ taps_w, int taps, const float* __restrict__ conv_state,
                     const int* __restrict__ token_entry, const int* __restrict__ entry_start,
                     const int* __restrict__ state_slots, const float* __restrict__ a_log,
                     const float* __restrict__ dt_bias, int G, int H, int dim, int vdim,
                     float* __restrict__ qkv_out /*[N, C]*/, float* __restrict__ beta, float* __restrict__ decay) {
    const int64_t t = blockIdx.x;
    const int e = token_entry[t];
    const int i = (int)t - entry_start[e];
    const int64_t slot = state_slots[e];
    const int C = 2 * G * dim + H * vdim;
    float* out = qkv_out + t * C;
    for (int c = threadIdx.x; c < C; c += 256) {
        float acc = 0.f;
        for (int d = 0; d < taps; ++d) {
            const float w = taps_w[c * taps + taps - 1 - d];
            float xv;
            if (i - d >= 0)
                xv = to_float(x[(t - d) * row_stride + c]);
            else
                xv = conv_state[(slot * (taps - 1) + (taps - 1 + i - d)) * C + c];
            acc += w * xv;
        }
        out[c] = silu_f(acc);
    }
    if (threadIdx.x < H) {
        const int h = threadIdx.x;
        beta[t * H + h] = 1.0f / (1.0f + expf(-ab[t * 2 * H + h]));
        decay[t * H + h] = expf(-expf(a_log[h]) * softplus_f(ab[t * 2 * H + H + h] + dt_bias[h]));
    }
    __syncthreads();
    // unit vectors per q and k head (2 G heads of dim channels, q heads first); q also times dim^-1/2
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

// After `prepare`: the last taps - 1 inputs of every entry's request, from the step's rows and, where the entry is
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

// The recurrence.  A wavefront (a workgroup of its own) owns DELTA_COLS columns of one (entry, head): lane = 4 *
// column + row group, and row group r of the four holds the rows r * RPL .. r * RPL + RPL - 1 of its column in
// registers (rows past dim are padding that stays zero).  A column evolves on its own: with a = (g S)^T k and
// b = (g S)^T q of the column, u = beta (v - a), the new column is g S + k u and o = b + u (k . q).  The token's k and
// q go through LDS (two buffers: the next token's are asked of memory before this token's arithmetic).  The order of
// the operations does not depend on how a prompt is cut, so float32 results are the same for every cut.
#define DELTA_COLS 16
#define DELTA_GROUPS 4

template <int RPL>
__global__ void __launch_bounds__(64)
delta_scan_kernel(const float* __restrict__ qkv /*[N, C]*/, const float* __restrict__ beta,
                  const float* __restrict__ decay, const int* __restrict__ entry_start,
                  const int* __restrict__ state_slots, float* __restrict__ state /*[slots, H, dim, vdim]*/, int G, int H,
                  int dim, int vdim, float* __restrict__ o /*[N, H, vdim]*/) {
    __shared__ float kq[2][2][DELTA_GROUPS * RPL];
    const int e = blockIdx.x, h = blockIdx.y;
    const int lane = threadIdx.x, col = blockIdx.z * DELTA_COLS + (lane >> 2), rg = lane & 3;
    const int g = h / (H / G);
    const int C = 2 * G * dim + H * vdim;
    const int start = entry_start[e], end = entry_start[e + 1];
    const bool live = col < vdim;
    float* S_mem = state + (((int64_t)state_slots[e] * H + h) * dim) * vdim;
    float S[RPL];
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
        const int d = rg * RPL + r;
        S[r] = (live && d < dim) ? S_mem[(int64_t)d * vdim + col] : 0.f;
    }
    const int padded = DELTA_GROUPS * RPL;
    // a lane stages the elements lane, lane + 64, ... of k and of q
    float nk[(DELTA_GROUPS * RPL + 63) / 64], nq[(DELTA_GROUPS * RPL + 63) / 64];
    float nv = 0.f, nb = 0.f, ng = 0.f;
    auto fetch = [&](int t) {
        const float* row = qkv + (int64_t)t * C;
#pragma unroll
        for (int j = 0; j < (DELTA_GROUPS * RPL + 63) / 64; ++j) {
            const int d = lane + 64 * j;
            nq[j] = d < dim ? row[g * dim + d] : 0.f;
            nk[j] = d < dim ? row[G * dim + g * dim + d] : 0.f;
        }
        nv = live ? row[2 * G * dim + h * vdim + col] : 0.f;
        nb = beta[(int64_t)t * H + h];
        ng = decay[(int64_t)t * H + h];
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int j = 0; j < (DELTA_GROUPS * RPL + 63) / 64; ++j) {
            const int d = lane + 64 * j;
            if (d < padded) {
                kq[buf][0][d] = nk[j];
                kq[buf][1][d] = nq[j];
            }
        }
    };
    if (start < end) {
        fetch(start);
        stage(0);
    }
    __syncthreads();
    for (int t = start; t < end; ++t) {
        const int buf = (t - start) & 1;
        const float v = nv, b_t = nb, g_t = ng;
        if (t + 1 < end) fetch(t + 1);
        const float* ks = kq[buf][0] + rg * RPL;
        const float* qs = kq[buf][1] + rg * RPL;
        float a = 0.f, b = 0.f, kdq = 0.f;
#pragma unroll
        for (int r = 0; r < RPL; ++r) {
            S[r] *= g_t;
            a += S[r] * ks[r];
            b += S[r] * qs[r];
            kdq += ks[r] * qs[r];
        }
        a += __shfl_xor(a, 1, 64);
        b += __shfl_xor(b, 1, 64);
        kdq += __shfl_xor(kdq, 1, 64);
        a += __shfl_xor(a, 2, 64);
        b += __shfl_xor(b, 2, 64);
        kdq += __shfl_xor(kdq, 2, 64);
        const float u = b_t * (v - a);
#pragma unroll
        for (int r = 0; r < RPL; ++r) S[r] += ks[r] * u;
        if (live && rg == 0) o[((int64_t)t * H + h) * vdim + col] = b + u * kdq;
        if (t + 1 < end) stage(buf ^ 1);
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
    SOMI_REQUIRE(heads <= 256, "delta_prepare: more than 256 heads");
    const int C = 2 * groups * dim + heads * vdim;
    SOMI_REQUIRE(row_stride >= C, "delta_prepare: rows too narrow");
    if (n_tokens == 0) return 0;
    const dim3 cgrid(n_entries, ceil_div(C, 256));
    if (dtype == SOMI_F32) {
        hipLaunchKernelGGL(delta_prepare_kernel<float>, dim3(n_tokens), dim3(256), 0, stream, (const float*)x, row_stride, ab,
                           taps_w, taps, conv_state, token_entry, entry_start, state_slots, a_log, dt_bias, groups, heads,
                           dim, vdim, qkv_out, beta, decay);
        if (taps > 1)
            hipLaunchKernelGGL(delta_conv_state_kernel<float>, cgrid, dim3(256), 0, stream, (const float*)x, row_stride, taps,
                               conv_state, entry_start, state_slots, C);
    } else if (dtype == SOMI_BF16) {
        hipLaunchKernelGGL(delta_prepare_kernel<bf16>, dim3(n_tokens), dim3(256), 0, stream, (const bf16*)x, row_stride, ab,
                           taps_w, taps, conv_state, token_entry, entry_start, state_slots, a_log, dt_bias, groups, heads,
                           dim, vdim, qkv_out, beta, decay);
        if (taps > 1)
            hipLaunchKernelGGL(delta_conv_state_kernel<bf16>, cgrid, dim3(256), 0, stream, (const bf16*)x, row_stride, taps,
                               conv_state, entry_start, state_slots, C);
    } else {
        return somi_fail("delta_prepare: unknown dtype %d", dtype);
    }
    SOMI_LAUNCH_CHECK("delta_prepare");
    return 0;
}

extern "C" int somi_delta_scan(const float* qkv, const float* beta, const float* decay, const int* entry_start,
                               const int* state_slots, float* state, int n_entries, int groups, int heads, int dim,
                               int vdim, float* o, hipStream_t stream) {
    SOMI_REQUIRE(n_entries >= 0 && groups > 0 && heads > 0 && heads % groups == 0 && dim > 0 && vdim > 0,
                 "delta_scan: bad sizes");
    SOMI_REQUIRE(dim <= 64 * DELTA_GROUPS, "delta_scan: a key size of %d is more than the supported %d", dim, 64 * DELTA_GROUPS);
    SOMI_REQUIRE(heads <= 65535 && ceil_div(vdim, DELTA_COLS) <= 65535, "delta_scan: too many heads or columns");
    if (n_entries == 0) return 0;
    const dim3 grid(n_entries, heads, ceil_div(vdim, DELTA_COLS));
    const int rpl = ceil_div(dim, DELTA_GROUPS);
#define SOMI_DELTA(R)                                                                                                  \
    hipLaunchKernelGGL(delta_scan_kernel<R>, grid, dim3(64), 0, stream, qkv, beta, decay, entry_start, state_slots, state, \
                       groups, heads, dim, vdim, o)
    if (rpl <= 8) SOMI_DELTA(8);
    else if (rpl <= 16) SOMI_DELTA(16);
    else if (rpl <= 32) SOMI_DELTA(32);
    else SOMI_DELTA(64);
#undef SOMI_DELTA
    SOMI_LAUNCH_CHECK("delta_scan");
    return 0;
}
