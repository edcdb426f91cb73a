// Gated linear attention: a recurrent state per request and head, carried from token to token.
//
//   alpha[t, h, d] = sigmoid(z)^(1/tau),  z = W2 (a[t]) + b           (a: the low-rank projection of the input)
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
// alpha[t, c] = exp(-softplus(-z) / tau), z = bias[c] + sum_r a[t, r] * w2[c, r].  One thread per (t, c).
template <typename T>
__global__ void __launch_bounds__(256)
gla_decay_kernel(const T* __restrict__ a, int64_t a_stride, const T* __restrict__ w2, const float* __restrict__ bias,
                 float inv_tau, float* __restrict__ alpha, int channels, int rank, int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) {
        const int64_t t = i / channels;
        const int c = (int)(i - t * channels);
        const T* ar = a + t * a_stride;
        const T* wr = w2 + (int64_t)c * rank;
        float z = 0.f;
        for (int r = 0; r < rank; ++r) z = fmaf(to_float(ar[r]), to_float(wr[r]), z);
        z += bias ? bias[c] : 0.f;
        // log sigmoid(z) = -softplus(-z) = -(max(-z, 0) + log1p(exp(-|z|)))
        const float log_sigmoid = -(fmaxf(-z, 0.f) + log1pf(expf(-fabsf(z))));
        alpha[i] = expf(log_sigmoid * inv_tau);
    }
}

extern "C" int somi_gla_decay(const void* a, int dtype, int64_t a_stride, const void* w2, const float* bias, float tau,
                              float* alpha, int n_tokens, int channels, int rank, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && channels > 0 && rank > 0 && a_stride >= rank, "gla_decay: bad sizes");
    SOMI_REQUIRE(tau > 0.f, "gla_decay: tau must be > 0");
    const int64_t count = (int64_t)n_tokens * channels;
    if (count == 0) return 0;
    const int grid = (int)(ceil_div64(count, 256) < 65536 ? ceil_div64(count, 256) : 65536);
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(gla_decay_kernel<float>, dim3(grid), dim3(256), 0, stream, (const float*)a, a_stride,
                           (const float*)w2, bias, 1.0f / tau, alpha, channels, rank, count);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(gla_decay_kernel<bf16>, dim3(grid), dim3(256), 0, stream, (const bf16*)a, a_stride,
                           (const bf16*)w2, bias, 1.0f / tau, alpha, channels, rank, count);
    else
        return somi_fail("gla_decay: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("gla_decay");
    return 0;
}

// ------------------------------------------------------------------------------------------------ the recurrence
// A wavefront owns GLA_COLS columns of one (entry, head): lane = column + GLA_COLS * row group; row group r of
// GLA_GROUPS holds the rows d = r, r + GLA_GROUPS, ... of its column in registers (RPL of them).  Per token the
// wavefront's alpha, k and q of the head are staged through LDS GLA_STAGE tokens at a time (a workgroup is one wavefront, which
// stages for itself), a lane updates its rows and sums its share of o, and the row groups'
// shares are added by two lane exchanges, always in the same order.
#define GLA_COLS 16
#define GLA_GROUPS 4
#define GLA_STAGE 16

template <typename T, int RPL>
__global__ void __launch_bounds__(64)
gla_scan_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, int64_t row_stride,
                const float* __restrict__ alpha, const int* __restrict__ entry_start,
                const int* __restrict__ state_slots, float* __restrict__ state, int heads, int dim, int vdim,
                float q_scale, float* __restrict__ o) {
    extern __shared__ float staged[];              // [3][GLA_STAGE][dim]: alpha, k, q (scaled)
    const int e = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int col = blockIdx.z * GLA_COLS + (lane % GLA_COLS), group = lane / GLA_COLS;
    const bool live = col < vdim;
    const int t0 = entry_start[e], t1 = entry_start[e + 1];
    float* S = state + (((int64_t)state_slots[e] * heads + h) * dim) * (int64_t)vdim;
    float s[RPL];
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
        const int d = group + i * GLA_GROUPS;
        s[i] = (live && d < dim) ? S[(int64_t)d * vdim + col] : 0.f;
    }
    float* sa = staged;
    float* sk = staged + GLA_STAGE * dim;
    float* sq = staged + 2 * GLA_STAGE * dim;
    for (int base = t0; base < t1; base += GLA_STAGE) {
        const int count = min(GLA_STAGE, t1 - base);
        for (int i = lane; i < count * dim; i += 64) {
            const int tt = i / dim, d = i - tt * dim;
            const int64_t at = (int64_t)(base + tt) * row_stride + (int64_t)h * dim + d;
            sa[i] = alpha[((int64_t)(base + tt) * heads + h) * dim + d];
            sk[i] = to_float(k[at]);
            sq[i] = to_float(q[at]) * q_scale;
        }
        __syncthreads();                           // one wavefront a workgroup: its stores to LDS before its reads
        for (int tt = 0; tt < count; ++tt) {
            const float vt = live ? to_float(v[(int64_t)(base + tt) * row_stride + (int64_t)h * vdim + col]) : 0.f;
            const float* a = sa + tt * dim;
            const float* kk = sk + tt * dim;
            const float* qq = sq + tt * dim;
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < RPL; ++i) {
                const int d = group + i * GLA_GROUPS;
                if (d < dim) {
                    s[i] = fmaf(a[d], s[i], kk[d] * vt);
                    acc = fmaf(s[i], qq[d], acc);
                }
            }
            acc += __shfl_xor(acc, GLA_COLS, 64);
            acc += __shfl_xor(acc, 2 * GLA_COLS, 64);
            if (live && group == 0) o[((int64_t)(base + tt) * heads + h) * vdim + col] = acc;
        }
        __syncthreads();                           // the reads, before the next tokens are staged
    }
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
        const int d = group + i * GLA_GROUPS;
        if (live && d < dim) S[(int64_t)d * vdim + col] = s[i];
    }
}

// q, k: [n_tokens, row_stride] with head h at columns h * dim ..; v: the same with head h at h * vdim ..
// alpha: [n_tokens, heads, dim] float32.  entry_start: [n_entries + 1] offsets of the entries' tokens;
// state_slots: [n_entries]; state: [slots, heads, dim, vdim] float32, read and written in place.
// o: [n_tokens, heads, vdim] float32.
extern "C" int somi_gla_scan(const void* q, const void* k, const void* v, int dtype, int64_t row_stride,
                             const float* alpha, const int* entry_start, const int* state_slots, float* state,
                             int n_entries, int heads, int dim, int vdim, float q_scale, float* o,
                             hipStream_t stream) {
    SOMI_REQUIRE(n_entries >= 0 && heads > 0 && dim > 0 && vdim > 0, "gla_scan: bad sizes");
    SOMI_REQUIRE(dim <= 64 * GLA_GROUPS, "gla_scan: a key size of %d is more than the supported %d", dim, 64 * GLA_GROUPS);
    SOMI_REQUIRE(row_stride >= (int64_t)heads * dim && row_stride >= (int64_t)heads * vdim, "gla_scan: rows too narrow");
    SOMI_REQUIRE(heads <= 65535 && ceil_div(vdim, GLA_COLS) <= 65535, "gla_scan: too many heads or columns");
    if (n_entries == 0) return 0;
    const dim3 grid(n_entries, heads, ceil_div(vdim, GLA_COLS));
    const size_t lds = (size_t)3 * GLA_STAGE * dim * sizeof(float);
    const int rpl = ceil_div(dim, GLA_GROUPS);
#define GLA_LAUNCH(T, R)                                                                                              \
    hipLaunchKernelGGL((gla_scan_kernel<T, R>), grid, dim3(64), lds, stream, (const T*)q, (const T*)k, (const T*)v,   \
                       row_stride, alpha, entry_start, state_slots, state, heads, dim, vdim, q_scale, o)
#define GLA_BY_ROWS(T)                                                                                                \
    do {                                                                                                              \
        if (rpl <= 8) GLA_LAUNCH(T, 8);                                                                               \
        else if (rpl <= 16) GLA_LAUNCH(T, 16);                                                                        \
        else if (rpl <= 32) GLA_LAUNCH(T, 32);                                                                        \
        else GLA_LAUNCH(T, 64);                                                                                       \
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
// y[t, h, c] = o / sqrt(mean_c(o^2) + eps) * w[c] * silu(g[t, h, c]).  One wavefront per (token, head).
template <typename T>
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
    const T* grow = g + t * g_stride + (int64_t)h * vdim;
    T* yrow = y + (t * heads + h) * vdim;
    for (int c = lane; c < vdim; c += 64) {
        const float gate = to_float(grow[c]);
        const float silu = gate / (1.0f + expf(-gate));
        yrow[c] = from_float<T>(orow[c] * inv * w[c] * silu);
    }
}

// o: [n_tokens, heads, vdim] float32; w: [vdim] float32; g: [n_tokens, g_stride] with head h at h * vdim ..;
// y: [n_tokens, heads * vdim] in the storage type.
extern "C" int somi_gla_norm_gate(const float* o, const float* w, const void* g, int dtype, int64_t g_stride, float eps,
                                  void* y, int n_tokens, int heads, int vdim, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && heads > 0 && vdim > 0 && g_stride >= (int64_t)heads * vdim, "gla_norm_gate: bad sizes");
    SOMI_REQUIRE(heads <= 65535, "gla_norm_gate: too many heads");
    if (n_tokens == 0) return 0;
    const dim3 grid(n_tokens, heads);
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(gla_norm_gate_kernel<float>, grid, dim3(64), 0, stream, o, w, (const float*)g, g_stride, eps,
                           (float*)y, heads, vdim);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(gla_norm_gate_kernel<bf16>, grid, dim3(64), 0, stream, o, w, (const bf16*)g, g_stride, eps,
                           (bf16*)y, heads, vdim);
    else
        return somi_fail("gla_norm_gate: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("gla_norm_gate");
    return 0;
}
