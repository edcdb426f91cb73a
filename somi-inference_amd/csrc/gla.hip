// Gated linear attention: a recurrent state per request and head, carried from token to token.
//
//   alpha[t, h, d] = sigmoid(z)^(1/tau),  z = W2 (a[t]) + b           (a: the low-rank projection of the input; z
//                                                                    comes from the engine's matrix products)
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
// alpha = sigmoid(z)^(1 / tau) = exp(-softplus(-z) / tau), in place on the float32 sums z of the decay's projection.
__global__ void __launch_bounds__(256)
gla_alpha_kernel(float* __restrict__ z, float inv_tau, int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) {
        const float x = z[i];
        // log sigmoid(x) = -softplus(-x) = -(max(-x, 0) + log1p(exp(-|x|)))
        const float log_sigmoid = -(fmaxf(-x, 0.f) + log1pf(expf(-fabsf(x))));
        z[i] = expf(log_sigmoid * inv_tau);
    }
}

extern "C" int somi_gla_alpha(float* z, float tau, int64_t count, hipStream_t stream) {
    SOMI_REQUIRE(count >= 0 && tau > 0.f, "gla_alpha: bad arguments");
    if (count == 0) return 0;
    const int grid = (int)(ceil_div64(count, 256) < 65536 ? ceil_div64(count, 256) : 65536);
    hipLaunchKernelGGL(gla_alpha_kernel, dim3(grid), dim3(256), 0, stream, z, 1.0f / tau, count);
    SOMI_LAUNCH_CHECK("gla_alpha");
    return 0;
}

// ------------------------------------------------------------------------------------------------ the recurrence
// A wavefront (a workgroup of its own) owns GLA_COLS columns of one (entry, head): lane = column + GLA_COLS * row
// group, and row group g of the four holds the rows d = g * RPL .. g * RPL + RPL - 1 of its column in registers (rows
// past dim are padding that stays zero).  The tokens' alpha, k and scaled q of the head go through LDS STAGE tokens at
// a time, laid out so that a lane reads its rows four at a time; the next tokens' values are asked of memory before
// the staged ones are worked on, so a token costs no memory latency.  Per token a lane updates its rows, sums its share
// of o, and the row groups' shares are added by two lane exchanges, always in the same order.
#define GLA_COLS 16
#define GLA_GROUPS 4

typedef __attribute__((ext_vector_type(4))) float gla_f32x4;

template <typename T, int RPL>
__global__ void __launch_bounds__(64)
gla_scan_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, int64_t row_stride,
                const float* __restrict__ alpha, const int* __restrict__ entry_start,
                const int* __restrict__ state_slots, float* __restrict__ state, int heads, int dim, int vdim,
                float q_scale, float* __restrict__ o) {
    constexpr int STAGE = RPL <= 16 ? 16 : (RPL <= 32 ? 8 : 4);       // tokens staged at a time
    constexpr int ROWS = GLA_GROUPS * RPL;                             // padded rows of a head
    constexpr int PER_LANE = STAGE * ROWS / 64;                        // staged elements of each array a lane moves
    __shared__ __attribute__((aligned(16))) float sa[STAGE * ROWS];
    __shared__ __attribute__((aligned(16))) float sk[STAGE * ROWS];
    __shared__ __attribute__((aligned(16))) float sq[STAGE * ROWS];
    const int e = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int col = blockIdx.z * GLA_COLS + (lane % GLA_COLS), group = lane / GLA_COLS;
    const bool live = col < vdim;
    const int t0 = entry_start[e], t1 = entry_start[e + 1];
    float* S = state + (((int64_t)state_slots[e] * heads + h) * dim) * (int64_t)vdim;
    float s[RPL];
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
        const int d = group * RPL + i;
        s[i] = (live && d < dim) ? S[(int64_t)d * vdim + col] : 0.f;
    }
    float na[PER_LANE], nk[PER_LANE], nq[PER_LANE], nv[STAGE];        // the next tokens, on their way from memory

    auto fetch = [&](int base) {
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j) {
            const int el = lane + 64 * j, tt = el / ROWS, d = el % ROWS, t = base + tt;
            const bool there = t < t1 && d < dim;
            const int64_t at = (int64_t)t * row_stride + (int64_t)h * dim + d;
            na[j] = there ? alpha[((int64_t)t * heads + h) * dim + d] : 0.f;
            nk[j] = there ? to_float(k[at]) : 0.f;
            nq[j] = there ? to_float(q[at]) * q_scale : 0.f;
        }
#pragma unroll
        for (int tt = 0; tt < STAGE; ++tt)
            nv[tt] = (live && base + tt < t1) ? to_float(v[(int64_t)(base + tt) * row_stride + (int64_t)h * vdim + col]) : 0.f;
    };

    if (t0 < t1) fetch(t0);
    for (int base = t0; base < t1; base += STAGE) {
        const int count = min(STAGE, t1 - base);
        float vt[STAGE];
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j) {
            sa[lane + 64 * j] = na[j];
            sk[lane + 64 * j] = nk[j];
            sq[lane + 64 * j] = nq[j];
        }
#pragma unroll
        for (int tt = 0; tt < STAGE; ++tt) vt[tt] = nv[tt];
        __syncthreads();                           // one wavefront a workgroup: its stores to LDS before its reads
        if (base + STAGE < t1) fetch(base + STAGE);
#pragma unroll
        for (int tt = 0; tt < STAGE; ++tt) {
            if (tt < count) {
                const float* a = sa + tt * ROWS + group * RPL;
                const float* kk = sk + tt * ROWS + group * RPL;
                const float* qq = sq + tt * ROWS + group * RPL;
                float acc = 0.f;
#pragma unroll
                for (int i = 0; i < RPL; i += 4) {
                    const gla_f32x4 a4 = *reinterpret_cast<const gla_f32x4*>(a + i);
                    const gla_f32x4 k4 = *reinterpret_cast<const gla_f32x4*>(kk + i);
                    const gla_f32x4 q4 = *reinterpret_cast<const gla_f32x4*>(qq + i);
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        s[i + x] = fmaf(a4[x], s[i + x], k4[x] * vt[tt]);
                        acc = fmaf(s[i + x], q4[x], acc);
                    }
                }
                acc += __shfl_xor(acc, GLA_COLS, 64);
                acc += __shfl_xor(acc, 2 * GLA_COLS, 64);
                if (live && group == 0) o[((int64_t)(base + tt) * heads + h) * vdim + col] = acc;
            }
        }
        __syncthreads();                           // the reads, before the next tokens are staged
    }
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
        const int d = group * RPL + i;
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
    const int rpl = ceil_div(dim, GLA_GROUPS);
#define GLA_LAUNCH(T, R)                                                                                              \
    hipLaunchKernelGGL((gla_scan_kernel<T, R>), grid, dim3(64), 0, stream, (const T*)q, (const T*)k, (const T*)v,     \
                       row_stride, alpha, entry_start, state_slots, state, heads, dim, vdim, q_scale, o)
#define GLA_BY_ROWS(T)                                                                                                \
    do {                                                                                                              \
        if (rpl <= 4) GLA_LAUNCH(T, 4);                                                                               \
        else if (rpl <= 8) GLA_LAUNCH(T, 8);                                                                          \
        else if (rpl <= 12) GLA_LAUNCH(T, 12);                                                                        \
        else if (rpl <= 16) GLA_LAUNCH(T, 16);                                                                        \
        else if (rpl <= 24) GLA_LAUNCH(T, 24);                                                                        \
        else if (rpl <= 32) GLA_LAUNCH(T, 32);                                                                        \
        else if (rpl <= 48) GLA_LAUNCH(T, 48);                                                                        \
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
