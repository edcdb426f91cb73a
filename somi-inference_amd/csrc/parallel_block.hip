// Kernels of the parallel block arrangement (one norm, mixer and feed-forward side by side, a scaled residual add),
// of the norm without statistics, of the join of two mixers and of the per-layer token input.
//
//   dynamic tanh        y = tanh(alpha x) w + b                       (alpha: one number, on the device)
//   scaled add          h += m (a + b); optionally a copy of the new h in the compute dtype
//   normed pair mean    y = (l / rms(l) wl + r / rms(r) wr) / 2       (float32 out)
//   normed add          h += m y / rms(y) w
//   gated table rows    y[t, c] = gelu_tanh(g[t, c]) table[id[t], offset + c]
//
// rms(x) = sqrt(mean(x^2) + eps).  All sums and the residual stream are float32.
#include "common.h"

template <typename TO>
__global__ void __launch_bounds__(256)
dyt_kernel(const float* __restrict__ h, const float* __restrict__ w, const float* __restrict__ b,
           const float* __restrict__ alpha, TO* __restrict__ out, int hidden) {
    const int64_t row = blockIdx.x;
    const float a = alpha[0];
    for (int i = threadIdx.x; i < hidden; i += 256)
        out[row * hidden + i] = from_float<TO>(tanhf(a * h[row * hidden + i]) * w[i] + b[i]);
}

extern "C" int somi_dyt(const float* h, const float* w, const float* b, const float* alpha, void* out, int dtype,
                        int n_rows, int hidden, hipStream_t stream) {
    SOMI_REQUIRE(n_rows >= 0 && hidden > 0, "dyt: bad sizes rows=%d hidden=%d", n_rows, hidden);
    if (n_rows == 0) return 0;
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(dyt_kernel<float>, dim3(n_rows), dim3(256), 0, stream, h, w, b, alpha, (float*)out, hidden);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(dyt_kernel<bf16>, dim3(n_rows), dim3(256), 0, stream, h, w, b, alpha, (bf16*)out, hidden);
    else
        return somi_fail("dyt: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("dyt");
    return 0;
}

// h += m (a + b); b may be null; COPY: the new h also leaves in TO.
template <typename TO, bool COPY>
__global__ void __launch_bounds__(256)
scaled_add_kernel(float* __restrict__ h, const float* __restrict__ a, const float* __restrict__ b, float m,
                  TO* __restrict__ copy, int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) {
        float delta = a[i];
        if (b != nullptr) delta += b[i];
        const float v = h[i] + m * delta;
        h[i] = v;
        if (COPY) copy[i] = from_float<TO>(v);
    }
}

extern "C" int somi_scaled_add(float* h, const float* a, const float* b, float m, void* copy, int copy_dtype,
                               int64_t count, hipStream_t stream) {
    SOMI_REQUIRE(count >= 0, "scaled_add: bad count");
    if (count == 0) return 0;
    const int grid = (int)(ceil_div64(count, 256) < 65536 ? ceil_div64(count, 256) : 65536);
    if (copy == nullptr)
        hipLaunchKernelGGL((scaled_add_kernel<float, false>), dim3(grid), dim3(256), 0, stream, h, a, b, m, (float*)nullptr, count);
    else if (copy_dtype == SOMI_F32)
        hipLaunchKernelGGL((scaled_add_kernel<float, true>), dim3(grid), dim3(256), 0, stream, h, a, b, m, (float*)copy, count);
    else if (copy_dtype == SOMI_BF16)
        hipLaunchKernelGGL((scaled_add_kernel<bf16, true>), dim3(grid), dim3(256), 0, stream, h, a, b, m, (bf16*)copy, count);
    else
        return somi_fail("scaled_add: unknown dtype %d", copy_dtype);
    SOMI_LAUNCH_CHECK("scaled_add");
    return 0;
}

// One workgroup per row: both rows' sums of squares, then the mean of the two normed rows.
template <typename T>
__global__ void __launch_bounds__(256)
normed_pair_mean_kernel(const T* __restrict__ l, const T* __restrict__ r, const float* __restrict__ wl,
                        const float* __restrict__ wr, float eps, float* __restrict__ out, int width) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    float sl = 0.f, sr = 0.f;
    for (int i = threadIdx.x; i < width; i += 256) {
        const float a = to_float(l[row * width + i]), b = to_float(r[row * width + i]);
        sl += a * a;
        sr += b * b;
    }
    sl = block_sum<256>(sl, red);
    sr = block_sum<256>(sr, red);
    const float il = 1.0f / sqrtf(sl / (float)width + eps), ir = 1.0f / sqrtf(sr / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += 256) {
        const float a = to_float(l[row * width + i]) * il * wl[i], b = to_float(r[row * width + i]) * ir * wr[i];
        out[row * width + i] = 0.5f * (a + b);
    }
}

extern "C" int somi_normed_pair_mean(const void* l, const void* r, int dtype, const float* wl, const float* wr, float eps,
                                     float* out, int n_rows, int width, hipStream_t stream) {
    SOMI_REQUIRE(n_rows >= 0 && width > 0, "normed_pair_mean: bad sizes");
    if (n_rows == 0) return 0;
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(normed_pair_mean_kernel<float>, dim3(n_rows), dim3(256), 0, stream, (const float*)l,
                           (const float*)r, wl, wr, eps, out, width);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(normed_pair_mean_kernel<bf16>, dim3(n_rows), dim3(256), 0, stream, (const bf16*)l,
                           (const bf16*)r, wl, wr, eps, out, width);
    else
        return somi_fail("normed_pair_mean: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("normed_pair_mean");
    return 0;
}

// h += m y / rms(y) w; COPY: the new h also leaves in TO.
template <typename TO, bool COPY>
__global__ void __launch_bounds__(256)
normed_add_kernel(float* __restrict__ h, const float* __restrict__ y, const float* __restrict__ w, float eps, float m,
                  TO* __restrict__ copy, int width) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += 256) {
        const float v = y[row * width + i];
        ss += v * v;
    }
    ss = block_sum<256>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += 256) {
        const float v = h[row * width + i] + m * (y[row * width + i] * inv * w[i]);
        h[row * width + i] = v;
        if (COPY) copy[row * width + i] = from_float<TO>(v);
    }
}

extern "C" int somi_normed_add(float* h, const float* y, const float* w, float eps, float m, void* copy, int copy_dtype,
                               int n_rows, int width, hipStream_t stream) {
    SOMI_REQUIRE(n_rows >= 0 && width > 0, "normed_add: bad sizes");
    if (n_rows == 0) return 0;
    if (copy == nullptr)
        hipLaunchKernelGGL((normed_add_kernel<float, false>), dim3(n_rows), dim3(256), 0, stream, h, y, w, eps, m, (float*)nullptr, width);
    else if (copy_dtype == SOMI_F32)
        hipLaunchKernelGGL((normed_add_kernel<float, true>), dim3(n_rows), dim3(256), 0, stream, h, y, w, eps, m, (float*)copy, width);
    else if (copy_dtype == SOMI_BF16)
        hipLaunchKernelGGL((normed_add_kernel<bf16, true>), dim3(n_rows), dim3(256), 0, stream, h, y, w, eps, m, (bf16*)copy, width);
    else
        return somi_fail("normed_add: unknown dtype %d", copy_dtype);
    SOMI_LAUNCH_CHECK("normed_add");
    return 0;
}

// y[t, c] = gelu_tanh(g[t, c]) * table[id[t], offset + c] for c < dim.
template <typename T>
__global__ void __launch_bounds__(256)
gated_table_rows_kernel(const T* __restrict__ g, const T* __restrict__ table, const int* __restrict__ ids, int vocab,
                        int table_width, int offset, int dim, T* __restrict__ out, int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) {
        const int64_t t = i / dim;
        const int c = (int)(i - t * dim);
        int id = ids[t];
        id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
        const float z = to_float(g[i]);
        const float act = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
        out[i] = from_float<T>(act * to_float(table[(int64_t)id * table_width + offset + c]));
    }
}

extern "C" int somi_gated_table_rows(const void* g, const void* table, int dtype, const int* ids, int vocab, int table_width,
                                     int offset, int dim, void* out, int n_tokens, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && dim > 0 && vocab > 0 && offset >= 0 && offset + dim <= table_width,
                 "gated_table_rows: columns %d..%d do not fit a table %d wide", offset, offset + dim, table_width);
    if (n_tokens == 0) return 0;
    const int64_t count = (int64_t)n_tokens * dim;
    const int grid = (int)(ceil_div64(count, 256) < 65536 ? ceil_div64(count, 256) : 65536);
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(gated_table_rows_kernel<float>, dim3(grid), dim3(256), 0, stream, (const float*)g,
                           (const float*)table, ids, vocab, table_width, offset, dim, (float*)out, count);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(gated_table_rows_kernel<bf16>, dim3(grid), dim3(256), 0, stream, (const bf16*)g,
                           (const bf16*)table, ids, vocab, table_width, offset, dim, (bf16*)out, count);
    else
        return somi_fail("gated_table_rows: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("gated_table_rows");
    return 0;
}

// In place: x *= s (the embedded tokens of a model that scales its embedding).
__global__ void __launch_bounds__(256) scale_kernel(float* __restrict__ x, float s, int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) x[i] *= s;
}

extern "C" int somi_scale_f32(float* x, float s, int64_t count, hipStream_t stream) {
    SOMI_REQUIRE(count >= 0, "scale: bad count");
    if (count == 0) return 0;
    const int grid = (int)(ceil_div64(count, 256) < 65536 ? ceil_div64(count, 256) : 65536);
    hipLaunchKernelGGL(scale_kernel, dim3(grid), dim3(256), 0, stream, x, s, count);
    SOMI_LAUNCH_CHECK("scale");
    return 0;
}
