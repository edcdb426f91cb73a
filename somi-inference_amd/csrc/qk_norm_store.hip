// Query and key norm over a whole projection, with the keys (and the values) into their pages.
//
// A token's row holds its nq query heads, then its nkv key heads (and, unless the values are the keys, nkv value
// heads), each of D channels.  q is divided by the root mean square of ALL its nq * D values (eps inside the root)
// and multiplied by a weight of that size, in place; k likewise over its nkv * D values, and the normed k goes into
// the key pages [pages, nkv, page, D].  The value pages [pages, nkv, D, page] get the token's values: the value heads
// of the row, or, with TIED, the keys as they were projected, before the norm.  A token whose slot is negative (a
// padding row) stores nothing.  Sums and the scaling are float32.
#include "common.h"

template <typename T, bool TIED>
__global__ void __launch_bounds__(256)
qk_norm_store_kernel(T* __restrict__ rows, int64_t row_stride, const int* __restrict__ slots,
                     const float* __restrict__ wq, const float* __restrict__ wk, float eps, int nq, int nkv, int D,
                     T* __restrict__ k_cache, T* __restrict__ v_cache, int page_size) {
    __shared__ float red[16];
    const int64_t t = blockIdx.x;
    T* q = rows + t * row_stride;
    T* k = q + (int64_t)nq * D;
    const T* v = TIED ? k : k + (int64_t)nkv * D;
    const int qn = nq * D, kn = nkv * D;
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < qn; i += 256) {
        const float x = to_float(q[i]);
        sq += x * x;
    }
    for (int i = threadIdx.x; i < kn; i += 256) {
        const float x = to_float(k[i]);
        sk += x * x;
    }
    sq = block_sum<256>(sq, red);
    sk = block_sum<256>(sk, red);
    const float iq = 1.0f / sqrtf(sq / (float)qn + eps), ik = 1.0f / sqrtf(sk / (float)kn + eps);
    for (int i = threadIdx.x; i < qn; i += 256) q[i] = from_float<T>(to_float(q[i]) * iq * wq[i]);
    const int slot = slots[t];
    if (slot < 0) return;
    const int64_t page = slot / page_size;
    const int off = slot - (int)page * page_size;
    for (int i = threadIdx.x; i < kn; i += 256) {
        const int g = i / D, d = i - g * D;
        v_cache[((page * nkv + g) * D + d) * page_size + off] = v[i];
        k_cache[((page * nkv + g) * page_size + off) * D + d] = from_float<T>(to_float(k[i]) * ik * wk[i]);
    }
}

extern "C" int somi_qk_norm_store(void* rows, int dtype, int64_t row_stride, const int* slots, const float* wq,
                                  const float* wk, float eps, int n_tokens, int nq, int nkv, int head_dim, int tied,
                                  void* k_cache, void* v_cache, int page_size, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && nq > 0 && nkv > 0 && head_dim > 0 && page_size > 0, "qk_norm_store: bad sizes");
    SOMI_REQUIRE(row_stride >= (int64_t)(nq + (tied ? 1 : 2) * nkv) * head_dim, "qk_norm_store: rows of %lld are too narrow",
                 (long long)row_stride);
    if (n_tokens == 0) return 0;
#define SOMI_QKN(T, TIED)                                                                                            \
    hipLaunchKernelGGL((qk_norm_store_kernel<T, TIED>), dim3(n_tokens), dim3(256), 0, stream, (T*)rows, row_stride, slots, \
                       wq, wk, eps, nq, nkv, head_dim, (T*)k_cache, (T*)v_cache, page_size)
    if (dtype == SOMI_F32) {
        if (tied) SOMI_QKN(float, true); else SOMI_QKN(float, false);
    } else if (dtype == SOMI_BF16) {
        if (tied) SOMI_QKN(bf16, true); else SOMI_QKN(bf16, false);
    } else {
        return somi_fail("qk_norm_store: unknown dtype %d", dtype);
    }
#undef SOMI_QKN
    SOMI_LAUNCH_CHECK("qk_norm_store");
    return 0;
}
