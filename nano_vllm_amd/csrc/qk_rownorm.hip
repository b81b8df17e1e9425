// Preparation of q, k and v of an attention whose query and key norms run over the whole
// projection, before it is split into heads, and whose positions enter through the length of the
// query only (no rotation):
//
//     q <- q / sqrt(mean(q^2) + eps) * wq * temp(p)        mean over all Hq * D entries of the token's q
//     k <- k / sqrt(mean(k^2) + eps) * wk                  mean over all Hkv * D entries
//     temp(p) = 1 + coef * ln(floor((p + 1) / every) + 1)  (coef 0: no temperature)
//     cache <- k, v                                        at the token's slot (slot < 0: nothing is written)
//
// The row is the packed projection [q | k | v] of Hq * D, Hkv * D and Hkv * DV entries, biases added
// by the product.  Sums of squares, scales, the logarithm and the products are float; q is written
// back in place and k, v into the cache, each rounded once to the element type.  The weights are
// plain (not one-plus), stored as elements or float.
// Cache layout: K [pages, Hkv, page, D], V [pages, Hkv, page / vt, DV, vt] (common.h).
// One workgroup per token.
#include "common.h"

template <typename T>
__global__ void __launch_bounds__(256)
qk_rownorm_store_kernel(T* __restrict__ qkv, int64_t stride, int num_heads, int num_kv_heads, int head_dim, int v_dim,
                        const void* __restrict__ q_weight, const void* __restrict__ k_weight, int w_is_f32, float eps,
                        const int32_t* __restrict__ positions, float temp_coef, int temp_every,
                        const int32_t* __restrict__ slots, T* __restrict__ k_cache, T* __restrict__ v_cache,
                        int page_size) {
    __shared__ float scratch[16];
    const int64_t t = blockIdx.x;
    T* row = qkv + t * stride;
    const int qd = num_heads * head_dim, kd = num_kv_heads * head_dim, vd = num_kv_heads * v_dim;
    const int tid = threadIdx.x;

    float sq = 0.f, sk = 0.f;
    for (int i = tid; i < qd; i += blockDim.x) {
        const float x = to_float(row[i]);
        sq += x * x;
    }
    for (int i = tid; i < kd; i += blockDim.x) {
        const float x = to_float(row[qd + i]);
        sk += x * x;
    }
    sq = block_sum(sq, scratch);
    sk = kd ? block_sum(sk, scratch) : 0.f;

    float q_scale = q_weight ? rsqrtf(sq / (float)qd + eps) : 1.f;
    if (temp_coef != 0.f) {
        const int steps = (positions[t] + 1) / temp_every;
        q_scale *= 1.f + temp_coef * logf((float)steps + 1.f);
    }
    for (int i = tid; i < qd; i += blockDim.x) {
        const float w = !q_weight ? 1.f : w_is_f32 ? static_cast<const float*>(q_weight)[i]
                                                   : to_float(static_cast<const T*>(q_weight)[i]);
        row[i] = from_float<T>(to_float(row[i]) * q_scale * w);
    }
    if (!kd) return;
    const int slot = slots ? slots[t] : -1;
    const float k_scale = k_weight ? rsqrtf(sk / (float)kd + eps) : 1.f;
    const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
    const int vt = nva_v_tile(page_size);
    for (int i = tid; i < kd; i += blockDim.x) {
        const float w = !k_weight ? 1.f : w_is_f32 ? static_cast<const float*>(k_weight)[i]
                                                   : to_float(static_cast<const T*>(k_weight)[i]);
        const T k = from_float<T>(to_float(row[qd + i]) * k_scale * w);
        row[qd + i] = k;
        if (slot >= 0 && k_cache) {
            const int g = i / head_dim, d = i % head_dim;
            k_cache[(((int64_t)page * num_kv_heads + g) * page_size + off) * head_dim + d] = k;
        }
    }
    if (slot >= 0 && v_cache) {
        for (int i = tid; i < vd; i += blockDim.x) {
            const int g = i / v_dim, d = i % v_dim;
            v_cache[((int64_t)page * num_kv_heads + g) * v_dim * (int64_t)page_size + nva_v_offset(off, d, v_dim, vt)] =
                row[qd + kd + i];
        }
    }
}

// qkv: [tokens, Hq * D + Hkv * D + Hkv * DV] with rows `stride` elements apart, q and k rewritten in place.
// q_weight [Hq * D], k_weight [Hkv * D]: both or none.  positions are needed with a temperature.
// slots (with the caches) may be null: nothing is stored then.  num_kv_heads 0: the row holds q only.
NVA_EXPORT int NVA_NAME(nva_qk_rownorm_store)(void* qkv, int64_t stride, int64_t tokens, int num_heads, int num_kv_heads,
                                              int head_dim, int v_dim, const void* q_weight, const void* k_weight,
                                              int w_is_f32, float eps, const int32_t* positions, float temp_coef,
                                              int temp_every, const int32_t* slots, void* k_cache, void* v_cache,
                                              int page_size, hipStream_t stream) {
    if (tokens == 0) return 0;
    if (tokens < 0 || tokens > 0x7fffffff) return nva_fail("qk_rownorm_store: bad token count %lld", (long long)tokens);
    if (num_heads <= 0 || num_kv_heads < 0 || head_dim <= 0 || v_dim <= 0)
        return nva_fail("qk_rownorm_store: bad sizes heads=%d kv_heads=%d head_dim=%d v_dim=%d", num_heads, num_kv_heads,
                        head_dim, v_dim);
    const int64_t width = (int64_t)(num_heads + num_kv_heads) * head_dim + (int64_t)num_kv_heads * v_dim;
    if (stride < width) return nva_fail("qk_rownorm_store: rows of %lld elements are %lld apart", (long long)width, (long long)stride);
    if (num_kv_heads && (q_weight == nullptr) != (k_weight == nullptr))
        return nva_fail("qk_rownorm_store: give both norm weights or none");
    if (temp_coef != 0.f && (!positions || temp_every <= 0))
        return nva_fail("qk_rownorm_store: a query temperature needs positions and a positive step");
    if ((k_cache || v_cache) && (!k_cache || !v_cache || !slots || page_size <= 0 || !num_kv_heads))
        return nva_fail("qk_rownorm_store: storing needs both caches, the slots and the page size");
    hipLaunchKernelGGL((qk_rownorm_store_kernel<elem_t>), dim3((unsigned)tokens), dim3(256), 0, stream, (elem_t*)qkv,
                       stride, num_heads, num_kv_heads, head_dim, v_dim, q_weight, k_weight, w_is_f32, eps, positions,
                       temp_coef, temp_every, slots, (elem_t*)k_cache, (elem_t*)v_cache, page_size);
    return nva_check_launch("qk_rownorm_store");
}

NVA_DEFINE_LAST_ERROR(nva_qk_rownorm)
