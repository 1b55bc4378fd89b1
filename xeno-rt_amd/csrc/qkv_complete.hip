// What lies between an attention's projection and its scores, for projections whose sums come in float32:
// biases, an RMS norm of every head of q and k (one weight [head_dim] for all heads), a rotation of pairs of dims by
// angles position * frequency[pair] with a table of frequencies of the caller's making (pairs of neighbours 2n, 2n + 1 or
// of halves n, n + rot_dims / 2; the first rot_dims dims of a head, the rest pass; cosines and sines times `magnitude`),
// a blend of the values with those of another layer, v <- (1 - lambda) v + lambda v_other, and the write of keys and
// values into the paged cache. Further options: a head norm without a gain (plain_norm), a query temperature (the queries of
// the token at position p times 1 + coef * ln(floor((p + 1) / every) + 1), after norm and rotation), and rows that hold
// queries only (queries_only: the layer reads another layer's keys and values). One wavefront per (token, head) of q, k and v; the head passes through LDS so that a
// lane finds its pair's other half there. Everything is float32 until the one rounding to the element type.
#include "cache_layout.h"
#include "xrt_hip.h"

namespace {

constexpr int COMPLETE_MAX_DIM = 512;

struct CompleteArgs {
    const float* proj; long proj_stride;          // rows [q heads | k heads | v heads | ...] of float32 sums
    int n_heads, n_kv_heads, head_dim, value_dim;
    const void* bias_q; const void* bias_k; const void* bias_v;           // [heads * dim] each, or null
    const void* norm_q; const void* norm_k; float norm_eps;               // [head_dim] each, or null
    int small_dtype;                                                      // element type of biases, norm weights and lambda
    const float* frequencies; int rot_dims; int neighbours; float magnitude;    // [rot_dims / 2], or null
    const float* values_in; float* values_out; const void* lambda;        // [tokens][n_kv_heads * value_dim] float32 each, or null
    const int* positions; const int* slots;
    void* q_out; long q_stride;                                           // rows of n_heads * head_dim of the element type
    void* k_cache; void* v_cache; const int* block_table; int table_stride; int n_blocks;
    int plain_norm; float temp_coef; int temp_every; int queries_only;
};

__device__ __forceinline__ float small(const void* p, int dtype, int i) {
    return dtype == XRT_F32 ? ((const float*)p)[i] : to_float(((const bf16*)p)[i]);
}

template <typename T>
__global__ void __launch_bounds__(XRT_WAVE) qkv_complete_kernel(const CompleteArgs a) {
    __shared__ float head[COMPLETE_MAX_DIM];
    const int lane = threadIdx.x;
    const int per_token = a.queries_only ? a.n_heads : a.n_heads + 2 * a.n_kv_heads;
    const long token = blockIdx.x / per_token;
    const int which = blockIdx.x % per_token;
    const int slot = a.slots[token], pos = a.positions[token];
    const float* row = a.proj + token * a.proj_stride;
    const int q_width = a.n_heads * a.head_dim, k_width = a.n_kv_heads * a.head_dim;

    if (which >= a.n_heads + a.n_kv_heads) {                   // ---- a head of v
        const int kv_head = which - a.n_heads - a.n_kv_heads;
        if (slot < 0) return;
        const int block = a.v_cache != nullptr ? a.block_table[(long)slot * a.table_stride + pos / XRT_BLOCK_TOKENS] : -1;
        const bool cached = block >= 0 && block < a.n_blocks;
        const long base = ((long)block * a.n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * a.value_dim;
        const float lam = a.values_in ? small(a.lambda, a.small_dtype, 0) : 0.f;
        for (int e = lane; e < a.value_dim; e += XRT_WAVE) {
            const int column = kv_head * a.value_dim + e;
            float v = row[q_width + k_width + column];
            if (a.bias_v) v += small(a.bias_v, a.small_dtype, column);
            const long shared = token * ((long)a.n_kv_heads * a.value_dim) + column;
            if (a.values_out) a.values_out[shared] = v;
            if (a.values_in) v = fmaf(lam, a.values_in[shared], (1.0f - lam) * v);
            if (cached) ((T*)a.v_cache)[base + cache_value_offset(e, pos % XRT_BLOCK_TOKENS, a.value_dim)] = from_float<T>(v);
        }
        return;
    }

    // ---- a head of q or k
    const bool is_q = which < a.n_heads;
    const int index = is_q ? which : which - a.n_heads;
    const int column0 = (is_q ? 0 : q_width) + index * a.head_dim;
    T* q_dst = is_q ? (T*)a.q_out + token * a.q_stride + (long)index * a.head_dim : nullptr;
    if (slot < 0) {
        if (is_q) for (int e = lane; e < a.head_dim; e += XRT_WAVE) q_dst[e] = from_float<T>(0.f);
        return;
    }
    const void* bias = is_q ? a.bias_q : a.bias_k;
    const void* gain = is_q ? a.norm_q : a.norm_k;
    float squares = 0.f;
    for (int e = lane; e < a.head_dim; e += XRT_WAVE) {
        float v = row[column0 + e];
        if (bias) v += small(bias, a.small_dtype, index * a.head_dim + e);
        head[e] = v;
        squares = fmaf(v, v, squares);
    }
    if (gain || a.plain_norm) {
        const float inv = 1.0f / sqrtf(wave_sum(squares) / (float)a.head_dim + a.norm_eps);
        for (int e = lane; e < a.head_dim; e += XRT_WAVE) head[e] = gain ? head[e] * inv * small(gain, a.small_dtype, e) : head[e] * inv;
    }
    const float temperature = is_q && a.temp_every > 0 ? 1.0f + a.temp_coef * logf((float)((pos + 1) / a.temp_every + 1)) : 1.0f;
    wave_sync();
    long base = -1;
    if (!is_q && a.k_cache != nullptr) {
        const int block = a.block_table[(long)slot * a.table_stride + pos / XRT_BLOCK_TOKENS];
        if (block >= 0 && block < a.n_blocks) base = ((long)block * a.n_kv_heads + index) * XRT_BLOCK_TOKENS * a.head_dim;
    }
    const int half = a.rot_dims / 2;
    for (int e = lane; e < a.head_dim; e += XRT_WAVE) {
        float v = head[e];
        if (a.frequencies != nullptr && e < a.rot_dims) {
            // the pair (first, second) turns to (first cos - second sin, second cos + first sin)
            const int pair = a.neighbours ? e / 2 : e % half;
            const bool is_first = a.neighbours ? e % 2 == 0 : e < half;
            const float other = head[a.neighbours ? e ^ 1 : (is_first ? e + half : e - half)];
            float sine, cosine;
            sincosf((float)pos * a.frequencies[pair], &sine, &cosine);
            sine *= a.magnitude;
            cosine *= a.magnitude;
            v = is_first ? v * cosine - other * sine : v * cosine + other * sine;
        }
        if (is_q) q_dst[e] = from_float<T>(v * temperature);
        else if (base >= 0) ((T*)a.k_cache)[base + cache_key_offset(pos % XRT_BLOCK_TOKENS, e, a.head_dim)] = from_float<T>(v);
    }
}

}  // namespace

extern "C" int xrt_qkv_complete(const float* proj, long proj_stride, int dtype, long tokens, int n_heads, int n_kv_heads, int head_dim,
                              int value_dim, const void* bias_q, const void* bias_k, const void* bias_v, const void* norm_q,
                              const void* norm_k, float norm_eps, int small_dtype, const float* frequencies, int rot_dims,
                              int neighbours, float magnitude, const float* values_in, float* values_out, const void* lambda,
                              const int* positions, const int* slots, void* q_out, long q_stride, void* k_cache, void* v_cache,
                              const int* block_table, int table_stride, int n_blocks, int plain_norm, float temp_coef, int temp_every,
                              int queries_only, void* stream) {
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "qkv_complete: unknown dtype %d", dtype);
    XRT_REQUIRE(temp_every >= 0 && (!plain_norm || norm_q == nullptr), "qkv_complete: a negative stretch of the query temperature, or a plain norm beside gains");
    XRT_REQUIRE(!queries_only || (k_cache == nullptr && values_in == nullptr && values_out == nullptr), "qkv_complete: queries only, and keys or values to write");
    XRT_REQUIRE(small_dtype == XRT_F32 || small_dtype == XRT_BF16, "qkv_complete: unknown dtype %d of the small tensors", small_dtype);
    XRT_REQUIRE(proj && positions && slots && q_out, "qkv_complete: null operand");
    XRT_REQUIRE(tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0 && head_dim > 0 && value_dim > 0,
                "qkv_complete: bad head counts or sizes");
    XRT_REQUIRE(head_dim <= COMPLETE_MAX_DIM, "qkv_complete: heads of up to %d dims", COMPLETE_MAX_DIM);
    XRT_REQUIRE(proj_stride >= (long)n_heads * head_dim + (queries_only ? 0L : (long)n_kv_heads * (head_dim + value_dim)) && q_stride >= (long)n_heads * head_dim,
                "qkv_complete: a row stride is shorter than its heads");
    XRT_REQUIRE((norm_q == nullptr) == (norm_k == nullptr), "qkv_complete: the norms of q and k come together");
    XRT_REQUIRE(frequencies == nullptr || (rot_dims > 0 && rot_dims % 2 == 0 && rot_dims <= head_dim),
                "qkv_complete: %d rotated dims of a head of %d", rot_dims, head_dim);
    XRT_REQUIRE(values_in == nullptr || lambda != nullptr, "qkv_complete: values to blend in need their share");
    XRT_REQUIRE((k_cache == nullptr) == (v_cache == nullptr) && (k_cache == nullptr || (block_table && table_stride > 0 && n_blocks > 0)),
                "qkv_complete: a cache to write needs keys, values and a block table");
    XRT_REQUIRE(tokens * (n_heads + 2 * n_kv_heads) < (1L << 31), "qkv_complete: too many (token, head) pairs");
    if (tokens == 0) return 0;
    const CompleteArgs a{proj, proj_stride, n_heads, n_kv_heads, head_dim, value_dim, bias_q, bias_k, bias_v, norm_q, norm_k, norm_eps,
                       small_dtype, frequencies, rot_dims, neighbours, magnitude, values_in, values_out, lambda, positions, slots,
                       q_out, q_stride, k_cache, v_cache, block_table, table_stride, n_blocks, plain_norm, temp_coef, temp_every, queries_only};
    const unsigned items = (unsigned)(tokens * (queries_only ? n_heads : n_heads + 2 * n_kv_heads));
    if (dtype == XRT_F32) qkv_complete_kernel<float><<<items, XRT_WAVE, 0, (hipStream_t)stream>>>(a);
    else qkv_complete_kernel<bf16><<<items, XRT_WAVE, 0, (hipStream_t)stream>>>(a);
    XRT_LAUNCH_CHECK("qkv_complete");
    return 0;
}
