// What a token brings beside its embedding row, and small operations on the residual stream and on a product's sums:
//   xrt_bigram_add      x <- x * scale + table[row], the row hashed from the token and the one before it; the token before a
//                       step's first is kept per sequence
//   xrt_gated_rows      out[t][c] = gelu_tanh(s[t][c]) * table[ids[t]][offset + c]: a slice of a token's row of a table, gated
//   xrt_add_weighted    residual += sum of scale_n * gain_n * y_n over up to four float32 matrices (gains per column, or none);
//                       the updated rows may be written once more in another element type, for a product that reads them
//   xrt_glu_clamped     out = g' * sigmoid(alpha g') * (u' + 1) with g' = min(g, limit), u' = clamp(u, -limit, limit), from
//                       float32 sums [rows][2 n] that hold g then u; times a weight per row, if given
//   xrt_softcap         x <- cap * tanh(x / cap), in place on float32
//   xrt_cast            out = x in another element type
// All arithmetic is float32. Tokens whose slot is negative are padding: they are computed like any other and touch no state.
#include "common.h"
#include "xrt_hip.h"

namespace {

__device__ __forceinline__ float load_as_float(const void* p, int dtype, long i) {
    return dtype == XRT_F32 ? ((const float*)p)[i] : to_float(((const bf16*)p)[i]);
}
__device__ __forceinline__ void store_from_float(void* p, int dtype, long i, float v) {
    if (dtype == XRT_F32) ((float*)p)[i] = v; else ((bf16*)p)[i] = from_float<bf16>(v);
}

// The row of the hashed table for the token at packed place t: `buckets` (the table's last row) for a sequence's first token.
__device__ __forceinline__ int bigram_row(const int* __restrict__ ids, const int* __restrict__ positions, const int* __restrict__ slots,
                                          const int* __restrict__ before, long t, int buckets, int mul_prev, int mul_cur) {
    const int pos = positions[t], slot = slots[t];
    if (pos <= 0) return buckets;
    int prev;
    if (t > 0 && slots[t - 1] == slot && positions[t - 1] == pos - 1) prev = ids[t - 1];     // the step brings the token before as well
    else prev = slot >= 0 ? before[slot] : 0;
    const long hashed = (long)prev * mul_prev + (long)ids[t] * mul_cur;
    return (int)(hashed % buckets);
}

__global__ void __launch_bounds__(256) bigram_add_kernel(float* __restrict__ x, int width, float scale, const void* __restrict__ table, int dtype,
                                                         const int* __restrict__ ids, const int* __restrict__ positions,
                                                         const int* __restrict__ slots, const int* __restrict__ before, int buckets,
                                                         int mul_prev, int mul_cur) {
    const long t = blockIdx.x;
    const bool hashed = table != nullptr;
    const long row = hashed ? bigram_row(ids, positions, slots, before, t, buckets, mul_prev, mul_cur) : 0;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        float v = x[t * width + c] * scale;
        if (hashed) v += load_as_float(table, dtype, row * width + c);
        x[t * width + c] = v;
    }
}

// after the rows are made: every sequence's last token of the step is the one before its next step's first
__global__ void bigram_keep_kernel(const int* __restrict__ ids, const int* __restrict__ seq_offsets, const int* __restrict__ seq_slots,
                                   int n_seqs, int* __restrict__ before) {
    const int seq = blockIdx.x * blockDim.x + threadIdx.x;
    if (seq >= n_seqs) return;
    const int slot = seq_slots[seq], end = seq_offsets[seq + 1];
    if (slot < 0 || end <= seq_offsets[seq]) return;
    before[slot] = ids[end - 1];
}

__device__ __forceinline__ float gelu_tanh(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

__global__ void gated_rows_kernel(const float* __restrict__ s, long s_stride, const void* __restrict__ table, int table_dtype, long table_width,
                                  long offset, int rows, const int* __restrict__ ids, void* __restrict__ out, int out_dtype, long tokens, int width) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= tokens * width) return;
    const long t = i / width;
    const int c = (int)(i % width), id = ids[t];
    const float e = id >= 0 && id < rows ? load_as_float(table, table_dtype, (long)id * table_width + offset + c) : 0.f;
    store_from_float(out, out_dtype, i, gelu_tanh(s[t * s_stride + c]) * e);
}

struct WeightedTerms {
    const float* y[4];
    const void* gain[4];
    float scale[4];
    int count, gain_dtype;
};

__global__ void add_weighted_kernel(float* __restrict__ residual, WeightedTerms terms, long count, int width, void* __restrict__ copy, int copy_dtype) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    const int c = (int)(i % width);
    float sum = 0.f;
#pragma unroll
    for (int n = 0; n < 4; ++n) {
        if (n < terms.count) {
            float v = terms.y[n][i] * terms.scale[n];
            if (terms.gain[n] != nullptr) v *= load_as_float(terms.gain[n], terms.gain_dtype, c);
            sum += v;
        }
    }
    const float updated = residual[i] + sum;
    residual[i] = updated;
    if (copy != nullptr) store_from_float(copy, copy_dtype, i, updated);
}

__device__ __forceinline__ float glu_clamped_of(float gate, float up, float limit, float alpha) {
    const float g = fminf(gate, limit);
    const float u = fminf(fmaxf(up, -limit), limit);
    return g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
}

__global__ void glu_clamped_kernel(const float* __restrict__ sums, void* __restrict__ out, int out_dtype, long rows, int n, float limit, float alpha,
                                   const float* __restrict__ row_weights) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * n) return;
    const long r = i / n;
    const int c = (int)(i % n);
    const float weight = row_weights != nullptr ? row_weights[r] : 1.0f;
    store_from_float(out, out_dtype, i, glu_clamped_of(sums[r * 2 * n + c], sums[r * 2 * n + n + c], limit, alpha) * weight);
}

// the same, four columns a thread (n a multiple of four: sixteen bytes a load)
__global__ void __launch_bounds__(256) glu_clamped_four_kernel(const float* __restrict__ sums, void* __restrict__ out, int out_dtype, long rows, int n,
                                                              float limit, float alpha, const float* __restrict__ row_weights) {
    const long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= rows * n) return;
    const long r = i / n;
    const int c = (int)(i % n);
    const float4 gate = *reinterpret_cast<const float4*>(sums + r * 2 * n + c), up = *reinterpret_cast<const float4*>(sums + r * 2 * n + n + c);
    const float weight = row_weights != nullptr ? row_weights[r] : 1.0f;
    const float made[4] = {glu_clamped_of(gate.x, up.x, limit, alpha) * weight, glu_clamped_of(gate.y, up.y, limit, alpha) * weight,
                           glu_clamped_of(gate.z, up.z, limit, alpha) * weight, glu_clamped_of(gate.w, up.w, limit, alpha) * weight};
    if (out_dtype == XRT_F32) {
        *reinterpret_cast<float4*>((float*)out + i) = make_float4(made[0], made[1], made[2], made[3]);
    } else {
        struct alignas(8) Four { bf16 e[4]; } four;
#pragma unroll
        for (int e = 0; e < 4; ++e) four.e[e] = from_float<bf16>(made[e]);
        *reinterpret_cast<Four*>((bf16*)out + i) = four;
    }
}

__global__ void softcap_kernel(float* __restrict__ x, long count, float cap) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) x[i] = cap * tanhf(x[i] / cap);
}

__global__ void cast_kernel(const void* __restrict__ x, int x_dtype, void* __restrict__ out, int out_dtype, long count) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) store_from_float(out, out_dtype, i, load_as_float(x, x_dtype, i));
}

bool known(int dtype) { return dtype == XRT_F32 || dtype == XRT_BF16; }

}  // namespace

extern "C" int xrt_bigram_add(float* x, long tokens, int width, float scale, const void* table, int table_dtype, int buckets, int mul_prev,
                              int mul_cur, const int* ids, const int* positions, const int* slots, const int* seq_offsets,
                              const int* seq_slots, int n_seqs, int* before, void* stream) {
    XRT_REQUIRE(x && tokens >= 0 && tokens < (1L << 31) && width > 0, "bigram_add: bad sizes");
    XRT_REQUIRE(table == nullptr || (known(table_dtype) && buckets > 0 && mul_prev >= 0 && mul_cur >= 0 && ids && positions && slots &&
                                     seq_offsets && seq_slots && before && n_seqs >= 0),
                "bigram_add: a hashed table needs its sizes, the step's tokens and sequences and the tokens kept per sequence");
    if (tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    bigram_add_kernel<<<(unsigned)tokens, 256, 0, s>>>(x, width, scale, table, table_dtype, ids, positions, slots, before, buckets, mul_prev, mul_cur);
    if (table != nullptr && n_seqs > 0) bigram_keep_kernel<<<(n_seqs + 255) / 256, 256, 0, s>>>(ids, seq_offsets, seq_slots, n_seqs, before);
    XRT_LAUNCH_CHECK("bigram_add");
    return 0;
}

extern "C" int xrt_gated_rows(const float* s, long s_stride, const void* table, int table_dtype, long table_width, long offset, int rows,
                              const int* ids, void* out, int out_dtype, long tokens, int width, void* stream) {
    XRT_REQUIRE(s && table && ids && out && known(table_dtype) && known(out_dtype), "gated_rows: null operand or unknown dtype");
    XRT_REQUIRE(tokens >= 0 && width > 0 && s_stride >= width && offset >= 0 && offset + width <= table_width && rows > 0 &&
                tokens * width < (1L << 40), "gated_rows: bad sizes");
    if (tokens == 0) return 0;
    const long blocks = (tokens * width + 255) / 256;
    XRT_REQUIRE(blocks < (1L << 31), "gated_rows: too many elements");
    gated_rows_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(s, s_stride, table, table_dtype, table_width, offset, rows, ids, out,
                                                                         out_dtype, tokens, width);
    XRT_LAUNCH_CHECK("gated_rows");
    return 0;
}

extern "C" int xrt_add_weighted(float* residual, int count, const float* const* y, const void* const* gains, const float* scales, int gain_dtype,
                                long rows, int width, void* copy, int copy_dtype, void* stream) {
    XRT_REQUIRE(copy == nullptr || known(copy_dtype), "add_weighted: unknown dtype of the copy");
    XRT_REQUIRE(residual && y && gains && scales && count >= 1 && count <= 4 && known(gain_dtype), "add_weighted: one to four terms");
    XRT_REQUIRE(rows >= 0 && width > 0, "add_weighted: bad sizes");
    if (rows == 0) return 0;
    WeightedTerms terms;
    terms.count = count;
    terms.gain_dtype = gain_dtype;
    for (int n = 0; n < 4; ++n) {
        terms.y[n] = n < count ? y[n] : nullptr;
        terms.gain[n] = n < count ? gains[n] : nullptr;
        terms.scale[n] = n < count ? scales[n] : 0.f;
        XRT_REQUIRE(n >= count || y[n] != nullptr, "add_weighted: null term");
    }
    const long blocks = (rows * width + 255) / 256;
    XRT_REQUIRE(blocks < (1L << 31), "add_weighted: too many elements");
    add_weighted_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(residual, terms, rows * width, width, copy, copy_dtype);
    XRT_LAUNCH_CHECK("add_weighted");
    return 0;
}

extern "C" int xrt_glu_clamped(const float* sums, void* out, int out_dtype, long rows, int n, float limit, float alpha, const float* row_weights,
                               void* stream) {
    XRT_REQUIRE(sums && out && known(out_dtype) && rows >= 0 && n > 0 && limit > 0.f, "glu_clamped: bad operands");
    if (rows == 0) return 0;
    if (n % 4 == 0 && (uintptr_t)sums % 16 == 0 && (uintptr_t)out % 16 == 0) {
        const long fours = (rows * n / 4 + 255) / 256;
        XRT_REQUIRE(fours < (1L << 31), "glu_clamped: too many elements");
        glu_clamped_four_kernel<<<(unsigned)fours, 256, 0, (hipStream_t)stream>>>(sums, out, out_dtype, rows, n, limit, alpha, row_weights);
        XRT_LAUNCH_CHECK("glu_clamped");
        return 0;
    }
    const long blocks = (rows * n + 255) / 256;
    XRT_REQUIRE(blocks < (1L << 31), "glu_clamped: too many elements");
    glu_clamped_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(sums, out, out_dtype, rows, n, limit, alpha, row_weights);
    XRT_LAUNCH_CHECK("glu_clamped");
    return 0;
}

extern "C" int xrt_softcap(float* x, long count, float cap, void* stream) {
    XRT_REQUIRE(x && count >= 0 && cap > 0.f, "softcap: bad operands");
    if (count == 0) return 0;
    const long blocks = (count + 255) / 256;
    XRT_REQUIRE(blocks < (1L << 31), "softcap: too many elements");
    softcap_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(x, count, cap);
    XRT_LAUNCH_CHECK("softcap");
    return 0;
}

extern "C" int xrt_cast(const void* x, int x_dtype, void* out, int out_dtype, long count, void* stream) {
    XRT_REQUIRE(x && out && known(x_dtype) && known(out_dtype) && count >= 0, "cast: bad operands");
    if (count == 0) return 0;
    const long blocks = (count + 255) / 256;
    XRT_REQUIRE(blocks < (1L << 31), "cast: too many elements");
    cast_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(x, x_dtype, out, out_dtype, count);
    XRT_LAUNCH_CHECK("cast");
    return 0;
}
