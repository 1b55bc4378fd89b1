// Attention whose keys and values are made from a latent: the cache keeps, for every token, one row [latent | turned key part]
// as the key of a single key/value head and the latent once more as its value. The scores against such a key are those of the
// design's per-head keys when the query's plain part has first been multiplied by the head's key matrix, transposed
// (q_h . (W_h c) = (W_h^T q_h) . c); the sum of the latents under the softmax's weights is turned into the head's output by
// the head's value matrix afterwards. Both are products with a matrix per head (xrt_linear_heads).
//   xrt_latent_complete  from the down projection's float32 sums [latent | key part]: the latent divided by its root mean
//                        square, times a gain; the first rot_dims of the key part turned in pairs of neighbours (2i, 2i + 1) by
//                        position * frequencies[i]; both into the cache
//   xrt_latent_queries   from the queries' float32 sums, head by head [plain | part to turn]: the plain parts to rows of
//                        their own, the turned parts to the tail of the rows that the attention kernel reads
//   xrt_linear_heads     out[t][h][n] = sum over k of a[t][h][k] * w[h][n][k], float32 sums (steps of many rows: on the matrix cores in
//                        bfloat16 with k in whole steps of 32, else in the order of k; steps of few: the lanes of a wavefront along k)
// A prompt that starts a sequence can have its scores as a matrix product of its own rows (all heads' queries of a stretch of
// tokens against the prompt's cached rows, which the step has at hand): then
//   xrt_causal_softmax   turns the float32 scores [queries x heads][keys] into the softmax's weights over the keys at or before
//                        each query, with the heads' sinks in the denominators, as two bfloat16 numbers each (the rounded weight
//                        and what the rounding left) for the product with the latents
//   xrt_transpose        dst[c][r] = src[r][c]: the latents with the tokens along the rows, as that product wants them
#include "cache_layout.h"
#include "xrt_hip.h"

namespace {

__device__ __forceinline__ float small_at(const void* p, int dtype, int i) {
    return dtype == XRT_F32 ? ((const float*)p)[i] : to_float(((const bf16*)p)[i]);
}

// the element e of a part of `rot_dim` numbers whose first rot_dims turn in pairs of neighbours
__device__ __forceinline__ float turned(const float* part, int e, int rot_dims, const float* __restrict__ frequencies, int pos) {
    if (e >= rot_dims) return part[e];
    float sine, cosine;
    sincosf((float)pos * frequencies[e / 2], &sine, &cosine);
    const float mine = part[e], other = part[e ^ 1];
    return e % 2 == 0 ? mine * cosine - other * sine : mine * cosine + other * sine;
}

template <typename T>
__global__ void __launch_bounds__(256) latent_complete_kernel(const float* __restrict__ down, long down_stride, int rank, int rot_dim, int rot_dims,
                                                             const void* __restrict__ gain, int gain_dtype, float eps,
                                                             const float* __restrict__ frequencies, const int* __restrict__ positions,
                                                             const int* __restrict__ slots, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                             const int* __restrict__ block_table, int table_stride, int n_blocks,
                                                             T* __restrict__ rows_out) {
    __shared__ float scratch[32];
    const long t = blockIdx.x;
    const int slot = slots[t], pos = positions[t];
    if (slot < 0) {                                            // (the whole workgroup)
        if (rows_out != nullptr) for (int e = threadIdx.x; e < rank + rot_dim; e += blockDim.x) rows_out[t * (rank + rot_dim) + e] = from_float<T>(0.f);
        return;
    }
    const int block = block_table[(long)slot * table_stride + pos / XRT_BLOCK_TOKENS];
    if (block < 0 || block >= n_blocks) return;
    const float* row = down + t * down_stride;
    float squares = 0.f;
    for (int e = threadIdx.x; e < rank; e += blockDim.x) squares = fmaf(row[e], row[e], squares);
    const float inv = 1.0f / sqrtf(block_sum(squares, scratch) / (float)rank + eps);
    const int head_dim = rank + rot_dim, place = pos % XRT_BLOCK_TOKENS;
    T* keys = k_cache + (long)block * XRT_BLOCK_TOKENS * head_dim;
    T* values = v_cache + (long)block * XRT_BLOCK_TOKENS * rank;
    for (int e = threadIdx.x; e < head_dim; e += blockDim.x) {
        if (e < rank) {
            const T c = from_float<T>(row[e] * inv * small_at(gain, gain_dtype, e));
            keys[cache_key_offset(place, e, head_dim)] = c;
            values[cache_value_offset(e, place, rank)] = c;
            if (rows_out != nullptr) rows_out[t * head_dim + e] = c;
        } else {
            const T k = from_float<T>(turned(row + rank, e - rank, rot_dims, frequencies, pos));
            keys[cache_key_offset(place, e, head_dim)] = k;
            if (rows_out != nullptr) rows_out[t * head_dim + e] = k;
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(XRT_WAVE) latent_queries_kernel(const float* __restrict__ q, long q_stride, int heads, int dim, int rot_dim,
                                                                 int rot_dims, const float* __restrict__ frequencies,
                                                                 const int* __restrict__ positions, T* __restrict__ plain, T* __restrict__ full,
                                                                 long full_stride, int rank) {
    const long t = blockIdx.x / heads;
    const int head = blockIdx.x % heads, pos = positions[t];
    const float* mine = q + t * q_stride + (long)head * (dim + rot_dim);
    for (int e = threadIdx.x; e < dim; e += XRT_WAVE) plain[(t * heads + head) * dim + e] = from_float<T>(mine[e]);
    T* tail = full + t * full_stride + (long)head * (rank + rot_dim) + rank;
    for (int e = threadIdx.x; e < rot_dim; e += XRT_WAVE) tail[e] = from_float<T>(turned(mine + dim, e, rot_dims, frequencies, pos));
}

// A tile of 64 rows x 64 outputs of one head a workgroup, k in steps of 16 through LDS, 4 x 4 outputs a thread; every
// output's sum runs over k in order, whatever the tile it falls into.
constexpr int HEADS_TILE = 64, HEADS_K = 16;

template <typename T>
__global__ void __launch_bounds__(256) linear_heads_kernel(const T* __restrict__ a, long a_stride, long a_head, const T* __restrict__ w,
                                                          T* __restrict__ out, long out_stride, long out_head, long rows, int n, int k) {
    __shared__ float as[HEADS_K][HEADS_TILE + 1], ws[HEADS_K][HEADS_TILE + 1];
    const int head = blockIdx.z;
    const long row0 = (long)blockIdx.x * HEADS_TILE;
    const int n0 = blockIdx.y * HEADS_TILE;
    const int tr = threadIdx.x / 16, tc = threadIdx.x % 16;
    const T* a_base = a + (long)head * a_head;
    const T* w_base = w + (long)head * n * k;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    for (int k0 = 0; k0 < k; k0 += HEADS_K) {
        for (int e = threadIdx.x; e < HEADS_TILE * HEADS_K; e += 256) {
            const int r = e / HEADS_K, kk = e % HEADS_K;
            as[kk][r] = row0 + r < rows && k0 + kk < k ? to_float(a_base[(row0 + r) * a_stride + k0 + kk]) : 0.f;
            ws[kk][r] = n0 + r < n && k0 + kk < k ? to_float(w_base[(long)(n0 + r) * k + k0 + kk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < HEADS_K; ++kk) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { av[i] = as[kk][tr * 4 + i]; wv[i] = ws[kk][tc * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const long r = row0 + tr * 4 + i;
            const int c = n0 + tc * 4 + j;
            if (r < rows && c < n) out[r * out_stride + (long)head * out_head + c] = from_float<T>(acc[i][j]);
        }
}

// A workgroup a row: row m is the query at position first_position + m / heads of head m % heads. Three passes over the row
// (largest visible score, sum, weights); keys behind the query's position get a weight of nothing.
__global__ void __launch_bounds__(256) causal_softmax_kernel(const float* __restrict__ scores, long keys, int heads, int first_position, float scale,
                                                            const float* __restrict__ sinks, bf16* __restrict__ rounded, bf16* __restrict__ rest) {
    __shared__ float scratch[32];
    const long row = blockIdx.x;
    const int head = (int)(row % heads), visible = min((long)first_position + row / heads + 1, keys);
    const float* mine = scores + row * keys;
    const float sink = sinks != nullptr ? sinks[head] : -INFINITY;
    float top = sink;
    for (int j = threadIdx.x; j < visible; j += 256) top = fmaxf(top, mine[j] * scale);
    top = wave_max(top);
    __syncthreads();
    if (threadIdx.x % XRT_WAVE == 0) scratch[threadIdx.x / XRT_WAVE] = top;
    __syncthreads();
    for (int w = 0; w < 256 / XRT_WAVE; ++w) top = fmaxf(top, scratch[w]);
    float sum = 0.f;
    for (int j = threadIdx.x; j < visible; j += 256) sum += expf(mine[j] * scale - top);
    sum = block_sum(sum, scratch);
    if (sinks != nullptr) sum += expf(sink - top);
    const float inv = 1.0f / sum;
    for (long j = threadIdx.x; j < keys; j += 256) {
        const float weight = j < visible ? expf(mine[j] * scale - top) * inv : 0.f;
        const bf16 first = from_float<bf16>(weight);
        rounded[row * keys + j] = first;
        rest[row * keys + j] = from_float<bf16>(weight - to_float(first));
    }
}

template <typename T>
__global__ void __launch_bounds__(256) transpose_kernel(const T* __restrict__ src, long src_stride, long rows, int cols, T* __restrict__ dst) {
    __shared__ T tile[32][33];
    const long r0 = (long)blockIdx.x * 32;
    const int c0 = blockIdx.y * 32, tx = threadIdx.x % 32, ty = threadIdx.x / 32;
    for (int i = ty; i < 32; i += 8)
        if (r0 + i < rows && c0 + tx < cols) tile[i][tx] = src[(r0 + i) * src_stride + c0 + tx];
    __syncthreads();
    for (int i = ty; i < 32; i += 8)
        if (c0 + i < cols && r0 + tx < rows) dst[(long)(c0 + i) * rows + r0 + tx] = tile[tx][i];
}

// The same product on the matrix cores, for bfloat16 steps of many rows with k in whole steps of 32: a wavefront takes 16 rows
// and 64 outputs of one head; both operands of v_mfma_f32_16x16x32_bf16 come straight from memory, sixteen bytes a lane (a row
// of a: 8 consecutive k of one token; a row of w: 8 consecutive k of one output), nothing passes LDS.
typedef __bf16 heads_bf16x8 __attribute__((ext_vector_type(8)));
typedef float heads_floatx4 __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(256) linear_heads_mfma_kernel(const bf16* __restrict__ a, long a_stride, long a_head, const bf16* __restrict__ w,
                                                               bf16* __restrict__ out, long out_stride, long out_head, long rows, int n, int k) {
    const int head = blockIdx.z, lane = threadIdx.x % XRT_WAVE, wave = threadIdx.x / XRT_WAVE, r = lane % 16, c = lane / 16;
    const long row0 = (long)blockIdx.x * 64 + wave * 16;
    if (row0 >= rows) return;                                  // (the whole wavefront)
    const int n0 = blockIdx.y * 64;
    const bf16* of_a = a + min(row0 + r, rows - 1) * a_stride + (long)head * a_head + c * 8;
    const bf16* of_w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) of_w[j] = w + ((long)head * n + min(n0 + 16 * j + r, n - 1)) * k + c * 8;
    heads_floatx4 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = heads_floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
    for (int k0 = 0; k0 < k; k0 += 32) {
        const heads_bf16x8 of_rows = *reinterpret_cast<const heads_bf16x8*>(of_a + k0);
        heads_bf16x8 of_outputs[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) of_outputs[j] = *reinterpret_cast<const heads_bf16x8*>(of_w[j] + k0);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(of_rows, of_outputs[j], acc[j], 0, 0, 0);
    }
    // register i of tile j is row row0 + 4 c + i, output n0 + 16 j + r
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const long row = row0 + 4 * c + i;
            const int column = n0 + 16 * j + r;
            if (row < rows && column < n) out[row * out_stride + (long)head * out_head + column] = (bf16)acc[j][i];
        }
}

// The same product for a step of few rows (a decode step): a wavefront an output column of one head, its lanes along k (a lane
// takes sixteen bytes of the column's row of w at a time, and the same stretch of every row of a), the lanes' sums added in
// the fixed order of the wavefront's butterfly. A row's result does not depend on the rows around it.
constexpr int HEADS_FEW = 16, FEW_WAVES = 4;

template <typename T>
__global__ void __launch_bounds__(FEW_WAVES * XRT_WAVE) linear_heads_few_kernel(const T* __restrict__ a, long a_stride, long a_head,
                                                                               const T* __restrict__ w, T* __restrict__ out, long out_stride,
                                                                               long out_head, int rows, int n, int k) {
    const int head = blockIdx.y, lane = threadIdx.x % XRT_WAVE, column = blockIdx.x * FEW_WAVES + threadIdx.x / XRT_WAVE;
    if (column >= n) return;                                   // (the whole wavefront)
    const T* of_w = w + ((long)head * n + column) * k;
    const T* of_a = a + (long)head * a_head;
    constexpr int PIECE = 16 / sizeof(T);
    struct alignas(16) Piece { T e[PIECE]; };
    const bool whole = k % PIECE == 0 && (uintptr_t)w % 16 == 0 && (uintptr_t)a % 16 == 0 && a_stride % PIECE == 0 && a_head % PIECE == 0;
    float acc[HEADS_FEW];
#pragma unroll
    for (int r = 0; r < HEADS_FEW; ++r) acc[r] = 0.f;
    for (int k0 = lane * PIECE; k0 < k; k0 += XRT_WAVE * PIECE) {
        float piece[PIECE];
        if (whole) {
            const Piece loaded = *reinterpret_cast<const Piece*>(of_w + k0);
#pragma unroll
            for (int e = 0; e < PIECE; ++e) piece[e] = to_float(loaded.e[e]);
        } else {
#pragma unroll
            for (int e = 0; e < PIECE; ++e) piece[e] = k0 + e < k ? to_float(of_w[k0 + e]) : 0.f;
        }
#pragma unroll
        for (int r = 0; r < HEADS_FEW; ++r) {
            if (r < rows) {
                const T* of_row = of_a + (long)r * a_stride + k0;
                if (whole) {
                    const Piece loaded = *reinterpret_cast<const Piece*>(of_row);
#pragma unroll
                    for (int e = 0; e < PIECE; ++e) acc[r] = fmaf(to_float(loaded.e[e]), piece[e], acc[r]);
                } else {
#pragma unroll
                    for (int e = 0; e < PIECE; ++e)
                        if (k0 + e < k) acc[r] = fmaf(to_float(of_row[e]), piece[e], acc[r]);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < HEADS_FEW; ++r) {
        if (r < rows) {
            const float sum = wave_sum(acc[r]);
            if (lane == 0) out[(long)r * out_stride + (long)head * out_head + column] = from_float<T>(sum);
        }
    }
}

}  // namespace

extern "C" int xrt_causal_softmax(const float* scores, long rows, long keys, int heads, int first_position, float scale, const float* sinks,
                                  void* rounded, void* rest, void* stream) {
    XRT_REQUIRE(scores && rounded && rest && rows >= 0 && rows < (1L << 31) && keys > 0 && keys < (1L << 31) && heads > 0 && first_position >= 0,
                "causal_softmax: bad operands");
    if (rows == 0) return 0;
    causal_softmax_kernel<<<(unsigned)rows, 256, 0, (hipStream_t)stream>>>(scores, keys, heads, first_position, scale, sinks, (bf16*)rounded, (bf16*)rest);
    XRT_LAUNCH_CHECK("causal_softmax");
    return 0;
}

extern "C" int xrt_transpose(const void* src, long src_stride, int dtype, long rows, int cols, void* dst, void* stream) {
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "transpose: unknown dtype %d", dtype);
    XRT_REQUIRE(src && dst && rows >= 0 && cols > 0 && src_stride >= cols && (rows + 31) / 32 < (1L << 31) && (cols + 31) / 32 <= 65535, "transpose: bad operands");
    if (rows == 0) return 0;
    const dim3 grid((unsigned)((rows + 31) / 32), (cols + 31) / 32);
    if (dtype == XRT_F32) transpose_kernel<float><<<grid, 256, 0, (hipStream_t)stream>>>((const float*)src, src_stride, rows, cols, (float*)dst);
    else transpose_kernel<bf16><<<grid, 256, 0, (hipStream_t)stream>>>((const bf16*)src, src_stride, rows, cols, (bf16*)dst);
    XRT_LAUNCH_CHECK("transpose");
    return 0;
}

extern "C" int xrt_latent_complete(const float* down, long down_stride, int dtype, long tokens, int rank, int rot_dim, int rot_dims,
                                   const void* gain, int gain_dtype, float eps, const float* frequencies, const int* positions, const int* slots,
                                   void* k_cache, void* v_cache, const int* block_table, int table_stride, int n_blocks, void* rows_out,
                                   void* stream) {
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "latent_complete: unknown dtype %d", dtype);
    XRT_REQUIRE(gain_dtype == XRT_F32 || gain_dtype == XRT_BF16, "latent_complete: unknown dtype %d of the gain", gain_dtype);
    XRT_REQUIRE(down && gain && positions && slots && k_cache && v_cache && block_table, "latent_complete: null operand");
    XRT_REQUIRE(tokens >= 0 && tokens < (1L << 31) && rank > 0 && rot_dim >= 0 && down_stride >= rank + rot_dim && table_stride > 0 && n_blocks > 0,
                "latent_complete: bad sizes");
    XRT_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= rot_dim && (rot_dims == 0 || frequencies != nullptr),
                "latent_complete: %d dims turn in pairs inside a part of %d", rot_dims, rot_dim);
    if (tokens == 0) return 0;
    if (dtype == XRT_F32)
        latent_complete_kernel<float><<<(unsigned)tokens, 256, 0, (hipStream_t)stream>>>(down, down_stride, rank, rot_dim, rot_dims, gain, gain_dtype, eps,
                                                                                      frequencies, positions, slots, (float*)k_cache, (float*)v_cache,
                                                                                      block_table, table_stride, n_blocks, (float*)rows_out);
    else
        latent_complete_kernel<bf16><<<(unsigned)tokens, 256, 0, (hipStream_t)stream>>>(down, down_stride, rank, rot_dim, rot_dims, gain, gain_dtype, eps,
                                                                                     frequencies, positions, slots, (bf16*)k_cache, (bf16*)v_cache,
                                                                                     block_table, table_stride, n_blocks, (bf16*)rows_out);
    XRT_LAUNCH_CHECK("latent_complete");
    return 0;
}

extern "C" int xrt_latent_queries(const float* q, long q_stride, int dtype, long tokens, int heads, int dim, int rot_dim, int rot_dims,
                                  const float* frequencies, const int* positions, void* plain, void* full, long full_stride, int rank,
                                  void* stream) {
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "latent_queries: unknown dtype %d", dtype);
    XRT_REQUIRE(q && positions && plain && full, "latent_queries: null operand");
    XRT_REQUIRE(tokens >= 0 && heads > 0 && tokens * heads < (1L << 31) && dim > 0 && rot_dim >= 0 && rank > 0 &&
                q_stride >= (long)heads * (dim + rot_dim) && full_stride >= (long)heads * (rank + rot_dim), "latent_queries: bad sizes");
    XRT_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= rot_dim && (rot_dims == 0 || frequencies != nullptr),
                "latent_queries: %d dims turn in pairs inside a part of %d", rot_dims, rot_dim);
    if (tokens == 0) return 0;
    if (dtype == XRT_F32)
        latent_queries_kernel<float><<<(unsigned)(tokens * heads), XRT_WAVE, 0, (hipStream_t)stream>>>(q, q_stride, heads, dim, rot_dim, rot_dims, frequencies,
                                                                                                    positions, (float*)plain, (float*)full, full_stride, rank);
    else
        latent_queries_kernel<bf16><<<(unsigned)(tokens * heads), XRT_WAVE, 0, (hipStream_t)stream>>>(q, q_stride, heads, dim, rot_dim, rot_dims, frequencies,
                                                                                                   positions, (bf16*)plain, (bf16*)full, full_stride, rank);
    XRT_LAUNCH_CHECK("latent_queries");
    return 0;
}

extern "C" int xrt_linear_heads(const void* a, long a_stride, long a_head, const void* w, int dtype, void* out, long out_stride, long out_head,
                                long rows, int heads, int n, int k, void* stream) {
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "linear_heads: unknown dtype %d", dtype);
    XRT_REQUIRE(a && w && out && rows >= 0 && heads > 0 && heads <= 65535 && n > 0 && k > 0, "linear_heads: bad operands");
    XRT_REQUIRE(a_head >= k && a_stride >= (heads - 1) * a_head + k && out_head >= n && out_stride >= (heads - 1) * out_head + n,
                "linear_heads: rows %ld and %ld apart do not hold %d heads %ld and %ld apart", a_stride, out_stride, heads, a_head, out_head);
    if (rows == 0) return 0;
    if (rows <= HEADS_FEW) {
        const dim3 few((n + FEW_WAVES - 1) / FEW_WAVES, heads);
        if (dtype == XRT_F32)
            linear_heads_few_kernel<float><<<few, FEW_WAVES * XRT_WAVE, 0, (hipStream_t)stream>>>((const float*)a, a_stride, a_head, (const float*)w,
                                                                                               (float*)out, out_stride, out_head, (int)rows, n, k);
        else
            linear_heads_few_kernel<bf16><<<few, FEW_WAVES * XRT_WAVE, 0, (hipStream_t)stream>>>((const bf16*)a, a_stride, a_head, (const bf16*)w,
                                                                                              (bf16*)out, out_stride, out_head, (int)rows, n, k);
        XRT_LAUNCH_CHECK("linear_heads");
        return 0;
    }
    if (dtype == XRT_BF16 && k % 32 == 0 && a_stride % 8 == 0 && a_head % 8 == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0 &&
        (rows + 63) / 64 < (1L << 31) && (n + 63) / 64 <= 65535) {
        const dim3 tiles((unsigned)((rows + 63) / 64), (n + 63) / 64, heads);
        linear_heads_mfma_kernel<<<tiles, 256, 0, (hipStream_t)stream>>>((const bf16*)a, a_stride, a_head, (const bf16*)w, (bf16*)out, out_stride, out_head,
                                                                         rows, n, k);
        XRT_LAUNCH_CHECK("linear_heads");
        return 0;
    }
    const long row_tiles = (rows + HEADS_TILE - 1) / HEADS_TILE;
    XRT_REQUIRE(row_tiles < (1L << 31) && (n + HEADS_TILE - 1) / HEADS_TILE <= 65535, "linear_heads: too many tiles");
    const dim3 grid((unsigned)row_tiles, (n + HEADS_TILE - 1) / HEADS_TILE, heads);
    if (dtype == XRT_F32)
        linear_heads_kernel<float><<<grid, 256, 0, (hipStream_t)stream>>>((const float*)a, a_stride, a_head, (const float*)w, (float*)out, out_stride,
                                                                       out_head, rows, n, k);
    else
        linear_heads_kernel<bf16><<<grid, 256, 0, (hipStream_t)stream>>>((const bf16*)a, a_stride, a_head, (const bf16*)w, (bf16*)out, out_stride,
                                                                      out_head, rows, n, k);
    XRT_LAUNCH_CHECK("linear_heads");
    return 0;
}
