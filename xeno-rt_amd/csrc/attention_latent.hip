// Attention of many query heads on ONE key/value head with large keys, on the matrix cores: the shape of attention through a
// cached latent (parts/latent.py), where all heads of a token read the same row [latent | turned key part] and the values are
// the latents. bfloat16, the queries alone in q; key size a multiple of 32 up to 512, value size a multiple of 32 up to 512
// (the sizes at which cache blocks lie in the tiles of cache_layout.h).
//
// A wavefront takes a token, sixteen of its heads and a chunk of the sequence's cache blocks. The sixteen heads are the
// sixteen columns of v_mfma_f32_16x16x32_bf16: S^T[key][head] = K Q^T with a tile of the cache (16 keys x 32 dims, in the
// order of the A operand: one load instruction takes a contiguous kilobyte) as A and the heads' queries, kept in registers,
// as B; after the two tiles of a group of 32 keys a lane holds the scores of eight consecutive keys of one head, which is the
// B operand of O^T[dim][head] += V^T P^T, whose A operand is a tile of the value block (16 dims x 32 tokens) as it lies.
// The softmax's weights are float32 and enter that product as two bfloat16 numbers each, the rounded weight and what the
// rounding left. Every chunk is worked off from empty hands; a second kernel merges a token's chunks in their order, adds the
// head's sink to the denominator (a learnt score without a value, or none) and writes the result.
#include "cache_layout.h"
#include "xrt_hip.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int LATENT_MOST = 512;                 // largest key and value size
constexpr int KEY_STEPS = LATENT_MOST / 32;      // steps of 32 dims of a score product
constexpr int VALUE_TILES = LATENT_MOST / 16;    // tiles of 16 dims of the value product
constexpr int HEADS_A_WAVE = 16;
constexpr int MOST_CHUNKS = 32;                  // chunks of blocks a sequence is cut into at most

// floats a (token, head group, chunk) leaves for the merge: for each of 16 heads the weighted values, the largest score, the sum
__host__ __device__ inline int head_floats(int value_dim) { return value_dim + 4; }     // (a multiple of four: a lane stores four at a time)
__host__ __device__ inline long partial_floats(int value_dim) { return (long)HEADS_A_WAVE * head_floats(value_dim); }

__global__ void __launch_bounds__(XRT_WAVE) latent_chunks_kernel(const bf16* __restrict__ q, long q_stride, int n_heads, int head_dim, int value_dim,
                                                                const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
                                                                const int* __restrict__ block_table, int table_stride, int n_blocks,
                                                                const int* __restrict__ positions, const int* __restrict__ slots, float scale,
                                                                int chunk_blocks, int chunks, float* __restrict__ partial) {
    const int lane = threadIdx.x, column = lane % 16, quarter = lane / 16;
    const int chunk = blockIdx.x, groups = gridDim.z, group = blockIdx.z;
    const long token = blockIdx.y;
    const int slot = slots[token], pos = positions[token];
    if (slot < 0) return;                                      // (the merge writes zeros)
    const int first_block = chunk * chunk_blocks, last_block = min(pos / XRT_BLOCK_TOKENS, first_block + chunk_blocks - 1);
    if (first_block > last_block) return;                      // (the merge knows from the position which chunks exist)
    const int head = group * HEADS_A_WAVE + column;
    const int key_steps = head_dim / 32, value_tiles = value_dim / 16;

    // the heads' queries: lane (column, quarter) holds dims 32 s + 8 quarter .. + 7 of head `column`, for every step s
    bf16x8 queries[KEY_STEPS];
    const bf16* mine = q + token * q_stride + (long)min(head, n_heads - 1) * head_dim + quarter * 8;
#pragma unroll
    for (int s = 0; s < KEY_STEPS; ++s) {
#pragma unroll
        for (int e = 0; e < 8; ++e) queries[s][e] = (bf16)0.f;
        if (s < key_steps && head < n_heads) queries[s] = *reinterpret_cast<const bf16x8*>(mine + s * 32);
    }
    floatx4 o[VALUE_TILES];
#pragma unroll
    for (int u = 0; u < VALUE_TILES; ++u) o[u] = floatx4{0.f, 0.f, 0.f, 0.f};
    float top = -INFINITY, sum = 0.f;                          // of this lane's head: top is shared by the head's four lanes, sum is this lane's share

    const int* table = block_table + (long)slot * table_stride;
    for (int b = first_block; b <= last_block; ++b) {
        const int block = min(max(table[b], 0), n_blocks - 1); // the host never hands out anything else
        const bf16* keys = k_cache + (long)block * XRT_BLOCK_TOKENS * head_dim;
        const bf16* values = v_cache + (long)block * XRT_BLOCK_TOKENS * value_dim;
        for (int g = 0; g < 2; ++g) {                          // the block's two groups of 32 keys
            const int k0 = b * XRT_BLOCK_TOKENS + g * 32;
            if (k0 > pos) break;
            // The tiles are asked for four steps at a time, both tiles of a step, before the products that use them (a branch
            // per step would have every load awaited alone); steps beyond the key's size read the last tile again and multiply
            // it with queries that are zeros.
            floatx4 s[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int step0 = 0; step0 < KEY_STEPS; step0 += 4) {
                if (step0 < key_steps) {
                    bf16x8 tiles[2][4];
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            tiles[t][i] = *reinterpret_cast<const bf16x8*>(keys + ((long)((g * 2 + t) * key_steps + min(step0 + i, key_steps - 1)) * XRT_WAVE + lane) * 8);
#pragma unroll
                    for (int i = 0; i < 4; ++i)
#pragma unroll
                        for (int t = 0; t < 2; ++t) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tiles[t][i], queries[step0 + i], s[t], 0, 0, 0);
                }
            }
            // register i of tile t is the key k0 + 8 quarter + 4 t + i, for this lane's head
            float scores[8];
            float here = -INFINITY;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                scores[e] = k0 + quarter * 8 + e <= pos ? s[e / 4][e % 4] * scale : -INFINITY;
                here = fmaxf(here, scores[e]);
            }
            here = fmaxf(here, __shfl_xor(here, 16, XRT_WAVE));
            here = fmaxf(here, __shfl_xor(here, 32, XRT_WAVE));
            const float top_new = fmaxf(top, here);            // (finite: the group's first key is at or before the query)
            const float correction = expf(top - top_new);      // 0 for empty hands
            top = top_new;
            sum *= correction;
            bf16x8 rounded, rest;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float weight = expf(scores[e] - top);     // 0 for a key behind the query
                sum += weight;
                rounded[e] = (bf16)weight;
                rest[e] = (bf16)(weight - (float)rounded[e]);
            }
            const bool edge = k0 + 31 > pos;                    // what lies behind the sequence's last key is not ours: kept away from the zeros
#pragma unroll
            for (int u0 = 0; u0 < VALUE_TILES; u0 += 4) {
                if (u0 < value_tiles) {                        // (tiles beyond the value's size read the last one again into sums that nobody reads)
                    bf16x8 tiles[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        tiles[i] = *reinterpret_cast<const bf16x8*>(values + ((long)(g * value_tiles + min(u0 + i, value_tiles - 1)) * XRT_WAVE + lane) * 8);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if (edge) {
#pragma unroll
                            for (int e = 0; e < 8; ++e)
                                if (k0 + quarter * 8 + e > pos) tiles[i][e] = (bf16)0.f;
                        }
#pragma unroll
                        for (int j = 0; j < 4; ++j) o[u0 + i][j] *= correction;
                        o[u0 + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tiles[i], rounded, o[u0 + i], 0, 0, 0);
                        o[u0 + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tiles[i], rest, o[u0 + i], 0, 0, 0);
                    }
                }
            }
        }
    }
    sum += __shfl_xor(sum, 16, XRT_WAVE);
    sum += __shfl_xor(sum, 32, XRT_WAVE);
    // register i of tile u is dim 16 u + 4 quarter + i of head `column`
    float* out = partial + ((token * groups + group) * chunks + chunk) * partial_floats(value_dim) + (long)column * head_floats(value_dim);
#pragma unroll
    for (int u = 0; u < VALUE_TILES; ++u) {
        if (u < value_tiles) *reinterpret_cast<floatx4*>(out + u * 16 + quarter * 4) = o[u];
    }
    if (quarter == 0) {
        out[value_dim] = top;
        out[value_dim + 1] = sum;
    }
}

// A workgroup a (token, head): the chunks' parts in their order, the sink, the quotient.
__global__ void __launch_bounds__(XRT_WAVE) latent_merge_kernel(const float* __restrict__ partial, int n_heads, int value_dim, int chunk_blocks, int chunks,
                                                               const int* __restrict__ positions, const int* __restrict__ slots,
                                                               const float* __restrict__ sinks, bf16* __restrict__ out) {
    const long token = blockIdx.x;
    const int head = blockIdx.y, lane = threadIdx.x, groups = (n_heads + HEADS_A_WAVE - 1) / HEADS_A_WAVE;
    bf16* dst = out + (token * n_heads + head) * value_dim;
    if (slots[token] < 0) {
        for (int d = lane; d < value_dim; d += XRT_WAVE) dst[d] = (bf16)0.f;
        return;
    }
    const int mine = positions[token] / XRT_BLOCK_TOKENS / chunk_blocks + 1;      // this sequence's chunks
    const float* parts = partial + ((token * groups + head / HEADS_A_WAVE) * chunks) * partial_floats(value_dim) + (long)(head % HEADS_A_WAVE) * head_floats(value_dim);
    constexpr int OWNED = LATENT_MOST / XRT_WAVE;
    float acc[OWNED], top = -INFINITY, sum = 0.f;
#pragma unroll
    for (int i = 0; i < OWNED; ++i) acc[i] = 0.f;
    // First the largest score of all chunks (lane c reads chunk c's), then every chunk's share relative to it, in the chunks'
    // order, four chunks' loads on their way at a time (chunks beyond the sequence's read the last one again with a share of nothing).
    const long stride = partial_floats(value_dim);
    const float my_top = lane < mine ? parts[(long)lane * stride + value_dim] : -INFINITY;
    top = wave_max(my_top);
    const float my_take = lane < mine ? expf(my_top - top) : 0.f;
    sum = wave_sum(lane < mine ? parts[(long)lane * stride + value_dim + 1] * my_take : 0.f);
#pragma unroll
    for (int c0 = 0; c0 < MOST_CHUNKS; c0 += 4) {
        if (c0 < mine) {
            float loaded[4][OWNED], take[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float* part = parts + (long)min(c0 + j, mine - 1) * stride;
                take[j] = __shfl(my_take, c0 + j, XRT_WAVE);       // (0 from a lane beyond the sequence's chunks)
#pragma unroll
                for (int i = 0; i < OWNED; ++i) loaded[j][i] = lane + i * XRT_WAVE < value_dim ? part[lane + i * XRT_WAVE] : 0.f;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < OWNED; ++i) acc[i] = fmaf(loaded[j][i], take[j], acc[i]);
        }
    }
    if (sinks != nullptr) {                                    // one more term of the denominator, without a value
        const float sink = sinks[head], top_new = fmaxf(top, sink);
        const float keep = expf(top - top_new);
        sum = fmaf(sum, keep, expf(sink - top_new));
#pragma unroll
        for (int i = 0; i < OWNED; ++i) acc[i] *= keep;
    }
    const float inv = sum > 0.f ? 1.0f / sum : 0.f;
#pragma unroll
    for (int i = 0; i < OWNED; ++i) {
        const int d = lane + i * XRT_WAVE;
        if (d < value_dim) dst[d] = (bf16)(acc[i] * inv);
    }
}

int chunk_blocks_for(int max_context) {
    const int blocks = (max(max_context, 1) + XRT_BLOCK_TOKENS - 1) / XRT_BLOCK_TOKENS;
    return (blocks + MOST_CHUNKS - 1) / MOST_CHUNKS;
}

}  // namespace

extern "C" int xrt_attention_latent_accepts(int dtype, int n_kv_heads, int head_dim, int value_dim) {
    return dtype == XRT_BF16 && n_kv_heads == 1 && head_dim % 32 == 0 && value_dim % 32 == 0 && head_dim > 0 && value_dim > 0 &&
           head_dim <= LATENT_MOST && value_dim <= LATENT_MOST;
}

extern "C" long xrt_attention_latent_workspace(long tokens, int n_heads, int value_dim, int max_context) {
    const int chunk_blocks = chunk_blocks_for(max_context);
    const int chunks = ((max(max_context, 1) + XRT_BLOCK_TOKENS - 1) / XRT_BLOCK_TOKENS + chunk_blocks - 1) / chunk_blocks;
    return tokens * ((n_heads + HEADS_A_WAVE - 1) / HEADS_A_WAVE) * chunks * partial_floats(value_dim);
}

extern "C" int xrt_attention_latent(const void* q, long q_stride, long tokens, int n_heads, int head_dim, int value_dim, const void* k_cache,
                                    const void* v_cache, const int* block_table, int table_stride, int n_blocks, const int* positions,
                                    const int* slots, void* out, float scale, const float* sink_scores, int max_context, float* workspace,
                                    long workspace_floats, void* stream) {
    XRT_REQUIRE(xrt_attention_latent_accepts(XRT_BF16, 1, head_dim, value_dim), "attention (latent): key and value sizes %d and %d: multiples of 32 up to %d",
                head_dim, value_dim, LATENT_MOST);
    XRT_REQUIRE(q && k_cache && v_cache && block_table && positions && slots && out, "attention (latent): null operand");
    XRT_REQUIRE(tokens >= 0 && tokens <= 65535 && n_heads > 0 && n_heads <= 65535 * HEADS_A_WAVE && table_stride > 0 && n_blocks > 0 && max_context > 0,
                "attention (latent): bad sizes (%ld tokens, %d heads)", tokens, n_heads);
    XRT_REQUIRE(q_stride >= (long)n_heads * head_dim && q_stride % 8 == 0 && (uintptr_t)q % 16 == 0 && (uintptr_t)k_cache % 16 == 0 && (uintptr_t)v_cache % 16 == 0,
                "attention (latent): rows of q %ld apart, or operands off their sixteen bytes", q_stride);
    XRT_REQUIRE(max_context <= table_stride * XRT_BLOCK_TOKENS, "attention (latent): a sequence of %d tokens exceeds the block table", max_context);
    if (tokens == 0) return 0;
    const int chunk_blocks = chunk_blocks_for(max_context);
    const int chunks = ((max_context + XRT_BLOCK_TOKENS - 1) / XRT_BLOCK_TOKENS + chunk_blocks - 1) / chunk_blocks;
    const int groups = (n_heads + HEADS_A_WAVE - 1) / HEADS_A_WAVE;
    XRT_REQUIRE(workspace != nullptr && workspace_floats >= tokens * groups * chunks * partial_floats(value_dim) && (uintptr_t)workspace % 16 == 0,
                "attention (latent): the workspace needs %ld floats", tokens * groups * chunks * partial_floats(value_dim));
    latent_chunks_kernel<<<dim3(chunks, (unsigned)tokens, groups), XRT_WAVE, 0, (hipStream_t)stream>>>(
        (const bf16*)q, q_stride, n_heads, head_dim, value_dim, (const bf16*)k_cache, (const bf16*)v_cache, block_table, table_stride, n_blocks,
        positions, slots, scale, chunk_blocks, chunks, workspace);
    XRT_LAUNCH_CHECK("attention (latent, chunks)");
    latent_merge_kernel<<<dim3((unsigned)tokens, n_heads), XRT_WAVE, 0, (hipStream_t)stream>>>(workspace, n_heads, value_dim, chunk_blocks, chunks, positions,
                                                                                              slots, sink_scores, (bf16*)out);
    XRT_LAUNCH_CHECK("attention (latent, merge)");
    return 0;
}
