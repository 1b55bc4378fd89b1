// Choosing experts for every token, and weighting what the experts made.
//   xrt_route_experts   from router logits z [tokens][experts] (float32): scores s = sigmoid(z), or softmax(z) over all experts
//                       (softmax != 0); the chosen weights are multiplied by `scale` in the end; the experts stand in `groups`
//                       equal groups of neighbours, a group's score is the sum of its `group_top` largest scores, only experts
//                       of the `keep` best groups can be chosen; the `top` largest scores among those are chosen, and their
//                       weights are their scores divided by the scores' sum (+ floor). Equal scores: the lower index wins.
//                       Out: weights [tokens][experts] (float32, zero for experts not chosen), and, if asked for, the chosen
//                       experts [tokens][top] (int32) in the order of their scores.
//   xrt_scale_blocks    act[t][e * width + c] *= weights[t][e]: every expert's stretch of a row times the token's weight for it
//   xrt_experts_sort    the picks (token, chosen expert) in the order of their experts, every expert's stretch filled up to whole
//                       tiles of rows, for products in which each expert multiplies only the tokens that chose it
//   xrt_linear_groups   such a product: every tile of rows with the matrix of its tile's expert (csrc/gemm_mfma.hip)
//   xrt_gather_rows, xrt_experts_combine   the tokens' rows into that order, and the experts' outputs back, weighted and summed
// One thread a token for the choice: the experts of a token are few (up to XRT_MOST_EXPERTS).
#include "common.h"
#include "packing.h"
#include "xrt_hip.h"

int xrt_linear_groups_tile(long rows, int groups);
bool xrt_linear_groups_mfma_accepts(const void* a, int lda, const void* w, int ldw, int N, int K, int mode, const Packing& packing);
int xrt_linear_groups_splits(int tiles_m, int N, int K, int mode);
int xrt_linear_groups_mfma(const void* a, int lda, const void* w, long w_stride, int ldw, void* out, int out_dtype, int tile, int tiles_m, int N,
                           int K, int mode, int activation, const int* tile_group, const Packing& packing, int splits, hipStream_t s);

namespace {

__device__ __forceinline__ float load_as_float(const void* p, int dtype, long i) {
    return dtype == XRT_F32 ? ((const float*)p)[i] : to_float(((const bf16*)p)[i]);
}
__device__ __forceinline__ void store_from_float(void* p, int dtype, long i, float v) {
    if (dtype == XRT_F32) ((float*)p)[i] = v; else ((bf16*)p)[i] = from_float<bf16>(v);
}

__global__ void __launch_bounds__(64) route_experts_kernel(const float* __restrict__ logits, long tokens, int experts, int top, int groups, int keep,
                                                           int group_top, float floor_, float* __restrict__ weights, int* __restrict__ chosen,
                                                           int softmax, float scale) {
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= tokens) return;
    float s[XRT_MOST_EXPERTS];
    unsigned char open[XRT_MOST_EXPERTS];          // 1: may still be chosen
    const int per_group = experts / groups;
    float top_logit = -INFINITY, total = 0.f;
    if (softmax) {
        for (int e = 0; e < experts; ++e) top_logit = fmaxf(top_logit, logits[t * experts + e]);
        for (int e = 0; e < experts; ++e) total += expf(logits[t * experts + e] - top_logit);
    }
    for (int e = 0; e < experts; ++e) {
        s[e] = softmax ? expf(logits[t * experts + e] - top_logit) / total : 1.0f / (1.0f + expf(-logits[t * experts + e]));
        open[e] = groups > 1 ? 0 : 1;
    }
    if (groups > 1) {
        float group_score[XRT_MOST_EXPERTS];
        for (int g = 0; g < groups; ++g) {
            // the sum of the group's group_top largest scores: taken one after another
            float sum = 0.f;
            unsigned long long taken_low = 0, taken_high = 0;      // (per_group <= 128 is enough: checked on the host)
            for (int round = 0; round < group_top && round < per_group; ++round) {
                int best = -1;
                for (int i = 0; i < per_group; ++i) {
                    const bool taken = i < 64 ? (taken_low >> i) & 1 : (taken_high >> (i - 64)) & 1;
                    if (!taken && (best < 0 || s[g * per_group + i] > s[g * per_group + best])) best = i;
                }
                sum += s[g * per_group + best];
                if (best < 64) taken_low |= 1ull << best; else taken_high |= 1ull << (best - 64);
            }
            group_score[g] = sum;
        }
        for (int round = 0; round < keep; ++round) {
            int best = -1;
            for (int g = 0; g < groups; ++g)
                if (!(group_score[g] < 0.f) && (best < 0 || group_score[g] > group_score[best])) best = g;    // (a score that is no number still stands for its group)
            group_score[best] = -1.f;                              // (scores are sums of sigmoids: never negative)
            for (int i = 0; i < per_group; ++i) open[best * per_group + i] = 1;
        }
    }
    for (int e = 0; e < experts; ++e) weights[t * experts + e] = 0.f;
    int picks[XRT_MOST_EXPERTS];
    float sum = 0.f;
    for (int round = 0; round < top; ++round) {
        int best = -1;
        for (int e = 0; e < experts; ++e)
            if (open[e] && (best < 0 || s[e] > s[best])) best = e;
        open[best] = 0;
        picks[round] = best;
        sum += s[best];
    }
    for (int round = 0; round < top; ++round) {
        weights[t * experts + picks[round]] = s[picks[round]] / (sum + floor_) * scale;
        if (chosen != nullptr) chosen[t * top + round] = picks[round];
    }
}

__global__ void scale_blocks_kernel(void* __restrict__ act, int dtype, const float* __restrict__ weights, long tokens, int experts, int width) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long row = (long)experts * width;
    if (i >= tokens * row) return;
    const long t = i / row;
    const int e = (int)(i % row / width);
    store_from_float(act, dtype, i, load_as_float(act, dtype, i) * weights[t * experts + e]);
}

// the same, eight columns a thread (width a multiple of eight, so that the eight share an expert; bfloat16: sixteen bytes a load)
__global__ void __launch_bounds__(256) scale_blocks_eight_kernel(bf16* __restrict__ act, const float* __restrict__ weights, long tokens, int experts, int width) {
    const long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 8;
    const long row = (long)experts * width;
    if (i >= tokens * row) return;
    const long t = i / row;
    const float w = weights[t * experts + (int)(i % row / width)];
    uint4 packed = *reinterpret_cast<const uint4*>(act + i);
    bf16* values = reinterpret_cast<bf16*>(&packed);
#pragma unroll
    for (int j = 0; j < 8; ++j) values[j] = from_float<bf16>(to_float(values[j]) * w);
    *reinterpret_cast<uint4*>(act + i) = packed;
}

// One workgroup sorts a step's picks: counts per expert, every expert's first row (its stretch filled up to whole tiles), the
// tiles' experts, then a row for every pick. Which pick of an expert gets which of its rows depends on the order in which the
// threads arrive; nothing that is computed from the rows depends on it (a row's products see that row alone).
__global__ void __launch_bounds__(1024) experts_sort_kernel(const int* __restrict__ chosen, long picks, int top, int experts, int tile, int room,
                                                            int* __restrict__ rows, int* __restrict__ places, int* __restrict__ tile_group) {
    __shared__ int count[XRT_MOST_EXPERTS], first[XRT_MOST_EXPERTS + 1];
    const int tid = threadIdx.x, threads = blockDim.x;
    for (int e = tid; e < experts; e += threads) count[e] = 0;
    for (int r = tid; r < room; r += threads) rows[r] = -1;
    __syncthreads();
    for (long i = tid; i < picks; i += threads) atomicAdd(&count[chosen[i]], 1);
    __syncthreads();
    if (tid == 0) {
        int at = 0;
        for (int e = 0; e < experts; ++e) {
            first[e] = at;
            at += (count[e] + tile - 1) / tile * tile;
        }
        first[experts] = at;
    }
    __syncthreads();
    for (int t = tid; t < room / tile; t += threads) {
        const int start = t * tile;
        int group = -1;
        if (start < first[experts]) {
            int low = 0, high = experts - 1;                    // the last expert whose first row is at or before start
            while (low < high) {
                const int middle = (low + high + 1) / 2;
                if (first[middle] <= start) low = middle; else high = middle - 1;
            }
            group = low;
        }
        tile_group[t] = group;
    }
    for (int e = tid; e < experts; e += threads) count[e] = 0;
    __syncthreads();
    for (long i = tid; i < picks; i += threads) {
        const int e = chosen[i];
        const int place = first[e] + atomicAdd(&count[e], 1);
        rows[place] = (int)(i / top);
        places[i] = place;
    }
}

// out[r] = x[rows[r]] (zeros where rows[r] < 0); a workgroup a row, eight columns a thread
__global__ void __launch_bounds__(256) gather_rows_kernel(const bf16* __restrict__ x, long x_stride, const int* __restrict__ rows, int width,
                                                          bf16* __restrict__ out) {
    const long r = blockIdx.x;
    const int from = rows[r];
    for (int c = threadIdx.x * 8; c < width; c += blockDim.x * 8) {
        uint4 piece = make_uint4(0u, 0u, 0u, 0u);
        if (from >= 0) piece = *reinterpret_cast<const uint4*>(x + (long)from * x_stride + c);
        *reinterpret_cast<uint4*>(out + r * width + c) = piece;
    }
}

// out[t][c] = sum over a token's picks, in their order, of weights[t][expert of the pick] * sorted[row of the pick][c]
// (sorted: [tiles][parts][tile][width], the parts' sums of a row added in their order first)
__global__ void __launch_bounds__(256) experts_combine_kernel(const float* __restrict__ sorted, const int* __restrict__ places,
                                                              const int* __restrict__ chosen, const float* __restrict__ weights, int top,
                                                              int experts, int width, int tile, int parts, float* __restrict__ out) {
    const long t = blockIdx.x;
    for (int c = threadIdx.x * 4; c < width; c += blockDim.x * 4) {
        float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int k = 0; k < top; ++k) {
            const float w = weights[t * experts + chosen[t * top + k]];
            const int place = places[t * top + k];
            const float* row = sorted + (((long)(place / tile) * parts) * tile + place % tile) * width + c;
            float4 v = *reinterpret_cast<const float4*>(row);
            for (int part = 1; part < parts; ++part) {
                const float4 more = *reinterpret_cast<const float4*>(row + (long)part * tile * width);
                v.x += more.x; v.y += more.y; v.z += more.z; v.w += more.w;
            }
            sum.x = fmaf(w, v.x, sum.x); sum.y = fmaf(w, v.y, sum.y); sum.z = fmaf(w, v.z, sum.z); sum.w = fmaf(w, v.w, sum.w);
        }
        *reinterpret_cast<float4*>(out + t * width + c) = sum;
    }
}

}  // namespace

extern "C" int xrt_route_experts(const float* logits, long tokens, int experts, int top, int groups, int keep, int group_top, float floor_,
                                 float* weights, int* chosen, int softmax, float scale, void* stream) {
    XRT_REQUIRE(logits && weights && tokens >= 0, "route_experts: null operand");
    XRT_REQUIRE(experts > 0 && experts <= XRT_MOST_EXPERTS && top > 0 && groups > 0 && experts % groups == 0 && keep > 0 && keep <= groups &&
                group_top > 0 && (groups == 1 || experts / groups <= 128) && top <= keep * (experts / groups),
                "route_experts: %d experts in %d groups of which %d are kept, %d chosen: up to %d experts in equal groups, and no more "
                "chosen than the kept groups hold", experts, groups, keep, top, XRT_MOST_EXPERTS);
    if (tokens == 0) return 0;
    route_experts_kernel<<<(unsigned)((tokens + 63) / 64), 64, 0, (hipStream_t)stream>>>(logits, tokens, experts, top, groups, keep, group_top,
                                                                                       floor_, weights, chosen, softmax, scale);
    XRT_LAUNCH_CHECK("route_experts");
    return 0;
}

extern "C" int xrt_scale_blocks(void* act, int dtype, const float* weights, long tokens, int experts, int width, void* stream) {
    XRT_REQUIRE(act && weights && (dtype == XRT_F32 || dtype == XRT_BF16) && tokens >= 0 && experts > 0 && width > 0, "scale_blocks: bad operands");
    if (tokens == 0) return 0;
    if (dtype == XRT_BF16 && width % 8 == 0 && (uintptr_t)act % 16 == 0) {
        const long eights = (tokens * experts * width / 8 + 255) / 256;
        XRT_REQUIRE(eights < (1L << 31), "scale_blocks: too many elements");
        scale_blocks_eight_kernel<<<(unsigned)eights, 256, 0, (hipStream_t)stream>>>((bf16*)act, weights, tokens, experts, width);
        XRT_LAUNCH_CHECK("scale_blocks");
        return 0;
    }
    const long blocks = (tokens * experts * width + 255) / 256;
    XRT_REQUIRE(blocks < (1L << 31), "scale_blocks: too many elements");
    scale_blocks_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(act, dtype, weights, tokens, experts, width);
    XRT_LAUNCH_CHECK("scale_blocks");
    return 0;
}

// rows of a tile for a step of `tokens` tokens that choose `top` of `experts` each
extern "C" int xrt_linear_groups_tile_rows(long tokens, int top, int experts) { return xrt_linear_groups_tile(tokens * top, experts); }

// rows a step's sorted picks need at most: every pick one, and every expert up to a tile less one of filling
extern "C" long xrt_experts_sort_room(long tokens, int top, int experts) {
    const long tile = xrt_linear_groups_tile(tokens * top, experts);
    return (tokens * top + (long)experts * (tile - 1) + tile - 1) / tile * tile;
}

extern "C" int xrt_experts_sort(const int* chosen, long tokens, int top, int experts, int* rows, long room, int* places, int* tile_group,
                                void* stream) {
    XRT_REQUIRE(chosen && rows && places && tile_group && tokens > 0 && top > 0 && experts > 0 && experts <= XRT_MOST_EXPERTS,
                "experts_sort: bad operands (%ld tokens, %d of %d experts)", tokens, top, experts);
    XRT_REQUIRE(room == xrt_experts_sort_room(tokens, top, experts) && room < (1L << 30), "experts_sort: room for %ld rows", room);
    experts_sort_kernel<<<1, 1024, 0, (hipStream_t)stream>>>(chosen, tokens * top, top, experts, xrt_linear_groups_tile(tokens * top, experts), (int)room, rows, places,
                                                             tile_group);
    XRT_LAUNCH_CHECK("experts_sort");
    return 0;
}

extern "C" int xrt_linear_groups_accepts(const void* a, int lda, const void* w, int ldw, int n, int k, int mode, const xrt_packing* packing) {
    const Packing none = {};
    return xrt_linear_groups_mfma_accepts(a, lda, w, ldw, n, k, mode, packing ? *packing : none) ? 1 : 0;
}

// out (rows of n, bfloat16 or float32) = for every tile t of `tile` rows (128 or 256) of a (bfloat16, rows lda apart)
// with tile_group[t] >= 0: its rows times the matrix at w + tile_group[t] * w_stride (rows ldw apart, k of their columns
// summed over; packed or not), mode 0, or mode 2 with an activation: act(gate) * up of a packed gated matrix of n pairs.
// parts: 1, or (mode 0) 2: k is split in two and out holds, tile after tile, the tile's rows of the first half's sums and then
// those of the second half's, for a reader that adds them (xrt_linear_groups_parts says which pays).
extern "C" int xrt_linear_groups_parts(long tiles, int n, int k, int coded_mode) { return xrt_linear_groups_splits((int)tiles, n, k, coded_mode & 255); }

extern "C" int xrt_linear_groups(const void* a, int lda, const void* w, long w_stride, int ldw, const xrt_packing* packing, void* out, int out_dtype,
                                 int tile, long tiles, int n, int k, int coded_mode, const int* tile_group, int parts, void* stream) {
    const Packing none = {};
    const int mode = coded_mode & 255, activation = coded_mode >> 8;
    XRT_REQUIRE(a && w && out && tile_group && tiles > 0 && tiles <= 65535 && n > 0 && w_stride >= 0, "linear_groups: bad operands");
    XRT_REQUIRE(out_dtype == XRT_F32 || out_dtype == XRT_BF16, "linear_groups: unknown dtype %d", out_dtype);
    XRT_REQUIRE(xrt_linear_groups_mfma_accepts(a, lda, w, ldw, n, k, mode, packing ? *packing : none),
                "linear_groups: not served (n %d, k %d, rows %d and %d apart, mode %d): k in whole tiles of 64, a gated matrix packed", n, k, lda, ldw, mode);
    XRT_REQUIRE(parts == 1 || (parts == 2 && mode == 0 && k % 128 == 0), "linear_groups: k in %d parts", parts);
    return xrt_linear_groups_mfma(a, lda, w, w_stride, ldw, out, out_dtype, tile, (int)tiles, n, k, mode, activation, tile_group,
                                  packing ? *packing : none, parts, (hipStream_t)stream);
}

extern "C" int xrt_gather_rows(const void* x, long x_stride, const int* rows, long count, int width, void* out, void* stream) {
    XRT_REQUIRE(x && rows && out && count > 0 && count < (1L << 31) && width > 0 && width % 8 == 0 && x_stride >= width && x_stride % 8 == 0 &&
                (uintptr_t)x % 16 == 0 && (uintptr_t)out % 16 == 0, "gather_rows: bfloat16 rows of a multiple of eight columns, aligned to 16 bytes");
    gather_rows_kernel<<<(unsigned)count, 256, 0, (hipStream_t)stream>>>((const bf16*)x, x_stride, rows, width, (bf16*)out);
    XRT_LAUNCH_CHECK("gather_rows");
    return 0;
}

extern "C" int xrt_experts_combine(const float* sorted, const int* places, const int* chosen, const float* weights, long tokens, int top,
                                   int experts, int width, int tile, int parts, float* out, void* stream) {
    XRT_REQUIRE(parts >= 1 && parts <= 2 && tile > 0, "experts_combine: %d parts of tiles of %d rows", parts, tile);
    XRT_REQUIRE(sorted && places && chosen && weights && out && tokens > 0 && tokens < (1L << 31) && top > 0 && experts > 0 && width > 0 &&
                width % 4 == 0 && (uintptr_t)sorted % 16 == 0 && (uintptr_t)out % 16 == 0, "experts_combine: bad operands");
    experts_combine_kernel<<<(unsigned)tokens, 256, 0, (hipStream_t)stream>>>(sorted, places, chosen, weights, top, experts, width,
                                                                              tile, parts, out);
    XRT_LAUNCH_CHECK("experts_combine");
    return 0;
}
