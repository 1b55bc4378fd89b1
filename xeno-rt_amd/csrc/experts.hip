// Choosing experts for every token, and weighting what the experts made.
//   xrt_route_experts   from router logits z [tokens][experts] (float32): scores s = sigmoid(z); the experts stand in `groups`
//                       equal groups of neighbours, a group's score is the sum of its `group_top` largest scores, only experts
//                       of the `keep` best groups can be chosen; the `top` largest scores among those are chosen, and their
//                       weights are their scores divided by the scores' sum (+ floor). Equal scores: the lower index wins.
//                       Out: weights [tokens][experts] (float32, zero for experts not chosen), and, if asked for, the chosen
//                       experts [tokens][top] (int32) in the order of their scores.
//   xrt_scale_blocks    act[t][e * width + c] *= weights[t][e]: every expert's stretch of a row times the token's weight for it
// One thread a token for the choice: the experts of a token are few (up to XRT_MOST_EXPERTS).
#include "common.h"
#include "xrt_hip.h"

namespace {

__device__ __forceinline__ float load_as_float(const void* p, int dtype, long i) {
    return dtype == XRT_F32 ? ((const float*)p)[i] : to_float(((const bf16*)p)[i]);
}
__device__ __forceinline__ void store_from_float(void* p, int dtype, long i, float v) {
    if (dtype == XRT_F32) ((float*)p)[i] = v; else ((bf16*)p)[i] = from_float<bf16>(v);
}

__global__ void __launch_bounds__(64) route_experts_kernel(const float* __restrict__ logits, long tokens, int experts, int top, int groups, int keep,
                                                           int group_top, float floor_, float* __restrict__ weights, int* __restrict__ chosen) {
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= tokens) return;
    float s[XRT_MOST_EXPERTS];
    unsigned char open[XRT_MOST_EXPERTS];          // 1: may still be chosen
    const int per_group = experts / groups;
    for (int e = 0; e < experts; ++e) {
        s[e] = 1.0f / (1.0f + expf(-logits[t * experts + e]));
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
                if (group_score[g] >= 0.f && (best < 0 || group_score[g] > group_score[best])) best = g;
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
        weights[t * experts + picks[round]] = s[picks[round]] / (sum + floor_);
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

}  // namespace

extern "C" int xrt_route_experts(const float* logits, long tokens, int experts, int top, int groups, int keep, int group_top, float floor_,
                                 float* weights, int* chosen, void* stream) {
    XRT_REQUIRE(logits && weights && tokens >= 0, "route_experts: null operand");
    XRT_REQUIRE(experts > 0 && experts <= XRT_MOST_EXPERTS && top > 0 && groups > 0 && experts % groups == 0 && keep > 0 && keep <= groups &&
                group_top > 0 && (groups == 1 || experts / groups <= 128) && top <= keep * (experts / groups),
                "route_experts: %d experts in %d groups of which %d are kept, %d chosen: up to %d experts in equal groups, and no more "
                "chosen than the kept groups hold", experts, groups, keep, top, XRT_MOST_EXPERTS);
    if (tokens == 0) return 0;
    route_experts_kernel<<<(unsigned)((tokens + 63) / 64), 64, 0, (hipStream_t)stream>>>(logits, tokens, experts, top, groups, keep, group_top,
                                                                                       floor_, weights, chosen);
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
