// The selective scan: per channel c a state S[c][0 .. n) that every token decays and feeds with its own step size,
//   step_c = softplus(z_c + bias_c),  S[c][j] <- exp(step_c * A[c][j]) S[c][j] + step_c x_c B_j,  y_c = sum_j S[c][j] C_j + D_c x_c,
// with A = -exp(a_log), then out = y * silu(gate). B and C [n] belong to the token, not to the channel. State, steps, decays
// and sums are float32 whatever the element type of x and out.
//
// A lane owns one channel and NP consecutive entries of its state in registers; a wavefront owns 64 channels, so the loads
// of x and the steps are whole lines and B, C are the same for all lanes. A state of more than NP entries is dealt to
// several wavefronts (`parts`), whose shares of y a last kernel adds in their order. A long prompt is cut into segments that
// run side by side: every segment but a sequence's last first works out what it adds to the state from empty hands and the
// sum of its steps (the product of a segment's decays is exp(A * that sum): the decays are diagonal); the states at the
// segments' beginnings follow in order; then every segment runs from its true state and writes its outputs. How a step is
// cut depends on the longest run of tokens in it only, never on the other sequences.
// Sequences whose slot is negative are padding: zeros out, no state touched.
#include "common.h"
#include "xrt_hip.h"

namespace {

__device__ __forceinline__ float load_as_float(const void* p, int dtype, long i) {
    return dtype == XRT_F32 ? ((const float*)p)[i] : to_float(((const bf16*)p)[i]);
}
__device__ __forceinline__ void store_from_float(void* p, int dtype, long i, float v) {
    if (dtype == XRT_F32) ((float*)p)[i] = v; else ((bf16*)p)[i] = from_float<bf16>(v);
}
__device__ __forceinline__ float silu_exact(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_exact(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

constexpr int SCAN_SEGMENT = 32;          // fewest tokens of a segment
constexpr int SCAN_WAVES_WANTED = 4096;   // segments are made until a launch has about this many wavefronts

struct ScanPlan {
    int np, parts, blocks, segment, segments;
    long raw_floats, state_floats, step_floats;
};

ScanPlan scan_plan(int n_seqs, int max_count, long tokens, int channels, int n) {
    ScanPlan p;
    p.np = (n % 16 == 0 || (n > 8 && n % 8 != 0)) ? 16 : 8;
    p.parts = (n + p.np - 1) / p.np;
    p.blocks = (channels + XRT_WAVE - 1) / XRT_WAVE;
    const long row = (long)max(1, n_seqs) * p.blocks * p.parts;
    const long wanted = max(1L, (SCAN_WAVES_WANTED + row - 1) / row);
    const long length = (max_count + wanted - 1) / wanted;
    p.segment = (int)max((long)SCAN_SEGMENT, (length + 15) / 16 * 16);
    p.segments = max(1, (max_count + p.segment - 1) / p.segment);
    p.raw_floats = p.parts > 1 ? tokens * channels * p.parts : 0;
    p.state_floats = p.segments > 1 ? (long)n_seqs * (p.segments + 1) * channels * n : 0;
    p.step_floats = p.segments > 1 ? (long)n_seqs * p.segments * channels : 0;
    return p;
}

// grid (sequences * segments, channel blocks, parts), one wavefront each.
// FINAL false: a segment from empty hands: what it adds goes to states[seq][segment], the sum of its steps to steps[seq][segment].
// FINAL true: from the state at the segment's beginning (the cache's for a sequence in one segment, else states[seq][...]: entry
// `segments` for the first segment, entry s - 1 for segment s); with one part the outputs are finished here, else the part's
// share of y goes to raw[part]; a sequence's last segment leaves the state in the cache.
template <int NP, bool FINAL>
__global__ void __launch_bounds__(XRT_WAVE) selective_scan_kernel(const xrt_selective_scan_args a, const int* __restrict__ seq_offsets,
                                                                 const int* __restrict__ seq_slots, int segment, int segments, int parts,
                                                                 float* __restrict__ states, float* __restrict__ steps, float* __restrict__ raw,
                                                                 long tokens) {
    const int seq = blockIdx.x / segments, seg = blockIdx.x % segments, part = blockIdx.z;
    const int c = blockIdx.y * XRT_WAVE + threadIdx.x;
    const int begin = seq_offsets[seq], count = seq_offsets[seq + 1] - begin, slot = seq_slots[seq];
    const int first = seg * segment, last = min(count, first + segment);
    if (first >= count || c >= a.channels) return;
    const bool ends_sequence = last == count, whole = count <= segment;
    if (!FINAL && ends_sequence) return;
    const int n = a.n, n0 = part * NP;
    if (slot < 0) {
        if (FINAL) {
            for (int t = first; t < last; ++t) {
                if (parts == 1) store_from_float(a.out, a.dtype, (long)(begin + t) * a.channels + c, 0.f);
                else raw[((long)part * tokens + begin + t) * a.channels + c] = 0.f;
            }
        }
        return;
    }
    float A[NP], S[NP];
#pragma unroll
    for (int j = 0; j < NP; ++j) A[j] = n0 + j < n ? -expf(load_as_float(a.a_log, a.small_dtype, (long)c * n + n0 + j)) : 0.f;
    float* cached = a.state + ((long)slot * a.channels + c) * n + n0;
    if (FINAL) {
        const float* from = whole ? cached : states + (((long)seq * (segments + 1) + (seg == 0 ? segments : seg - 1)) * a.channels + c) * n + n0;
#pragma unroll
        for (int j = 0; j < NP; ++j) S[j] = n0 + j < n ? from[j] : 0.f;
    } else {
#pragma unroll
        for (int j = 0; j < NP; ++j) S[j] = 0.f;
    }
    const float bias = a.step_bias != nullptr ? load_as_float(a.step_bias, a.small_dtype, c) : 0.f;
    const float skip = FINAL && a.skip != nullptr ? load_as_float(a.skip, a.small_dtype, c) : 0.f;
    float step_sum = 0.f;
    for (int t = first; t < last; ++t) {
        const long row = begin + t;
        const float x = load_as_float(a.x, a.dtype, row * a.x_stride + c);
        const float step = softplus_exact(a.step[row * a.step_stride + c] + bias);
        const float fed = step * x;
        const float* B = a.b + row * a.b_stride + n0;          // (the same for all lanes)
        const float* C = a.c + row * a.c_stride + n0;
        float y0 = 0.f, y1 = 0.f;
#pragma unroll
        for (int j = 0; j < NP; ++j) {
            if (n0 + j < n) {
                S[j] = fmaf(expf(step * A[j]), S[j], fed * B[j]);
                if (FINAL) { if (j % 2 == 0) y0 = fmaf(S[j], C[j], y0); else y1 = fmaf(S[j], C[j], y1); }
            }
        }
        if (FINAL) {
            const float y = y0 + y1;
            if (parts == 1) {
                float v = fmaf(skip, x, y);
                if (a.gate != nullptr) v *= silu_exact(load_as_float(a.gate, a.gate_dtype, row * a.gate_stride + c));
                store_from_float(a.out, a.dtype, row * a.channels + c, v);
            } else {
                raw[((long)part * tokens + row) * a.channels + c] = y;
            }
        } else {
            step_sum += step;
        }
    }
    if (FINAL) {
        if (ends_sequence) {
#pragma unroll
            for (int j = 0; j < NP; ++j)
                if (n0 + j < n) cached[j] = S[j];
        }
    } else {
        float* to = states + (((long)seq * (segments + 1) + seg) * a.channels + c) * n + n0;
#pragma unroll
        for (int j = 0; j < NP; ++j)
            if (n0 + j < n) to[j] = S[j];
        if (part == 0) steps[((long)seq * segments + seg) * a.channels + c] = step_sum;
    }
}

// The states at the segments' beginnings, in place of what the segments add: entry `segments` takes the cache's state, entry s
// what segment s + 1 starts from. A thread per (sequence, channel, entry of the state).
__global__ void __launch_bounds__(256) selective_scan_combine_kernel(const xrt_selective_scan_args a, const int* __restrict__ seq_offsets,
                                                                    const int* __restrict__ seq_slots, int segment, int segments,
                                                                    float* __restrict__ states, const float* __restrict__ steps) {
    const int seq = blockIdx.y;
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;        // c * n + j
    const long per = (long)a.channels * a.n;
    if (e >= per) return;
    const int count = seq_offsets[seq + 1] - seq_offsets[seq], slot = seq_slots[seq];
    if (slot < 0 || count <= segment) return;
    const int mine = (count + segment - 1) / segment, c = (int)(e / a.n);
    const float A = -expf(load_as_float(a.a_log, a.small_dtype, e));
    float s = a.state[(long)slot * per + e];
    float* entries = states + (long)seq * (segments + 1) * per + e;
    entries[(long)segments * per] = s;
    for (int g = 0; g + 1 < mine; ++g) {
        s = fmaf(expf(A * steps[((long)seq * segments + g) * a.channels + c]), s, entries[(long)g * per]);
        entries[(long)g * per] = s;
    }
}

// the parts' shares of y in their order, the skip, the gate
__global__ void __launch_bounds__(256) selective_scan_finish_kernel(const xrt_selective_scan_args a, const float* __restrict__ raw, int parts,
                                                                   const int* __restrict__ token_slots, long tokens) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= tokens * a.channels) return;
    const long row = i / a.channels;
    const int c = (int)(i % a.channels);
    if (token_slots[row] < 0) { store_from_float(a.out, a.dtype, i, 0.f); return; }
    float y = raw[i];
    for (int part = 1; part < parts; ++part) y += raw[(long)part * tokens * a.channels + i];
    if (a.skip != nullptr) y = fmaf(load_as_float(a.skip, a.small_dtype, c), load_as_float(a.x, a.dtype, row * a.x_stride + c), y);
    if (a.gate != nullptr) y *= silu_exact(load_as_float(a.gate, a.gate_dtype, row * a.gate_stride + c));
    store_from_float(a.out, a.dtype, i, y);
}

}  // namespace

extern "C" long xrt_selective_scan_workspace(int n_seqs, int max_count, long tokens, int channels, int n) {
    if (n_seqs <= 0 || max_count <= 0 || tokens <= 0 || channels <= 0 || n <= 0) return 0;
    const ScanPlan p = scan_plan(n_seqs, max_count, tokens, channels, n);
    return p.raw_floats + p.state_floats + p.step_floats;
}

extern "C" int xrt_selective_scan(const xrt_selective_scan_args* args, const int* seq_offsets, const int* seq_slots, int n_seqs, int max_count,
                                  const int* token_slots, long tokens, float* workspace, long workspace_floats, void* stream) {
    XRT_REQUIRE(args != nullptr && seq_offsets && seq_slots && token_slots, "selective_scan: null operand");
    const xrt_selective_scan_args a = *args;
    const auto known = [](int d) { return d == XRT_F32 || d == XRT_BF16; };
    XRT_REQUIRE(known(a.dtype) && known(a.small_dtype) && known(a.gate_dtype), "selective_scan: unknown dtype");
    XRT_REQUIRE(a.x && a.step && a.b && a.c && a.a_log && a.state && a.out, "selective_scan: null operand");
    XRT_REQUIRE(a.channels > 0 && a.n > 0 && a.n <= 4096, "selective_scan: %d channels with %d entries of state each", a.channels, a.n);
    XRT_REQUIRE(a.x_stride >= a.channels && a.step_stride >= a.channels && a.b_stride >= a.n && a.c_stride >= a.n &&
                (a.gate == nullptr || a.gate_stride >= a.channels), "selective_scan: a row stride is shorter than its row");
    XRT_REQUIRE(n_seqs >= 0 && max_count >= 0 && tokens >= 0 && tokens < (1L << 31), "selective_scan: bad sizes");
    if (n_seqs == 0 || tokens == 0 || max_count == 0) return 0;
    const ScanPlan p = scan_plan(n_seqs, max_count, tokens, a.channels, a.n);
    XRT_REQUIRE((long)n_seqs * p.segments < (1L << 31) && p.blocks <= 65535 && p.parts <= 65535, "selective_scan: a step this large is not served");
    XRT_REQUIRE(p.raw_floats + p.state_floats + p.step_floats == 0 || (workspace != nullptr && workspace_floats >= p.raw_floats + p.state_floats + p.step_floats),
                "selective_scan: the workspace needs %ld floats", p.raw_floats + p.state_floats + p.step_floats);
    hipStream_t s = (hipStream_t)stream;
    float* raw = workspace;
    float* states = raw + p.raw_floats;
    float* steps = states + p.state_floats;
    const dim3 grid((unsigned)(n_seqs * p.segments), p.blocks, p.parts);
#define XRT_SCAN(NP_, FINAL_) selective_scan_kernel<NP_, FINAL_><<<grid, XRT_WAVE, 0, s>>>(a, seq_offsets, seq_slots, p.segment, p.segments, \
        p.parts, states, steps, raw, tokens)
    if (p.segments > 1) {
        if (p.np == 16) XRT_SCAN(16, false); else XRT_SCAN(8, false);
        const long per = (long)a.channels * a.n;
        selective_scan_combine_kernel<<<dim3((unsigned)((per + 255) / 256), n_seqs), 256, 0, s>>>(a, seq_offsets, seq_slots, p.segment, p.segments,
                                                                                               states, steps);
    }
    if (p.np == 16) XRT_SCAN(16, true); else XRT_SCAN(8, true);
#undef XRT_SCAN
    if (p.parts > 1) {
        const long blocks = (tokens * a.channels + 255) / 256;
        XRT_REQUIRE(blocks < (1L << 31), "selective_scan: too many elements");
        selective_scan_finish_kernel<<<(unsigned)blocks, 256, 0, s>>>(a, raw, p.parts, token_slots, tokens);
    }
    XRT_LAUNCH_CHECK("selective_scan");
    return 0;
}
