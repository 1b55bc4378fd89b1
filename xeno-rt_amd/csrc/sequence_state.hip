// Mixing along the sequence with state of fixed size per sequence, and the small operations around it:
//   xrt_short_conv          causal convolution over time on each channel (a few taps), the last taps - 1 inputs kept per sequence;
//                           also as "input plus convolution" and as the interpolation between a token and the one before it
//   xrt_linear_recurrence   per head a matrix state S [dim x vdim]: S <- diag(decay) S + k v^T, read with q before or after the
//                           update; the decay a constant per head, given per token and channel, or worked out here from a
//                           projection (two forms); then per head an RMS norm, a weight and a gate
//   xrt_add_normed          residual += scale * sum of RMS-normed rows with their gains
//   xrt_activation          tanh, silu, and the two-parameter activation xIELU, elementwise
//   xrt_rows_add            out[t] += table[ids[t]]
//   xrt_kv_store            the step's keys and values into the paged cache, values of a width of their own
// Everything that is state, a decay, a norm or a sum onto the residual stream is float32 whatever the element type of the
// activations. A sequence's tokens are worked off in their order and nothing depends on where a step begins or on which
// other sequences the step holds, so a request gives the same bits however it is cut into steps and batched.
// Sequences whose slot is negative are padding: their rows of the output are zeros and no state is touched.
#include "cache_layout.h"
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

// ---- short convolution -----------------------------------------------------------------------------------------

constexpr int CONV_MAX_TAPS = 16;
constexpr int CONV_SEGMENT = 16;          // tokens of a sequence that one workgroup walks
constexpr int CONV_THREADS = 256;         // channels of a workgroup

// Input `at` (counted from the step's first token of the sequence; negative: before the step) of channel c.
template <typename T>
__device__ __forceinline__ float conv_input(const T* __restrict__ x, long x_stride, int begin, int at, const float* __restrict__ state,
                                            int taps, int channels, int c) {
    if (at >= 0) return to_float(x[(long)(begin + at) * x_stride + c]);
    return state[(long)(taps - 1 + at) * channels + c];
}

// grid (sequences, segments, channel chunks). phase 0: outputs only; 1: outputs and the state (one segment per sequence);
// 2: the state only (a launch of its own after phase 0, so that no workgroup reads a state another one is writing).
// bias [n_out][channels] of the filters' type (or null) is added to the sum, then the activation (XRT_CONV_ACT_*) is applied.
template <typename TI, typename T>
__global__ void __launch_bounds__(CONV_THREADS) short_conv_kernel(
    const TI* __restrict__ x, long x_stride, int channels, const void* __restrict__ w, int w_dtype, int taps, int n_out, int mode,
    float* __restrict__ state, const int* __restrict__ seq_offsets, const int* __restrict__ seq_slots, T* __restrict__ out,
    long tokens, int phase, const void* __restrict__ bias, int activation) {
#pragma clang fp contract(off)      // (only the products and sums written as fmaf are fused: the same in every kernel that does this convolution)
    const int seq = blockIdx.x, c = blockIdx.z * CONV_THREADS + threadIdx.x;
    if (c >= channels) return;
    const int begin = seq_offsets[seq], count = seq_offsets[seq + 1] - begin, slot = seq_slots[seq];
    const int first = blockIdx.y * CONV_SEGMENT, last = min(count, first + CONV_SEGMENT);
    if (first >= count && !(phase == 2 && first == 0)) return;
    if (slot < 0) {
        if (phase != 2)
            for (int o = 0; o < n_out; ++o)
                for (int t = first; t < last; ++t) out[((long)o * tokens + begin + t) * channels + c] = from_float<T>(0.f);
        return;
    }
    float* mine = state + (long)slot * (taps - 1) * channels;
    float window[CONV_MAX_TAPS - 1];
    if (phase == 2) {                                      // what the sequence's last taps - 1 inputs are after this step
#pragma unroll
        for (int m = 0; m < CONV_MAX_TAPS - 1; ++m)
            if (m < taps - 1) window[m] = conv_input(x, x_stride, begin, count - (taps - 1) + m, mine, taps, channels, c);
#pragma unroll
        for (int m = 0; m < CONV_MAX_TAPS - 1; ++m)
            if (m < taps - 1) mine[(long)m * channels + c] = window[m];
        return;
    }
#pragma unroll
    for (int m = 0; m < CONV_MAX_TAPS - 1; ++m)
        window[m] = m < taps - 1 ? conv_input(x, x_stride, begin, first - (taps - 1) + m, mine, taps, channels, c) : 0.f;
    for (int t = first; t < last; ++t) {
        const float now = to_float(x[(long)(begin + t) * x_stride + c]);
        for (int o = 0; o < n_out; ++o) {
            float y;
            if (mode == XRT_CONV_TOWARDS_LAST) {           // taps == 2: x + (the input before - x) * w
                y = fmaf(window[0] - now, load_as_float(w, w_dtype, (long)o * channels + c), now);
            } else {
                const long w_at = ((long)o * channels + c) * taps;
                y = 0.f;
#pragma unroll
                for (int m = 0; m < CONV_MAX_TAPS - 1; ++m)
                    if (m < taps - 1) y = fmaf(load_as_float(w, w_dtype, w_at + m), window[m], y);
                y = fmaf(load_as_float(w, w_dtype, w_at + taps - 1), now, y);
                if (mode == XRT_CONV_PLUS_INPUT) y += now;
            }
            if (bias != nullptr) y += load_as_float(bias, w_dtype, (long)o * channels + c);
            if (activation == XRT_CONV_ACT_SILU) y = silu_exact(y);
            out[((long)o * tokens + begin + t) * channels + c] = from_float<T>(y);
        }
#pragma unroll
        for (int m = 0; m < CONV_MAX_TAPS - 2; ++m) window[m] = window[m + 1];
        if (taps >= 2) {
#pragma unroll
            for (int m = 0; m < CONV_MAX_TAPS - 1; ++m)
                if (m == taps - 2) window[m] = now;
        }
    }
    if (phase == 1) {
#pragma unroll
        for (int m = 0; m < CONV_MAX_TAPS - 1; ++m)
            if (m < taps - 1) mine[(long)m * channels + c] = window[m];
    }
}

// ---- linear recurrence -----------------------------------------------------------------------------------------
// A wavefront owns 64 columns of one head's state, a lane one column: S[0 .. dim) in registers. The token's q, k and decays
// lie across the lanes (lane l holds channels l, l + 64, ...), are brought into their final form there (scales, the decay's
// exponentials), and reach the products as scalar operands, one lane's value at a time; the next token's loads are on their
// way meanwhile. A long prompt is cut into segments of tokens that run side by side: first every segment but a sequence's
// last works out what it adds to the state from empty hands (L) and the product of its decays (P); then the states at the
// segments' beginnings follow from S <- P S + L in their order; then every segment runs again from its true state and
// writes the outputs. The heads' norm, weight and gate are a pass of their own over the raw outputs.

constexpr int REC_SEGMENT = 32;           // fewest tokens of a segment
constexpr int REC_WAVES_WANTED = 4096;    // segments are made until the launch has about this many wavefronts (a few to every SIMD)

constexpr int REC_SPLIT_ROWS = 32;        // rows of the state that a wavefront takes where the rows of a head are split

struct RecurrencePlan {
    int vslices, segment, segments;       // wavefronts per head; tokens per segment; segments of the longest sequence
    int row_split;                        // wavefronts that share the rows of a head's state (their outputs are added afterwards)
    long raw_floats, state_floats, decay_floats;
};

RecurrencePlan recurrence_plan(int n_seqs, int max_count, long tokens, int heads, int dim, int vdim) {
    RecurrencePlan p;
    p.vslices = (vdim + XRT_WAVE - 1) / XRT_WAVE;
    const long row = (long)max(1, n_seqs) * heads * p.vslices;
    const long wanted = max(1L, (REC_WAVES_WANTED + row - 1) / row);
    const long length = (max_count + wanted - 1) / wanted;
    p.segment = (int)max((long)REC_SEGMENT, (length + 15) / 16 * 16);
    p.segments = max(1, (max_count + p.segment - 1) / p.segment);
    // A step of few tokens a sequence (a decode step above all) has little to do and much to wait for: the rows of a state
    // are then dealt to wavefronts of REC_SPLIT_ROWS rows each. The rule looks at the longest run of tokens only, never at
    // how many sequences there are, so a request's bits do not depend on what else is in the batch.
    p.row_split = max_count <= REC_SEGMENT ? (dim + REC_SPLIT_ROWS - 1) / REC_SPLIT_ROWS : 1;
    p.raw_floats = tokens * heads * vdim * p.row_split;
    p.state_floats = p.segments > 1 ? (long)n_seqs * (p.segments + 1) * heads * dim * vdim : 0;
    p.decay_floats = p.segments > 1 ? (long)n_seqs * p.segments * heads * dim : 0;
    return p;
}

__device__ __forceinline__ float lane_value(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// What a token brings, across the lanes: channel lane + 64 m in element m. Channels beyond dim read as q = k = 0, decay = 1.
template <int M>
struct TokenInputs {
    float q[M], k[M], d[M], v;
};

// XRT_DECAY_STEP: the token's step size of a head, softplus(z + bias), from decay [tokens][decay_stride] and decay_bias [heads]
__device__ __forceinline__ float step_of(const xrt_recurrence& a, long row, int head) {
    float z = a.decay[row * a.decay_stride + head];
    if (a.decay_bias != nullptr) z += load_as_float(a.decay_bias, a.decay_bias_dtype, head);
    return softplus_exact(z);
}
// the head of q and k that `head` reads: heads may share them in groups of neighbours
__device__ __forceinline__ int qk_head_of(const xrt_recurrence& a, int head) {
    return a.qk_heads > 0 && a.qk_heads < a.heads ? head / (a.heads / a.qk_heads) : head;
}

// The decay of key channel `at` (head * dim + channel) at the token in `row`.
__device__ __forceinline__ float decay_of(const xrt_recurrence& a, long row, int head, long at) {
    if (a.decay_mode == XRT_DECAY_PER_HEAD) return a.decay[head];
    float z = a.decay[row * (long)a.heads * a.dim + at];
    if (a.decay_bias != nullptr) z += load_as_float(a.decay_bias, a.decay_bias_dtype, at);
    if (a.decay_mode == XRT_DECAY_EXP_NEG_EXP) return expf(-expf(z));
    if (a.decay_mode == XRT_DECAY_SIGMOID_POWER) return expf(-softplus_exact(-z) * a.decay_power);       // sigmoid(z)^power
    return z;
}

// rows: the channels row0 .. row0 + rows of the head are this wavefront's
template <int M>
__device__ __forceinline__ void load_token(TokenInputs<M>& in, const xrt_recurrence& a, int dtype, long row, int head, int column, bool owner,
                                           int row0, int rows) {
    const int lane = threadIdx.x;
    const bool stepped = a.decay_mode == XRT_DECAY_STEP;
    float step = 1.f, stepped_decay = 1.f;
    if (stepped) {                                         // one decay for the head's channels, and the step also scales what is fed
        step = step_of(a, row, head);
        stepped_decay = expf(-expf(load_as_float(a.decay_rate, a.decay_rate_dtype, head)) * step);
    }
    const int qk_head = qk_head_of(a, head);
#pragma unroll
    for (int m = 0; m < M; ++m) {
        const int i = lane + XRT_WAVE * m;
        in.q[m] = 0.f; in.k[m] = 0.f; in.d[m] = 1.f;
        if (i < rows) {
            const long at = (long)head * a.dim + row0 + i, qk_at = (long)qk_head * a.dim + row0 + i;
            float q = load_as_float(a.q, dtype, row * a.q_stride + qk_at), k = load_as_float(a.k, dtype, row * a.k_stride + qk_at);
            if (a.input_silu) { q = silu_exact(q); k = silu_exact(k); }
            in.q[m] = q * a.q_scale;
            in.k[m] = k * a.k_scale;
            in.d[m] = stepped ? stepped_decay : decay_of(a, row, head, at);
        }
    }
    float v = owner ? load_as_float(a.v, dtype, row * a.v_stride + (long)head * a.vdim + column) : 0.f;
    if (a.input_silu) v = silu_exact(v);
    in.v = v * step;
}

// grid (sequences, heads * vslices * row_split, segments), one wavefront each. With row_split > 1 (one segment only) a wavefront
// has DIM rows of the state, and what it writes to raw, into a part of its own, is its rows' share of the outputs. With a bonus
// the token is read before it enters the state; what its own k v^T adds to its output is left to the pass over the raw outputs.
// FINAL false: a segment from empty hands, no outputs: its L to states[seq][segment], its P to decays[seq][segment].
// FINAL true: from the state at the segment's beginning (the cache's for a sequence in one segment, else states[...]: entry
// `segments` for the first segment, entry c - 1 for segment c), raw outputs to raw [tokens][heads * vdim]; a sequence's last
// segment leaves the state in the cache.
template <int DIM, bool BONUS, bool FINAL>
__global__ void __launch_bounds__(XRT_WAVE) recurrence_kernel(const xrt_recurrence a, int dtype, const int* __restrict__ seq_offsets,
                                                             const int* __restrict__ seq_slots, int segment, int segments, int vslices, int row_split,
                                                             float* __restrict__ states, float* __restrict__ decays, float* __restrict__ raw_all,
                                                             long tokens) {
    constexpr int M = (DIM + XRT_WAVE - 1) / XRT_WAVE;
    const int seq = blockIdx.x, part = blockIdx.y % row_split, head = blockIdx.y / row_split / vslices, vslice = blockIdx.y / row_split % vslices;
    const int lane = threadIdx.x;
    const int begin = seq_offsets[seq], count = seq_offsets[seq + 1] - begin, slot = seq_slots[seq];
    const int first = blockIdx.z * segment, last = min(count, first + segment);
    if (first >= count) return;
    const int vdim = a.vdim, heads = a.heads;
    const int row0 = row_split > 1 ? part * DIM : 0, dim = min(row_split > 1 ? DIM : a.dim, a.dim - row0);     // this wavefront's rows
    float* raw = raw_all + (long)part * tokens * heads * vdim;
    const int column = vslice * XRT_WAVE + lane;
    const bool owner = column < vdim;
    const bool ends_sequence = last == count, whole = count <= segment;
    if (!FINAL && ends_sequence) return;                   // nobody asks what a sequence's last segment adds
    if (slot < 0) {
        if (FINAL && owner)
            for (int t = first; t < last; ++t) raw[(long)(begin + t) * heads * vdim + (long)head * vdim + column] = 0.f;
        return;
    }
    const long per_head = (long)a.dim * vdim;
    float* cached = a.state + ((long)slot * heads + head) * per_head + (long)row0 * vdim + column;
    float* at_segment = states + (((long)seq * (segments + 1) + blockIdx.z) * heads + head) * per_head + column;
    float S[DIM];
    if (FINAL) {
        const float* from = whole ? cached
                                  : states + (((long)seq * (segments + 1) + (blockIdx.z == 0 ? segments : blockIdx.z - 1)) * heads + head) * per_head + column;
#pragma unroll
        for (int i = 0; i < DIM; ++i) S[i] = owner && i < dim ? from[(long)i * vdim] : 0.f;
    } else {
#pragma unroll
        for (int i = 0; i < DIM; ++i) S[i] = 0.f;
    }
    float product[M];
#pragma unroll
    for (int m = 0; m < M; ++m) product[m] = 1.f;

    TokenInputs<M> now, next;
    load_token<M>(now, a, dtype, begin + first, head, column, owner, row0, dim);
    for (int t = first; t < last; ++t) {
        if (t + 1 < last) load_token<M>(next, a, dtype, begin + t + 1, head, column, owner, row0, dim);
        float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int g = 0; g < DIM / 16; ++g) {
            if (g * 16 < dim) {                            // (channels from dim up to the next multiple of 16 hold zeros and stay zero)
                // (the group's scalars are taken from the lanes here and not earlier: all of a token's would not fit the scalar registers)
                asm volatile("" : "+v"(now.q[g * 16 / XRT_WAVE]), "+v"(now.k[g * 16 / XRT_WAVE]), "+v"(now.d[g * 16 / XRT_WAVE]));
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int i = g * 16 + e;
                    const float s_k = lane_value(now.k[i / XRT_WAVE], i % XRT_WAVE);
                    const float s_d = lane_value(now.d[i / XRT_WAVE], i % XRT_WAVE);
                    const float kv = s_k * now.v;
                    if constexpr (FINAL) {
                        const float s_q = lane_value(now.q[i / XRT_WAVE], i % XRT_WAVE);
                        if constexpr (BONUS) {             // the token reads the state as the tokens before it left it
                            o[e % 4] = fmaf(S[i], s_q, o[e % 4]);
                            S[i] = fmaf(s_d, S[i], kv);
                        } else {
                            S[i] = fmaf(s_d, S[i], kv);
                            o[e % 4] = fmaf(S[i], s_q, o[e % 4]);
                        }
                    } else {
                        S[i] = fmaf(s_d, S[i], kv);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);         // (one group's scalars at a time: all of a token's would not fit the scalar registers)
            }
        }
        if constexpr (FINAL) {
            float out = (o[0] + o[1]) + (o[2] + o[3]);
            if (owner) raw[(long)(begin + t) * heads * vdim + (long)head * vdim + column] = out;
        } else {
#pragma unroll
            for (int m = 0; m < M; ++m) product[m] *= now.d[m];
        }
        now = next;
    }
    if (FINAL) {
        if (ends_sequence && owner) {
#pragma unroll
            for (int i = 0; i < DIM; ++i)
                if (i < dim) cached[(long)i * vdim] = S[i];
        }
    } else {
        if (owner) {
#pragma unroll
            for (int i = 0; i < DIM; ++i)
                if (i < dim) at_segment[(long)i * vdim] = S[i];
        }
        if (vslice == 0) {
#pragma unroll
            for (int m = 0; m < M; ++m)
                if (lane + XRT_WAVE * m < dim)
                    decays[(((long)seq * segments + blockIdx.z) * heads + head) * a.dim + lane + XRT_WAVE * m] = product[m];
        }
    }
}

// The states at the segments' beginnings, in place of what the segments add: entry `segments` takes the cache's state (the first
// segment's), entry c what segment c + 1 starts from. grid (sequences, heads * vslices, dim): a wavefront a row of the state,
// a lane a column; the segments' additions are fetched eight at a time before the chain of products that needs them.
__global__ void __launch_bounds__(XRT_WAVE) recurrence_combine_kernel(const xrt_recurrence a, const int* __restrict__ seq_offsets,
                                                                     const int* __restrict__ seq_slots, int segment, int segments, int vslices,
                                                                     float* __restrict__ states, const float* __restrict__ decays) {
    const int seq = blockIdx.x, head = blockIdx.y / vslices, column = blockIdx.y % vslices * XRT_WAVE + threadIdx.x, i = blockIdx.z;
    const int count = seq_offsets[seq + 1] - seq_offsets[seq], slot = seq_slots[seq];
    if (slot < 0 || count <= segment || column >= a.vdim) return;
    const int mine = (count + segment - 1) / segment;      // this sequence's segments
    const long per_head = (long)a.dim * a.vdim, within = (long)i * a.vdim + column;
    float s = a.state[((long)slot * a.heads + head) * per_head + within];
    float* entries = states + ((long)seq * (segments + 1) * a.heads + head) * per_head + within;      // entry c: + c * heads * per_head
    const float* products = decays + ((long)seq * segments * a.heads + head) * a.dim + i;               // of segment c: + c * heads * dim
    entries[(long)segments * a.heads * per_head] = s;
    for (int c0 = 0; c0 + 1 < mine; c0 += 8) {
        float added[8], decay[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const bool there = c0 + e + 1 < mine;
            added[e] = there ? entries[(long)(c0 + e) * a.heads * per_head] : 0.f;
            decay[e] = there ? products[(long)(c0 + e) * a.heads * a.dim] : 0.f;
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (c0 + e + 1 < mine) {
                s = fmaf(decay[e], s, added[e]);
                entries[(long)(c0 + e) * a.heads * per_head] = s;
            }
        }
    }
}

__device__ __forceinline__ float gate_value(float g, int act) {
    return act == XRT_GATE_SILU ? silu_exact(g) : act == XRT_GATE_SIGMOID ? 1.0f / (1.0f + expf(-g)) : g;
}

// The heads' raw outputs of one token: norm over vdim, weight, gate. A wavefront per (token, head).
__global__ void __launch_bounds__(XRT_WAVE) recurrence_finish_kernel(const xrt_recurrence a, int dtype, const float* __restrict__ raw,
                                                                    const int* __restrict__ token_slots, int row_split, long tokens) {
    const long row = blockIdx.x;
    const int head = blockIdx.y, lane = threadIdx.x, vdim = a.vdim;
    const long out_at = row * a.heads * vdim + (long)head * vdim;
    if (token_slots[row] < 0) {
        for (int c = lane; c < vdim; c += XRT_WAVE) store_from_float(a.out, dtype, out_at + c, 0.f);
        return;
    }
    // what the token's own k v^T adds to its output where it is read with a bonus: v * sum over the channels of bonus * k * q
    float bonus_dot = 0.f;
    if (a.bonus != nullptr) {
        for (int i = lane; i < a.dim; i += XRT_WAVE) {
            const long at = (long)head * a.dim + i, qk_at = (long)qk_head_of(a, head) * a.dim + i;
            const float k = load_as_float(a.k, dtype, row * a.k_stride + qk_at) * a.k_scale, q = load_as_float(a.q, dtype, row * a.q_stride + qk_at) * a.q_scale;
            bonus_dot = fmaf(load_as_float(a.bonus, a.bonus_dtype, at) * k, q, bonus_dot);
        }
        bonus_dot = wave_sum(bonus_dot);
    }
    // the parts of the wavefronts that shared the state's rows, in their order
    auto whole = [&](int c) {
        float sum = raw[out_at + c];
        for (int part = 1; part < row_split; ++part) sum += raw[(long)part * tokens * a.heads * vdim + out_at + c];
        if (a.bonus != nullptr) sum = fmaf(bonus_dot, load_as_float(a.v, dtype, row * a.v_stride + (long)head * vdim + c), sum);
        if (a.skip != nullptr) sum = fmaf(load_as_float(a.skip, a.skip_dtype, head), load_as_float(a.v, dtype, row * a.v_stride + (long)head * vdim + c), sum);
        return sum;
    };
    float inv = 1.f;
    if (a.norm) {
        float squares = 0.f;
        for (int c = lane; c < vdim; c += XRT_WAVE) { const float o = whole(c); squares = fmaf(o, o, squares); }
        inv = 1.0f / sqrtf(wave_sum(squares) / (float)vdim + a.eps);
    }
    for (int c = lane; c < vdim; c += XRT_WAVE) {
        float value = whole(c) * inv;
        if (a.norm_weight != nullptr)
            value *= load_as_float(a.norm_weight, a.norm_weight_dtype, a.norm_weight_per_head ? (long)head * vdim + c : c);
        if (a.gate != nullptr) {
            const float g = load_as_float(a.gate, a.gate_is_float32 ? XRT_F32 : dtype, row * a.gate_stride + (long)head * vdim + c);
            value *= gate_value(g, a.gate_act);
        }
        store_from_float(a.out, dtype, out_at + c, value);
    }
}

// The same for a norm that comes after the gate and spans equal parts of the token's whole row (heads x vdim), whatever the
// heads are: value = raw (+ skip * v) times the gate, then divided by the root mean square of its part, times the weight
// [heads * vdim]. A workgroup per (token, part); a thread keeps up to FINISH_KEPT of its gated values in registers between the
// pass that sums their squares and the pass that writes them (columns beyond that are worked out twice).
constexpr int FINISH_THREADS = 512, FINISH_KEPT = 8;
__global__ void __launch_bounds__(FINISH_THREADS) recurrence_finish_groups_kernel(const xrt_recurrence a, int dtype, const float* __restrict__ raw,
                                                                                 const int* __restrict__ token_slots, int row_split, long tokens) {
    __shared__ float scratch[32];
    const long row = blockIdx.x;
    const int width = a.heads * a.vdim, part_width = width / a.norm_groups, c0 = blockIdx.y * part_width;
    const long out_at = row * width;
    if (token_slots[row] < 0) {
        for (int c = threadIdx.x; c < part_width; c += FINISH_THREADS) store_from_float(a.out, dtype, out_at + c0 + c, 0.f);
        return;
    }
    auto finished = [&](float sum, int c) {                // the parts' sum of column c of the whole row, with the skip and the gate
        if (a.skip != nullptr) sum = fmaf(load_as_float(a.skip, a.skip_dtype, c / a.vdim), load_as_float(a.v, dtype, row * a.v_stride + c), sum);
        if (a.gate != nullptr && !a.gate_after_norm) {
            const float g = load_as_float(a.gate, a.gate_is_float32 ? XRT_F32 : dtype, row * a.gate_stride + c);
            sum *= gate_value(g, a.gate_act);
        }
        return sum;
    };
    auto late_gate = [&](int c) {                          // the gate of column c of the whole row, where it follows the norm
        if (a.gate == nullptr || !a.gate_after_norm) return 1.f;
        return gate_value(load_as_float(a.gate, a.gate_is_float32 ? XRT_F32 : dtype, row * a.gate_stride + c), a.gate_act);
    };
    auto gated = [&](int c) {
        float sum = raw[out_at + c];
        for (int part = 1; part < row_split; ++part) sum += raw[(long)part * tokens * width + out_at + c];
        return finished(sum, c);
    };
    // the kept columns' parts are asked for side by side, part after part (a decode step's rows come in many parts, and column
    // after column every load would wait for the one before it); each column's sum still adds its parts in their order
    float kept[FINISH_KEPT];
    float squares = 0.f;
#pragma unroll
    for (int i = 0; i < FINISH_KEPT; ++i) kept[i] = 0.f;
#pragma unroll 2
    for (int part = 0; part < row_split; ++part) {
        const float* from = raw + (long)part * tokens * width + out_at + c0;
#pragma unroll
        for (int i = 0; i < FINISH_KEPT; ++i) {
            const int c = threadIdx.x + i * FINISH_THREADS;
            if (c < part_width) kept[i] = part == 0 ? from[c] : kept[i] + from[c];
        }
    }
    // likewise what the skip and the gate read: every kind of load for all kept columns at once, the element types decided
    // outside the loops (inside, each column's loads would wait for the column before)
    auto load_kept = [&](const void* from, bool is_float32, long at, long step, float (&into)[FINISH_KEPT]) {
        if (is_float32) {
#pragma unroll
            for (int i = 0; i < FINISH_KEPT; ++i) {
                const int c = threadIdx.x + i * FINISH_THREADS;
                into[i] = c < part_width ? ((const float*)from)[at + (long)c * step] : 0.f;
            }
        } else {
#pragma unroll
            for (int i = 0; i < FINISH_KEPT; ++i) {
                const int c = threadIdx.x + i * FINISH_THREADS;
                into[i] = c < part_width ? to_float(((const bf16*)from)[at + (long)c * step]) : 0.f;
            }
        }
    };
    if (a.skip != nullptr) {
        float values[FINISH_KEPT];
        load_kept(a.v, dtype == XRT_F32, row * a.v_stride + c0, 1, values);
#pragma unroll
        for (int i = 0; i < FINISH_KEPT; ++i) {
            const int c = min(threadIdx.x + i * FINISH_THREADS, part_width - 1);
            kept[i] = fmaf(load_as_float(a.skip, a.skip_dtype, (c0 + c) / a.vdim), values[i], kept[i]);
        }
    }
    float gates[FINISH_KEPT];
#pragma unroll
    for (int i = 0; i < FINISH_KEPT; ++i) gates[i] = 1.f;
    if (a.gate != nullptr) {
        load_kept(a.gate, a.gate_is_float32 || dtype == XRT_F32, row * a.gate_stride + c0, 1, gates);
#pragma unroll
        for (int i = 0; i < FINISH_KEPT; ++i) gates[i] = gate_value(gates[i], a.gate_act);
        if (!a.gate_after_norm) {
#pragma unroll
            for (int i = 0; i < FINISH_KEPT; ++i) { kept[i] *= gates[i]; gates[i] = 1.f; }
        }
    }
#pragma unroll
    for (int i = 0; i < FINISH_KEPT; ++i) {
        const int c = threadIdx.x + i * FINISH_THREADS;
        if (c >= part_width) kept[i] = 0.f;
        squares = fmaf(kept[i], kept[i], squares);
    }
    for (int c = threadIdx.x + FINISH_KEPT * FINISH_THREADS; c < part_width; c += FINISH_THREADS) { const float o = gated(c0 + c); squares = fmaf(o, o, squares); }
    const float inv = 1.0f / sqrtf(block_sum(squares, scratch) / (float)part_width + a.eps);
    float weights[FINISH_KEPT];
#pragma unroll
    for (int i = 0; i < FINISH_KEPT; ++i) weights[i] = 1.f;
    if (a.norm_weight != nullptr) load_kept(a.norm_weight, a.norm_weight_dtype == XRT_F32, c0, 1, weights);
#pragma unroll
    for (int i = 0; i < FINISH_KEPT; ++i) {
        const int c = threadIdx.x + i * FINISH_THREADS;
        if (c < part_width) store_from_float(a.out, dtype, out_at + c0 + c, kept[i] * inv * weights[i] * gates[i]);
    }
    for (int c = threadIdx.x + FINISH_KEPT * FINISH_THREADS; c < part_width; c += FINISH_THREADS) {
        float value = gated(c0 + c) * inv;
        if (a.norm_weight != nullptr) value *= load_as_float(a.norm_weight, a.norm_weight_dtype, c0 + c);
        store_from_float(a.out, dtype, out_at + c0 + c, value * late_gate(c0 + c));
    }
}

// ---- residual += scale * sum_n rms(x_n) * gain_n --------------------------------------------------------------

__global__ void __launch_bounds__(256) add_normed_kernel(float* __restrict__ residual, const float* __restrict__ x0, const void* __restrict__ g0,
                                                         const float* __restrict__ x1, const void* __restrict__ g1, int gain_dtype,
                                                         int width, float eps, float scale) {
    __shared__ float scratch[32];
    const long row = blockIdx.x;
    const float* in[2] = {x0, x1};
    const void* gains[2] = {g0, g1};
    float inv[2] = {0.f, 0.f};
    for (int n = 0; n < 2; ++n) {
        if (in[n] == nullptr) continue;
        float squares = 0.f;
        for (int c = threadIdx.x; c < width; c += blockDim.x) squares = fmaf(in[n][row * width + c], in[n][row * width + c], squares);
        inv[n] = 1.0f / sqrtf(block_sum(squares, scratch) / (float)width + eps);
    }
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        float sum = 0.f;
        for (int n = 0; n < 2; ++n)
            if (in[n] != nullptr) sum += in[n][row * width + c] * inv[n] * load_as_float(gains[n], gain_dtype, c);
        residual[row * width + c] += scale * sum;
    }
}

// ---- activations -------------------------------------------------------------------------------------------------

__global__ void activation_kernel(const void* __restrict__ x, int x_dtype, void* __restrict__ out, int out_dtype, long count, int kind,
                                  const void* __restrict__ params, int params_dtype) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    const float z = load_as_float(x, x_dtype, i);
    float y;
    if (kind == XRT_UNARY_TANH) {
        y = tanhf(z);
    } else if (kind == XRT_UNARY_SILU) {
        y = silu_exact(z);
    } else {                                               // xIELU with the numbers (p, q)
        const float p = load_as_float(params, params_dtype, 0), q = load_as_float(params, params_dtype, 1);
        if (z > 0.f) y = fmaf(softplus_exact(p) * z, z, 0.5f * z);
        else y = fmaf(0.5f + softplus_exact(q), expm1f(z) - z, 0.5f * z);
    }
    store_from_float(out, out_dtype, i, y);
}

template <typename T>
__global__ void rows_add_kernel(const T* __restrict__ table, const int* __restrict__ ids, float* __restrict__ out, int width, int rows) {
    const long token = blockIdx.x;
    const int id = ids[token];
    if (id < 0 || id >= rows) return;
    for (int c = threadIdx.x; c < width; c += blockDim.x) out[token * width + c] += to_float(table[(long)id * width + c]);
}

// one wavefront per (token, key/value head)
template <typename T>
__global__ void kv_store_kernel(const T* __restrict__ k, long k_stride, const T* __restrict__ v, long v_stride, int n_kv_heads, int head_dim,
                                int value_dim, const int* __restrict__ positions, const int* __restrict__ slots, T* __restrict__ k_cache,
                                T* __restrict__ v_cache, const int* __restrict__ block_table, int table_stride, int n_blocks) {
    const int token = blockIdx.x / n_kv_heads, kv_head = blockIdx.x % n_kv_heads, lane = threadIdx.x;
    const int slot = slots[token], pos = positions[token];
    if (slot < 0) return;
    const int block = block_table[(long)slot * table_stride + pos / XRT_BLOCK_TOKENS];
    if (block < 0 || block >= n_blocks) return;
    const int within = pos % XRT_BLOCK_TOKENS;
    const long key_base = ((long)block * n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * head_dim;
    const long value_base = ((long)block * n_kv_heads + kv_head) * XRT_BLOCK_TOKENS * value_dim;
    for (int e = lane; e < head_dim; e += XRT_WAVE)
        k_cache[key_base + cache_key_offset(within, e, head_dim)] = k[(long)token * k_stride + (long)kv_head * head_dim + e];
    for (int e = lane; e < value_dim; e += XRT_WAVE)
        v_cache[value_base + cache_value_offset(e, within, value_dim)] = v[(long)token * v_stride + (long)kv_head * value_dim + e];
}

}  // namespace

extern "C" int xrt_short_conv_with(const void* x, int dtype, long tokens, long x_stride, int channels, const void* w, int w_dtype, int taps,
                                   int n_out, int mode, float* state, const int* seq_offsets, const int* seq_slots, int n_seqs, int max_count,
                                   void* out, int out_dtype, const void* bias, int activation, void* stream) {
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "short_conv: unknown dtype %d", dtype);
    XRT_REQUIRE(out_dtype == dtype || (dtype == XRT_F32 && out_dtype == XRT_BF16), "short_conv: the result has the input's type, or is bfloat16 of float32 inputs");
    XRT_REQUIRE(w_dtype == XRT_F32 || w_dtype == XRT_BF16, "short_conv: unknown weight dtype %d", w_dtype);
    XRT_REQUIRE(x && w && (state || taps == 1) && seq_offsets && seq_slots && out, "short_conv: null operand");
    XRT_REQUIRE(taps >= 1 && taps <= CONV_MAX_TAPS, "short_conv: %d taps, 1 to %d are served", taps, CONV_MAX_TAPS);
    XRT_REQUIRE(mode == XRT_CONV_PLAIN || mode == XRT_CONV_PLUS_INPUT || (mode == XRT_CONV_TOWARDS_LAST && taps == 2),
                "short_conv: unknown mode %d (the interpolation towards the input before has two taps)", mode);
    XRT_REQUIRE(activation == XRT_CONV_ACT_NONE || activation == XRT_CONV_ACT_SILU, "short_conv: unknown activation %d", activation);
    XRT_REQUIRE(channels > 0 && n_out > 0 && x_stride >= channels && tokens >= 0 && n_seqs >= 0 && max_count >= 0, "short_conv: bad sizes");
    if (n_seqs == 0 || max_count == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const int segments = (max_count + CONV_SEGMENT - 1) / CONV_SEGMENT;
    const int chunks = (channels + CONV_THREADS - 1) / CONV_THREADS;
    XRT_REQUIRE(segments <= 65535 && chunks <= 65535, "short_conv: a step this long is not served");
#define XRT_CONV(TI, T, segments_, phase_)                                                                                     \
    short_conv_kernel<TI, T><<<dim3(n_seqs, segments_, chunks), CONV_THREADS, 0, s>>>((const TI*)x, x_stride, channels, w, w_dtype, taps, \
        n_out, mode, state, seq_offsets, seq_slots, (T*)out, tokens, phase_, bias, activation)
#define XRT_CONV_TYPES(segments_, phase_)                                                          \
    do {                                                                                           \
        if (dtype == XRT_F32 && out_dtype == XRT_F32) XRT_CONV(float, float, segments_, phase_);   \
        else if (dtype == XRT_F32) XRT_CONV(float, bf16, segments_, phase_);                       \
        else XRT_CONV(bf16, bf16, segments_, phase_);                                              \
    } while (0)
    if (segments == 1 || taps == 1) {                      // (one tap: no state, nothing that one workgroup writes and another reads)
        XRT_CONV_TYPES(segments, 1);
    } else {
        XRT_CONV_TYPES(segments, 0);
        XRT_CONV_TYPES(1, 2);
    }
#undef XRT_CONV_TYPES
#undef XRT_CONV
    XRT_LAUNCH_CHECK("short_conv");
    return 0;
}

extern "C" int xrt_short_conv(const void* x, int dtype, long tokens, long x_stride, int channels, const void* w, int w_dtype, int taps,
                              int n_out, int mode, float* state, const int* seq_offsets, const int* seq_slots, int n_seqs, int max_count,
                              void* out, void* stream) {
    return xrt_short_conv_with(x, dtype, tokens, x_stride, channels, w, w_dtype, taps, n_out, mode, state, seq_offsets, seq_slots, n_seqs,
                               max_count, out, dtype, nullptr, XRT_CONV_ACT_NONE, stream);
}

extern "C" long xrt_linear_recurrence_workspace(int n_seqs, int max_count, long tokens, int heads, int dim, int vdim) {
    if (n_seqs <= 0 || max_count <= 0 || tokens <= 0 || heads <= 0 || dim <= 0 || vdim <= 0) return 0;
    const RecurrencePlan p = recurrence_plan(n_seqs, max_count, tokens, heads, dim, vdim);
    return p.raw_floats + p.state_floats + p.decay_floats;
}

extern "C" int xrt_linear_recurrence(const xrt_recurrence* args, int dtype, const int* seq_offsets, const int* seq_slots, int n_seqs,
                                     int max_count, const int* token_slots, long tokens, float* workspace, long workspace_floats,
                                     void* stream) {
    XRT_REQUIRE(args != nullptr && seq_offsets && seq_slots && token_slots, "linear_recurrence: null operand");
    const xrt_recurrence a = *args;
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "linear_recurrence: unknown dtype %d", dtype);
    XRT_REQUIRE(a.q && a.k && a.v && a.state && a.out, "linear_recurrence: null operand");
    XRT_REQUIRE(a.heads > 0 && a.dim > 0 && a.dim <= 256 && a.vdim > 0 && (long)a.heads * ((a.vdim + XRT_WAVE - 1) / XRT_WAVE) <= 65535,
                "linear_recurrence: %d heads of %d x %d: key sizes up to 256 are served", a.heads, a.dim, a.vdim);
    XRT_REQUIRE(a.decay_mode >= XRT_DECAY_PER_HEAD && a.decay_mode <= XRT_DECAY_STEP && a.decay != nullptr,
                "linear_recurrence: unknown decay mode %d, or no decays", a.decay_mode);
    XRT_REQUIRE(a.decay_mode != XRT_DECAY_STEP || (a.decay_rate != nullptr && a.decay_stride >= a.heads),
                "linear_recurrence: decays from step sizes need a rate per head and the steps' row stride");
    XRT_REQUIRE(!a.input_silu || (a.bonus == nullptr && a.skip == nullptr), "linear_recurrence: activated inputs go with neither a bonus nor a skip");
    XRT_REQUIRE(!a.gate_after_norm || a.norm_groups > 0, "linear_recurrence: a gate after the norm goes with a norm over parts of the whole row");
    XRT_REQUIRE(a.gate_act >= XRT_GATE_PLAIN && a.gate_act <= XRT_GATE_SIGMOID, "linear_recurrence: unknown gate activation %d", a.gate_act);
    XRT_REQUIRE(a.qk_heads == 0 || (a.qk_heads > 0 && a.heads % a.qk_heads == 0), "linear_recurrence: %d heads cannot share %d heads of q and k", a.heads, a.qk_heads);
    XRT_REQUIRE(a.norm_groups == 0 || (a.norm != 0 && a.norm_groups > 0 && (a.heads * a.vdim) % a.norm_groups == 0 && a.norm_groups <= 65535 &&
                                       (a.norm_weight == nullptr || a.norm_weight_per_head || a.heads == 1)),
                "linear_recurrence: a norm in %d parts of a row of %d, with a weight over the whole row", a.norm_groups, a.heads * a.vdim);
    const int qk_rows = (a.qk_heads > 0 ? a.qk_heads : a.heads) * a.dim;
    XRT_REQUIRE(a.q_stride >= qk_rows && a.k_stride >= qk_rows && a.v_stride >= a.heads * a.vdim &&
                (a.gate == nullptr || a.gate_stride >= a.heads * a.vdim), "linear_recurrence: a row stride is shorter than its heads");
    XRT_REQUIRE(n_seqs >= 0 && max_count >= 0 && tokens >= 0 && tokens < (1L << 31), "linear_recurrence: bad sizes");
    if (n_seqs == 0 || tokens == 0 || max_count == 0) return 0;
    const RecurrencePlan p = recurrence_plan(n_seqs, max_count, tokens, a.heads, a.dim, a.vdim);
    XRT_REQUIRE(p.segments <= 65535, "linear_recurrence: a step this long is not served");
    XRT_REQUIRE(workspace != nullptr && workspace_floats >= p.raw_floats + p.state_floats + p.decay_floats,
                "linear_recurrence: the workspace needs %ld floats", p.raw_floats + p.state_floats + p.decay_floats);
    hipStream_t s = (hipStream_t)stream;
    float* raw = workspace;
    float* states = raw + p.raw_floats;
    float* decays = states + p.state_floats;
    const bool bonus = a.bonus != nullptr;
    XRT_REQUIRE((long)a.heads * p.vslices * p.row_split <= 65535, "linear_recurrence: too many heads for one launch");
    const dim3 grid(n_seqs, a.heads * p.vslices * p.row_split, p.segments);
#define XRT_REC(DIM_, BONUS_, FINAL_) recurrence_kernel<DIM_, BONUS_, FINAL_><<<grid, XRT_WAVE, 0, s>>>(a, dtype, seq_offsets, seq_slots, \
        p.segment, p.segments, p.vslices, p.row_split, states, decays, raw, tokens)
#define XRT_REC_DIM(BONUS_, FINAL_)                                                                \
    do {                                                                                           \
        if (a.dim <= 32 || p.row_split > 1) XRT_REC(REC_SPLIT_ROWS, BONUS_, FINAL_); else if (a.dim <= 64) XRT_REC(64, BONUS_, FINAL_); \
        else if (a.dim <= 128) XRT_REC(128, BONUS_, FINAL_); else XRT_REC(256, BONUS_, FINAL_);    \
    } while (0)
    if (p.segments > 1) {
        XRT_REC_DIM(false, false);                         // (what a segment adds to the state does not know of the bonus)
        recurrence_combine_kernel<<<dim3(n_seqs, a.heads * p.vslices, a.dim), XRT_WAVE, 0, s>>>(a, seq_offsets, seq_slots, p.segment, p.segments,
                                                                                        p.vslices, states, decays);
    }
    if (bonus) XRT_REC_DIM(true, true); else XRT_REC_DIM(false, true);
#undef XRT_REC_DIM
#undef XRT_REC
    if (a.norm_groups > 0)
        recurrence_finish_groups_kernel<<<dim3((unsigned)tokens, a.norm_groups), FINISH_THREADS, 0, s>>>(a, dtype, raw, token_slots, p.row_split, tokens);
    else
        recurrence_finish_kernel<<<dim3((unsigned)tokens, a.heads), XRT_WAVE, 0, s>>>(a, dtype, raw, token_slots, p.row_split, tokens);
    XRT_LAUNCH_CHECK("linear_recurrence");
    return 0;
}

extern "C" int xrt_add_normed(float* residual, const float* x0, const void* gain0, const float* x1, const void* gain1, int gain_dtype,
                              long rows, int width, float eps, float scale, void* stream) {
    XRT_REQUIRE(residual && x0 && gain0 && (x1 == nullptr) == (gain1 == nullptr), "add_normed: null operand");
    XRT_REQUIRE(gain_dtype == XRT_F32 || gain_dtype == XRT_BF16, "add_normed: unknown dtype %d", gain_dtype);
    XRT_REQUIRE(rows >= 0 && rows < (1L << 31) && width > 0, "add_normed: bad sizes");
    if (rows == 0) return 0;
    add_normed_kernel<<<(unsigned)rows, 256, 0, (hipStream_t)stream>>>(residual, x0, gain0, x1, gain1, gain_dtype, width, eps, scale);
    XRT_LAUNCH_CHECK("add_normed");
    return 0;
}

extern "C" int xrt_activation(const void* x, int x_dtype, void* out, int out_dtype, long count, int kind, const void* params,
                              int params_dtype, void* stream) {
    XRT_REQUIRE(x && out && count >= 0, "activation: null operand");
    XRT_REQUIRE((x_dtype == XRT_F32 || x_dtype == XRT_BF16) && (out_dtype == XRT_F32 || out_dtype == XRT_BF16), "activation: unknown dtype");
    XRT_REQUIRE(kind == XRT_UNARY_TANH || kind == XRT_UNARY_SILU || (kind == XRT_UNARY_XIELU && params != nullptr),
                "activation: unknown kind %d, or xIELU without its two numbers", kind);
    if (count == 0) return 0;
    const long blocks = (count + 255) / 256;
    XRT_REQUIRE(blocks < (1L << 31), "activation: too many elements");
    activation_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(x, x_dtype, out, out_dtype, count, kind, params, params_dtype);
    XRT_LAUNCH_CHECK("activation");
    return 0;
}

extern "C" int xrt_rows_add(const void* table, int dtype, const int* ids, float* out, long tokens, int width, int rows, void* stream) {
    XRT_REQUIRE(table && ids && out, "rows_add: null operand");
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "rows_add: unknown dtype %d", dtype);
    XRT_REQUIRE(tokens >= 0 && tokens < (1L << 31) && width > 0 && rows > 0, "rows_add: bad sizes");
    if (tokens == 0) return 0;
    if (dtype == XRT_F32) rows_add_kernel<float><<<(unsigned)tokens, 256, 0, (hipStream_t)stream>>>((const float*)table, ids, out, width, rows);
    else rows_add_kernel<bf16><<<(unsigned)tokens, 256, 0, (hipStream_t)stream>>>((const bf16*)table, ids, out, width, rows);
    XRT_LAUNCH_CHECK("rows_add");
    return 0;
}

extern "C" int xrt_kv_store(const void* k, long k_stride, const void* v, long v_stride, int dtype, long tokens, int n_kv_heads, int head_dim,
                            int value_dim, const int* positions, const int* slots, void* k_cache, void* v_cache, const int* block_table,
                            int table_stride, int n_blocks, void* stream) {
    XRT_REQUIRE(k && v && positions && slots && k_cache && v_cache && block_table, "kv_store: null operand");
    XRT_REQUIRE(dtype == XRT_F32 || dtype == XRT_BF16, "kv_store: unknown dtype %d", dtype);
    XRT_REQUIRE(tokens >= 0 && n_kv_heads > 0 && head_dim > 0 && value_dim > 0 && tokens * n_kv_heads < (1L << 31), "kv_store: bad sizes");
    XRT_REQUIRE(k_stride >= (long)n_kv_heads * head_dim && v_stride >= (long)n_kv_heads * value_dim, "kv_store: a row stride is shorter than its heads");
    if (tokens == 0) return 0;
    const unsigned items = (unsigned)(tokens * n_kv_heads);
    if (dtype == XRT_F32)
        kv_store_kernel<float><<<items, XRT_WAVE, 0, (hipStream_t)stream>>>((const float*)k, k_stride, (const float*)v, v_stride, n_kv_heads, head_dim,
            value_dim, positions, slots, (float*)k_cache, (float*)v_cache, block_table, table_stride, n_blocks);
    else
        kv_store_kernel<bf16><<<items, XRT_WAVE, 0, (hipStream_t)stream>>>((const bf16*)k, k_stride, (const bf16*)v, v_stride, n_kv_heads, head_dim,
            value_dim, positions, slots, (bf16*)k_cache, (bf16*)v_cache, block_table, table_stride, n_blocks);
    XRT_LAUNCH_CHECK("kv_store");
    return 0;
}
