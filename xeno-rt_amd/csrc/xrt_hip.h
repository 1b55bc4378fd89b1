// C interface of the kernel library. Every function returns 0 on success; otherwise
// xrt_last_error() describes what was refused. Pointers are device pointers unless
// said otherwise; `stream` is a hipStream_t. Element type codes: 0 = float32, 1 = bfloat16.
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

const char* xrt_last_error(void);

// tokens in one block of the cache. A cache is [blocks][kv_heads][xrt_block_tokens() * head_dim elements], keys and
// values apart. Whoever keeps the block tables must count in the same blocks.
int xrt_block_tokens(void);
// Where the elements lie inside the part of a block that belongs to one key/value head: the element offset of dim
// `dim` of the key (of the value) of the block's token `token`. Heads whose size is a multiple of 32 lie in the order
// in which the matrix cores take them in a decode step (csrc/cache_layout.h); others as keys [token][dim], values
// [dim][token]. Host functions, for whoever wants to fill or read a cache outside the kernels.
int xrt_cache_key_offset(int token, int dim, int head_dim);
int xrt_cache_value_offset(int dim, int token, int head_dim);

// How a bfloat16 weight matrix w[rows][K] is laid out. XRT_PACK_NONE (or a null pointer wherever a packing
// is passed): rows contiguous along k. Otherwise tiles of 16 rows x 32 columns in the order in which the matrix
// cores take them, rows padded to a multiple of 16 with zeros, K a multiple of 32; the rows may also be
// regrouped so that outputs which an epilogue combines share a tile (csrc/packing.h says how):
// XRT_PACK_GATED for [gate rows | up rows] (gated_n outputs, a multiple of 8), XRT_PACK_ROTARY for rows
// [heads][head_dim] whose first rotated_heads heads are rotated over the whole head.
// Products that are bound by reading w (few rows of a) stream a packed w faster; all others take either form.
enum { XRT_PACK_NONE = 0, XRT_PACK_TILES = 1, XRT_PACK_GATED = 2, XRT_PACK_ROTARY = 3 };
typedef struct xrt_packing { int kind; int gated_n; int head_dim; int rotated_heads; } xrt_packing;
// packed[...] = w in the layout `packing` (rows padded to a multiple of 16: the packed matrix has
// (rows + 15) / 16 * 16 * K elements); XRT_PACK_GATED needs rows = 2 * gated_n, XRT_PACK_ROTARY rows a
// multiple of head_dim
int xrt_pack_weight(const void* w, void* packed, int rows, int K, const xrt_packing* packing, void* stream);
// whether packing pays for a matrix of these sizes (its tiles divide evenly among the compute units)
int xrt_packing_suits(int rows, int K);

// out[t, :] = table[ids[t], :] as float32
int xrt_embed(const void* table, int table_dtype, const xrt_packing* packing, const int* ids, float* out, int tokens,
              int hidden, int vocab, void* stream);

// out[i] = element i of the random-weights stream `key`: float(2 * (sum of twelve 10-bit fields of two
// splitmix64 words) - 12 * 1023) * scale + offset, the same values as the host-side generator gives
int xrt_random_normal(void* out, int dtype, long count, unsigned long long key, float scale, float offset,
                      void* stream);

// Probes for the benchmark's measured ceilings; nothing of the model runs through them.
// xrt_probe_read reads xrt_probe_read_bytes(bytes) bytes of `buffer` once (plain or non-temporal loads) and
// writes nothing (sink: 4 bytes that stay as they are). xrt_probe_mfma runs `iterations` rounds of four
// 32x32x16 bfloat16 matrix-core products per wavefront on tiles held in registers, in XRT_PROBE_MFMA_GROUPS
// workgroups of four wavefronts: XRT_PROBE_MFMA_GROUPS * 4 * iterations * 4 * 2 * 32 * 32 * 16 flops. Its operands
// are small whole numbers, or with random_operands numbers of either sign with random mantissas, on which
// the chip holds a lower clock.
#define XRT_PROBE_MFMA_GROUPS 512
int xrt_probe_read(const void* buffer, long bytes, int nontemporal, void* sink, void* stream);
long xrt_probe_read_bytes(long bytes);
int xrt_probe_mfma(long iterations, int random_operands, void* sink, void* stream);

// residual[i] += delta[i]
int xrt_add(float* residual, const void* delta, int delta_dtype, long count, void* stream);

// out[r, :] = rmsnorm(x[rows ? rows[r] : r, :]) * weight ; x float32, out of out_dtype
int xrt_rmsnorm(const float* x, const void* weight, int weight_dtype, float eps, void* out, int out_dtype,
                const int* rows, int n_rows, int hidden, void* stream);

// xrt_rmsnorm of every row, then xrt_short_conv of the normed rows (plain, or plus the input), for a step in which row r is the
// one new token of the sequence in slot token_slots[r] (negative: padding, the row becomes zeros): one kernel, the same bits.
int xrt_rmsnorm_conv_step(const float* x, const void* weight, int weight_dtype, float eps, void* out, int out_dtype, int n_rows,
                          int hidden, const void* conv_w, int conv_w_dtype, int taps, int plus_input, float* state,
                          const int* token_slots, void* stream);

// out[m, n] (+)= sum_k a[m, k] * w[n, k]   (mode 0 store, 1 accumulate into float32 out,
// 2 gated: out[m, n] = act(a.w[n]) * (a.w[n + N]) with w of 2N rows; the activation's code rides above the
// mode's low byte, XRT_GATED(XRT_ACT_SILU) == 2: silu(z) = z / (1 + exp(-z)) is the one that exists)
#define XRT_ACT_SILU 0
#define XRT_GATED(activation) (2 | ((activation) << 8))
// Some products (17 to 64 rows of a, or more rows and a narrow w) run faster split along k, through a workspace of float32
// sums: xrt_linear_workspace says how many floats that takes (0: none); without it the product
// takes another kernel.
int xrt_linear(const void* a, const void* w, int dtype, void* out, int out_dtype, int M, int N, int K,
               int mode, float* workspace, long workspace_floats, void* stream);
long xrt_linear_workspace(const void* a, const void* w, int dtype, int M, int N, int K, int mode);
// the same with w in the layout `packing` (null: rows contiguous along k)
int xrt_linear_with(const void* a, const void* w, const xrt_packing* packing, int dtype, void* out, int out_dtype, int M, int N,
                    int K, int mode, float* workspace, long workspace_floats, void* stream);

// xrt_linear for callers that cannot allocate device memory: code under HIP graph capture, tight serving
// loops, harnesses that forbid hipMalloc. It has no counterpart in the reference. The partial sums of a
// product split along k go to a fixed array of XRT_LINEAR_STATIC_FLOATS floats (16 MiB) that the library
// holds in device memory on every GPU it is used on; the call allocates nothing and refuses a product
// whose partial sums do not fit (xrt_linear_workspace says how many floats a product needs). Calls on one
// GPU share that array: calls that overlap there (different streams) race.
#define XRT_LINEAR_STATIC_FLOATS (4L << 20)
long xrt_linear_static_floats(void);       // XRT_LINEAR_STATIC_FLOATS, for callers that do not read this header
int xrt_linear_static(const void* a, const void* w, int dtype, void* out, int out_dtype, int M, int N, int K,
                      int mode, void* stream);

// An RMSNorm between two products, x += a w^T; y = rmsnorm(x) * gain; z = y v^T, without a kernel of
// its own. The first product (mode 1) also writes scaled_out[m, n] = bfloat16(x[m, n] * gain[n]) and
// squares_out[t * XRT_SQUARES_STRIDE + m], the sum of x[m, n]^2 over the columns n of tile t (xrt_linear_norm_tiles of them, 16 columns or fewer each). The
// second takes scaled_out as its a, squares_in (tiles_in = ceil(width_in / 16) tiles) and multiplies its
// rows by 1 / sqrt(sum of squares / width_in + eps) before its epilogue. A half left all zero is not done.
// xrt_linear_takes_norm says whether an accumulating product can write these (bfloat16 operands, up to 64 rows,
// and with more than 16 rows: split along k, N a multiple of 64); then the product after it (same rows) can
// take them, and xrt_linear_normed refuses what cannot. workspace: as for xrt_linear.
// xrt_linear_takes_norm returns 2 for an accumulating product of many rows that runs as large tiles splitting k: its second
// kernel then does the whole norm. For that, scaled_out, gain, gain_dtype and eps are set and the other fields left zero:
// scaled_out[m, n] = bfloat16((x[m, n] / rms(x[m, :])) * gain[n]), the norm kernel's result to the bit, which the product after
// it takes like any rows. Its workspace has xrt_linear_whole_norm_workspace(...) floats.
#define XRT_SQUARES_STRIDE 64
typedef struct xrt_linear_norm {
    const float* squares_in; int tiles_in; int width_in; float eps;
    void* scaled_out; const void* gain; int gain_dtype; float* squares_out;
} xrt_linear_norm;
int xrt_linear_takes_norm(const void* a, const void* w, const xrt_packing* packing, int dtype, int M, int N, int K, int mode);
int xrt_linear_norm_tiles(const void* a, const void* w, const xrt_packing* packing, int dtype, int M, int N, int K);   // rows of the table at squares_out
long xrt_linear_whole_norm_workspace(const void* a, const void* w, int dtype, int M, int N, int K, int mode);
int xrt_linear_normed(const void* a, const void* w, const xrt_packing* packing, int dtype, void* out, int out_dtype, int M, int N,
                      int K, int mode, const xrt_linear_norm* norm, float* workspace, long workspace_floats, void* stream);

// per-head RMSNorm of q and k (optional), rotation of q and k (optional), write of k and v
// into the cache (optional); qkv rows are [q heads | k heads | v heads]. longest_run: the most
// consecutive tokens that one sequence brings (0 if unknown); it only picks the faster way to
// write the values
int xrt_qkv_prepare(void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                    const int* positions, const int* slots,
                    const void* q_norm, const void* k_norm, int norm_dtype, float norm_eps,
                    const float* rope_theta, int rope_dim, float rope_scale,
                    void* k_cache, void* v_cache, const int* block_table, int table_stride, int n_blocks,
                    int longest_run, void* stream);

// The q/k/v projection qkv = a w^T followed by xrt_qkv_prepare (same arguments), in one kernel where a
// decode step allows it (bfloat16, at most 16 rows, no head norms), else in two. norm: null, or the
// squares_in half of an RMSNorm before the projection (then a is what xrt_linear_normed would take).
// workspace as for xrt_linear.
int xrt_linear_qkv(const void* a, const void* w, const xrt_packing* packing, int dtype, void* qkv, int M, int K, const xrt_linear_norm* norm,
                   int n_heads, int n_kv_heads, int head_dim, const int* positions, const int* slots,
                   const void* q_norm, const void* k_norm, int norm_dtype, float norm_eps,
                   const float* rope_theta, int rope_dim, float rope_scale,
                   void* k_cache, void* v_cache, const int* block_table, int table_stride, int n_blocks,
                   int longest_run, float* workspace, long workspace_floats, void* stream);

// causal attention of every token of a step over its sequence's cache. The sequences of the
// step may be described (seq_* arrays, n_seqs, the largest token count of a sequence and the
// longest sequence after the step): then the matrix-core kernels can be used; a decode step (max_count 1)
// then needs a workspace of xrt_attention_workspace(...) floats for the partial results of the parts that
// its keys are cut into (0: none), and takes the general kernel without it. distance_slopes (null: none): one
// float per query head; a key at position j then adds slope * (j - P) to the scaled score of the query at
// position P, for position encodings that act on the scores (the general kernel serves them).
long xrt_attention_workspace(int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim, int window,
                             int max_count, int max_context);
// A decode step (every sequence brings one token) of bfloat16 heads of 64 or 128 dims can leave to the attention what
// xrt_qkv_prepare would do between the projection and it: qkv then holds the projection as it came, and the attention
// kernel norms the heads of q and k (q_norm null: no head norms), rotates them over the whole head (rope_table null: no
// rotation; rope_dim must be head_dim), uses the new key and value and writes them into the cache, which must be
// writable. The cosines and sines of the rotation are read from rope_table, which xrt_rope_table has made and which
// must cover the step's positions (table_positions >= the longest sequence after the step).
// xrt_attention_finishes_qkv says whether a step is one that xrt_attention_finishing takes.
typedef struct xrt_qkv_finish {
    const void* q_norm; const void* k_norm; int norm_dtype; float norm_eps;
    int rope_dim; const float* rope_table; int table_positions;
} xrt_qkv_finish;
// table[p][i] = (cos, sin) of the angle p * rope_scale / rope_theta[i] for p < positions, i < rope_dim / 2, float32:
// the values that the kernels which rotate work out for themselves
int xrt_rope_table(const float* rope_theta, int rope_dim, float rope_scale, int positions, float* table, void* stream);
int xrt_attention_finishes_qkv(int dtype, int n_heads, int n_kv_heads, int head_dim, int window, int max_count, int rope_dim,
                               int table_positions, int max_context);
int xrt_attention_finishing(const void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                            void* k_cache, void* v_cache, const int* block_table, int table_stride,
                            int n_blocks, const int* positions, const int* slots, void* out, float scale,
                            const xrt_qkv_finish* finish, int max_context, float* workspace, long workspace_floats, void* stream);
int xrt_attention(const void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                  const void* k_cache, const void* v_cache, const int* block_table, int table_stride,
                  int n_blocks, const int* positions, const int* slots, void* out, float scale, int window,
                  const float* distance_slopes, const int* seq_offsets, const int* seq_slots, const int* seq_starts, int n_seqs,
                  int max_count, int max_context, float* workspace, long workspace_floats, void* stream);

// one token per row of float32 logits. With a workspace of xrt_sample_workspace(rows, vocab) bytes (0: this
// vocabulary gains nothing from it) rows with a top-k of 1 to 64 are sampled from candidates that
// workgroups find slice by slice, instead of in eight passes over the row; without, all rows take the passes.
// The penalty of row r reads history[history_spans[2r] .. history_spans[2r + 1]); with append_at (may be
// null) the row's token is also written to history[append_at[r]] (nowhere if that is negative), so that a
// caller can keep the sequences' tokens on the device.
int xrt_sample(const float* logits, int rows, int vocab, int* out, const float* temperature,
               const int* top_k, const float* top_p, const float* penalty, int* history,
               const int* history_spans, const int* append_at, const float* uniforms, void* workspace,
               long workspace_bytes, void* stream);
long xrt_sample_workspace(int rows, int vocab);

// ---- mixing along the sequence with state of fixed size per sequence (csrc/sequence_state.hip) -------------------------
// A step's sequences are described by seq_offsets [n_seqs + 1] (where each one's tokens begin among the packed tokens) and
// seq_slots [n_seqs] (negative: padding, whose output rows become zeros); per-sequence state is indexed by slot.

// Causal convolution over time on each channel: out[o][t][c] = sum_j w[o][c][j] * x[t - taps + 1 + j][c] with the inputs
// before the step taken from state [slots][taps - 1][channels] (float32; zeros at a sequence's start), which afterwards holds
// the sequence's last taps - 1 inputs. x rows are x_stride elements apart; out is [n_out][tokens][channels] of x's type.
// XRT_CONV_PLUS_INPUT adds x[t][c]; XRT_CONV_TOWARDS_LAST (taps 2, w [n_out][channels]) gives x + (x[t - 1] - x) * w.
enum { XRT_CONV_PLAIN = 0, XRT_CONV_PLUS_INPUT = 1, XRT_CONV_TOWARDS_LAST = 2 };
enum { XRT_CONV_ACT_NONE = 0, XRT_CONV_ACT_SILU = 1 };
// The same with a bias [n_out][channels] (of the filters' type, or null) added to every sum and an activation applied to the
// result, and with a result of a type of its own (bfloat16 of float32 inputs: the state then keeps the inputs unrounded).
int xrt_short_conv_with(const void* x, int dtype, long tokens, long x_stride, int channels, const void* w, int w_dtype, int taps,
                        int n_out, int mode, float* state, const int* seq_offsets, const int* seq_slots, int n_seqs, int max_count,
                        void* out, int out_dtype, const void* bias, int activation, void* stream);
int xrt_short_conv(const void* x, int dtype, long tokens, long x_stride, int channels, const void* w, int w_dtype, int taps,
                   int n_out, int mode, float* state, const int* seq_offsets, const int* seq_slots, int n_seqs, int max_count,
                   void* out, void* stream);

// Per head a state S [dim][vdim] (float32, state [slots][heads][dim][vdim]): with q, k (rows of heads x dim, times q_scale and
// k_scale) and v (heads x vdim) of every token in turn  S <- diag(decay) S + k v^T  and  o = S^T q;  with a bonus u [heads][dim]
// the token is read before the update, o = (S + diag(u) k v^T)^T q. The decay of a key channel: decay[head] for all tokens
// (XRT_DECAY_PER_HEAD), or from decay [tokens][heads * dim] (float32) plus decay_bias [heads * dim] (or null): the number itself
// (GIVEN), exp(-exp(z)) (EXP_NEG_EXP) or sigmoid(z)^decay_power (SIGMOID_POWER). Then, per head: o / sqrt(mean(o^2) + eps) if
// norm, times norm_weight ([vdim] for all heads, or [heads * vdim]) if given, times gate (rows of heads x vdim of the element
// type, through silu with XRT_GATE_SILU) if given; out rows are heads x vdim.
// XRT_DECAY_STEP: a step size per token and head, step = softplus(decay[token][head] + decay_bias[head]) with decay rows
// decay_stride apart; all channels of the head decay by exp(-exp(decay_rate[head]) * step), and v enters the state times step.
// qk_heads (0: as many as heads): heads of q and k; head h reads head h / (heads / qk_heads) of them. skip [heads]: o += skip * v.
// norm_groups > 0 (with norm): the gate comes first, then the token's whole row of heads x vdim is divided by the root mean
// square of each of its norm_groups equal parts, times norm_weight [heads * vdim]. gate_is_float32: the gate's rows are float32
// whatever the element type.
enum { XRT_DECAY_PER_HEAD = 0, XRT_DECAY_GIVEN = 1, XRT_DECAY_EXP_NEG_EXP = 2, XRT_DECAY_SIGMOID_POWER = 3, XRT_DECAY_STEP = 4 };
enum { XRT_GATE_PLAIN = 0, XRT_GATE_SILU = 1, XRT_GATE_SIGMOID = 2 };
typedef struct {
    const void *q, *k, *v;
    long q_stride, k_stride, v_stride;
    int heads, dim, vdim;
    float q_scale, k_scale;
    int decay_mode;
    const float* decay;
    const void* decay_bias;
    int decay_bias_dtype;
    float decay_power;
    const void* bonus;
    int bonus_dtype;
    float* state;
    int norm;
    float eps;
    const void* norm_weight;
    int norm_weight_dtype, norm_weight_per_head;
    const void* gate;
    long gate_stride;
    int gate_act;
    void* out;
    long decay_stride;
    const void* decay_rate;
    int decay_rate_dtype;
    int qk_heads;
    const void* skip;
    int skip_dtype;
    int norm_groups;
    int gate_is_float32;
    int input_silu;          // q, k and v are silu of what the pointers hold
    int gate_after_norm;     // with norm_groups: norm and weight first, then the gate
} xrt_recurrence;
// token_slots [tokens]: the slot of every token's sequence. The workspace holds the raw outputs and, where a long prompt is cut
// into segments that run side by side, the segments' states; xrt_linear_recurrence_workspace says how many floats.
long xrt_linear_recurrence_workspace(int n_seqs, int max_count, long tokens, int heads, int dim, int vdim);
int xrt_linear_recurrence(const xrt_recurrence* args, int dtype, const int* seq_offsets, const int* seq_slots, int n_seqs,
                          int max_count, const int* token_slots, long tokens, float* workspace, long workspace_floats, void* stream);

// residual[r] += scale * (x0[r] / rms(x0[r]) * gain0 + x1[r] / rms(x1[r]) * gain1); x float32 [rows][width], x1 may be null
int xrt_add_normed(float* residual, const float* x0, const void* gain0, const float* x1, const void* gain1, int gain_dtype,
                   long rows, int width, float eps, float scale, void* stream);

// out[i] = f(x[i]): tanh, silu, or xIELU with params = (p, q): z > 0: softplus(p) z^2 + z / 2, else (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2
enum { XRT_UNARY_TANH = 0, XRT_UNARY_SILU = 1, XRT_UNARY_XIELU = 2 };
int xrt_activation(const void* x, int x_dtype, void* out, int out_dtype, long count, int kind, const void* params, int params_dtype,
                   void* stream);

// out[t] += table[ids[t]] (out float32 [tokens][width]; ids outside the table's rows add nothing)
int xrt_rows_add(const void* table, int dtype, const int* ids, float* out, long tokens, int width, int rows, void* stream);

// The step's keys (rows of n_kv_heads x head_dim) and values (n_kv_heads x value_dim) into the cache at their tokens' places.
int xrt_kv_store(const void* k, long k_stride, const void* v, long v_stride, int dtype, long tokens, int n_kv_heads, int head_dim,
                 int value_dim, const int* positions, const int* slots, void* k_cache, void* v_cache, const int* block_table,
                 int table_stride, int n_blocks, void* stream);

// The general attention kernel with values of a width of their own and, with sink, one more key that has no value: its score is 0,
// or, with sink_scores (float32 [n_heads]), the head's own number, which is neither scaled nor biased.
// q_stride: 0 (rows of qkv are q, k and v side by side), or the distance between the rows of q where they lie alone (keys and
// values are read from the cache only). distance_bias: null, or float32 [n_heads][bias_span]: a key d tokens behind the query
// adds distance_bias[h][min(d, bias_span - 1)] to its scaled score (any bias that is a function of head and distance and
// stays constant from some distance on). chunk: 0, or the size of the stretches that positions are cut into from a
// sequence's first token on; a query then sees only the keys of its own stretch (at or before it).
int xrt_attention_general(const void* qkv, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim, int value_dim,
                          const void* k_cache, const void* v_cache, const int* block_table, int table_stride, int n_blocks,
                          const int* positions, const int* slots, void* out, float scale, int window,
                          const float* distance_slopes, int sink, const float* sink_scores, long q_stride, const float* distance_bias,
                          int bias_span, int chunk, void* stream);

// The matrix-core attention for a step that brings sequences of many tokens, with the queries alone in q (rows q_stride
// apart; keys and values are in the cache) and, with chunk > 0, queries that see the keys of their own stretch of `chunk`
// positions only. `accepts` says which element type, head sizes and stretches it serves (stretches of whole cache blocks).
// Tokens of the step that belong to no sequence keep what `out` held. distance_bias (float32 [n_heads][bias_span], or null) and
// sink_scores (float32 [n_heads], or null) as in xrt_attention_general.
int xrt_attention_stretches_accepts(int dtype, int head_dim, int value_dim, int chunk);
int xrt_attention_stretches(const void* q, long q_stride, int dtype, int tokens, int n_heads, int n_kv_heads, int head_dim,
                            const void* k_cache, const void* v_cache, const int* block_table, int table_stride, int n_blocks,
                            const int* seq_offsets, const int* seq_slots, const int* seq_starts, int n_seqs, void* out,
                            float scale, int chunk, const float* distance_bias, int bias_span, const float* sink_scores, void* stream);

// Attention without a softmax: the weight of a visible key is sigmoid(score_h + head_bias[h]), not normalised over the keys;
// before that the heads' scaled scores of a (query, key) pair are mixed, score_h <- sum_g head_mix[h][g] score_g
// (head_mix float32 [n_heads][n_heads], or null); a head's summed values are multiplied by sigmoid(gate[token][h]) (float32
// rows gate_stride apart, or null). q: rows of n_heads x head_dim, q_stride apart; out rows n_heads x value_dim; keys and
// values come from the cache (the step's own included, which must have been written). window 0: none. A step of few tokens
// runs faster shared out among more workgroups, through a workspace of xrt_attention_sigmoid_workspace(...) floats (0:
// not needed; max_context: the longest sequence after the step, 0 if unknown); without it the step runs a workgroup a
// token, to the same bits.
long xrt_attention_sigmoid_workspace(long tokens, int n_heads, int head_dim, int value_dim, int window, int max_context);
int xrt_attention_sigmoid(const void* q, long q_stride, int dtype, long tokens, int n_heads, int n_kv_heads, int head_dim,
                          int value_dim, const void* k_cache, const void* v_cache, const int* block_table, int table_stride,
                          int n_blocks, const int* positions, const int* slots, void* out, float scale, int window,
                          const float* head_mix, const float* head_bias, const float* gate, long gate_stride,
                          int max_context, float* workspace, long workspace_floats, void* stream);

// Between an attention's projection (float32 sums, rows [q heads | k heads | v heads | anything], proj_stride apart) and its
// scores: biases ([heads * dim] each, or null); an RMS norm of every head of q and k with one weight [head_dim] each (or
// null); a rotation of the first rot_dims dims of every head of q and k by the angles position * frequencies[pair]
// (frequencies float32 [rot_dims / 2], or null; pairs of neighbours (2n, 2n + 1), or of halves (n, n + rot_dims / 2); cosines
// and sines times magnitude); values_out (or null) takes the values as projected (float32 [tokens][n_kv_heads * value_dim]);
// with values_in (same shape, or null) v <- (1 - lambda) v + lambda values_in, lambda one number on the device; q goes to
// q_out (element type `dtype`, rows q_stride apart), k and v into the cache (or nowhere, if the caches are null). Biases, norm
// weights and lambda have the element type small_dtype. plain_norm: the head norm without a gain (norm_q and norm_k null).
// temp_every > 0: the queries of the token at position p are multiplied by 1 + temp_coef * ln(floor((p + 1) / temp_every) + 1).
// queries_only: the rows of proj hold [q heads | anything] and nothing is written but q_out.
int xrt_qkv_complete(const float* proj, long proj_stride, int dtype, long tokens, int n_heads, int n_kv_heads, int head_dim,
                   int value_dim, const void* bias_q, const void* bias_k, const void* bias_v, const void* norm_q,
                   const void* norm_k, float norm_eps, int small_dtype, const float* frequencies, int rot_dims,
                   int neighbours, float magnitude, const float* values_in, float* values_out, const void* lambda,
                   const int* positions, const int* slots, void* q_out, long q_stride, void* k_cache, void* v_cache,
                   const int* block_table, int table_stride, int n_blocks, int plain_norm, float temp_coef, int temp_every,
                   int queries_only, void* stream);

// Layer norm of whole rows, y = (x - mean) / sqrt(mean of squared deviations + eps) * weight + bias; x float32, weight and
// bias of w_dtype. xrt_layernorm: out[r] = norm(x[rows ? rows[r] : r]).
int xrt_layernorm(const float* x, const void* weight, const void* bias, int w_dtype, float eps, void* out, int out_dtype,
                  const int* rows, int n_rows, int hidden, void* stream);
// The norm h of every row, then out[r] = h[r] + (h_before - h[r]) * mix, where h_before is the norm of the row before it if
// that row is a token of the same sequence (token_slots), else the sequence's state (state [slots][hidden] float32, zeros
// for a sequence that starts); afterwards the state holds the norm of the sequence's last row. Padding rows (slot < 0): zeros.
int xrt_layernorm_shift(const float* x, const void* weight, const void* bias, const void* mix, int w_dtype, float eps,
                        float* state, const int* token_slots, const int* seq_offsets, const int* seq_slots, int n_seqs,
                        int max_count, void* out, int out_dtype, int n_rows, int hidden, void* stream);
// residual[r] += scale * norm(y[r] + pre_bias) (pre_bias [hidden] or null); with next_out the kernel goes on to
// next_out[r] = the layer norm (next_weight, next_bias, next_eps) of the row of the residual it has just written.
int xrt_add_layernormed(float* residual, const float* y, const void* pre_bias, const void* weight, const void* bias, int w_dtype,
                        float eps, float scale, const void* next_weight, const void* next_bias, float next_eps, void* next_out,
                        int out_dtype, long rows, int hidden, void* stream);

// ---- the selective scan (csrc/selective_scan.hip) ----------------------------------------------------------------------
// Per channel c a state [n] (float32, state [slots][channels][n]): with step = softplus(step[t][c] + step_bias[c]) of every
// token in turn  S[c][j] <- exp(step * A[c][j]) S[c][j] + step x[t][c] b[t][j],  y = sum_j S[c][j] c[t][j] + skip[c] x[t][c],
// A = -exp(a_log) ([channels][n]); out = y * silu(gate[t][c]) (gate may be null). x, out: element type dtype; step, b, c:
// float32; step_bias, a_log, skip: small_dtype; gate: gate_dtype. Rows lie their strides apart; out rows are `channels` wide.
typedef struct {
    const void* x; long x_stride; int dtype;
    const float* step; long step_stride;
    const void* step_bias;
    const float* b; long b_stride;
    const float* c; long c_stride;
    const void* a_log;
    const void* skip;
    int small_dtype;
    const void* gate; long gate_stride; int gate_dtype;
    float* state;
    void* out;
    int channels, n;
} xrt_selective_scan_args;
long xrt_selective_scan_workspace(int n_seqs, int max_count, long tokens, int channels, int n);
int xrt_selective_scan(const xrt_selective_scan_args* args, const int* seq_offsets, const int* seq_slots, int n_seqs, int max_count,
                       const int* token_slots, long tokens, float* workspace, long workspace_floats, void* stream);

// ---- what a token brings beside its embedding row, and small operations on rows (csrc/token_inputs.hip) -----------------
// x[t] <- x[t] * scale + table[row(t)] (x float32 [tokens][width]; table [buckets + 1][width], or null: the scale alone).
// row(t) = (before * mul_prev + id * mul_cur) mod buckets with `before` the token before t in its sequence: the one at the
// packed place before it if that is the same sequence's, else before[slot] (what the step before left; int32 [slots]); a
// sequence's first token (position 0) reads row `buckets`. Afterwards before[slot] is the sequence's last token of the step.
int xrt_bigram_add(float* x, long tokens, int width, float scale, const void* table, int table_dtype, int buckets, int mul_prev,
                   int mul_cur, const int* ids, const int* positions, const int* slots, const int* seq_offsets,
                   const int* seq_slots, int n_seqs, int* before, void* stream);
// out[t][c] = gelu_tanh(s[t][c]) * table[ids[t]][offset + c] for c < width; s float32 rows s_stride apart; table [rows][table_width]
int xrt_gated_rows(const float* s, long s_stride, const void* table, int table_dtype, long table_width, long offset, int rows,
                   const int* ids, void* out, int out_dtype, long tokens, int width, void* stream);
// residual += sum over n < count of scales[n] * gains[n][column] * y[n] (y float32 [rows][width]; a null gain is all ones);
// copy (or null): the updated rows once more, in copy_dtype
int xrt_add_weighted(float* residual, int count, const float* const* y, const void* const* gains, const float* scales, int gain_dtype,
                     long rows, int width, void* copy, int copy_dtype, void* stream);
// out[r][c] = g * sigmoid(alpha * g) * (u + 1), g = min(sums[r][c], limit), u = clamp(sums[r][n + c], -limit, limit); times
// row_weights[r] (float32 [rows]) unless that is null
int xrt_glu_clamped(const float* sums, void* out, int out_dtype, long rows, int n, float limit, float alpha, const float* row_weights,
                    void* stream);
// x <- cap * tanh(x / cap), float32 in place
int xrt_softcap(float* x, long count, float cap, void* stream);
int xrt_cast(const void* x, int x_dtype, void* out, int out_dtype, long count, void* stream);

// ---- experts (csrc/experts.hip) --------------------------------------------------------------------------------------------
// The choice of experts for every token from router logits [tokens][experts] (float32): scores sigmoid(z); `groups` equal
// groups of neighbours, a group's score the sum of its group_top largest scores, experts of the `keep` best groups stay
// open; the `top` largest open scores are chosen; weights [tokens][experts] (float32) get score / (sum of the chosen scores
// + floor) for the chosen and 0 for the others; chosen (or null) [tokens][top] the experts in the order of their scores.
// softmax != 0: the scores are softmax(z) over all experts instead; scale multiplies the chosen experts' weights.
#define XRT_MOST_EXPERTS 256
int xrt_route_experts(const float* logits, long tokens, int experts, int top, int groups, int keep, int group_top, float floor_,
                      float* weights, int* chosen, int softmax, float scale, void* stream);
// act[t][e * width + c] *= weights[t][e]
int xrt_scale_blocks(void* act, int dtype, const float* weights, long tokens, int experts, int width, void* stream);

// Experts that multiply only the tokens that chose them. xrt_experts_sort puts a step's picks (chosen [tokens][top]) in the
// order of their experts, every expert's stretch filled up to whole tiles of xrt_linear_groups_tile_rows() rows (128, or 256 where an expert has some hundred picks on average): rows [room]
// takes the token of every row (-1: filling), places [tokens][top] the row of every pick, tile_group [room / tile] the expert
// of every tile (-1: beyond the last); room is xrt_experts_sort_room(). xrt_gather_rows copies rows of bfloat16 x (zeros
// where rows[r] < 0). xrt_linear_groups multiplies every tile of rows of a with the matrix of its tile's group, w + group *
// w_stride (elements), whose rows lie ldw apart and of which k columns are summed over (coded_mode as in xrt_linear_with: 0,
// or 2 | activation << 8 with a packed gated matrix of n pairs per group); `accepts` says what it serves.
// xrt_experts_combine: out[t] = sum over the picks of t, in their order, of weights[t][chosen[t][k]] * sorted[places[t][k]].
int xrt_linear_groups_tile_rows(long tokens, int top, int experts);
long xrt_experts_sort_room(long tokens, int top, int experts);
int xrt_experts_sort(const int* chosen, long tokens, int top, int experts, int* rows, long room, int* places, int* tile_group, void* stream);
int xrt_gather_rows(const void* x, long x_stride, const int* rows, long count, int width, void* out, void* stream);
int xrt_linear_groups_accepts(const void* a, int lda, const void* w, int ldw, int n, int k, int mode, const xrt_packing* packing);
// parts: 1, or with plain sums 2: k in two halves whose sums lie tile after tile, [tiles][parts][tile rows][n], for
// xrt_experts_combine to add (xrt_linear_groups_parts: which of the two pays, from the number of tiles).
int xrt_linear_groups_parts(long tiles, int n, int k, int coded_mode);
int xrt_linear_groups(const void* a, int lda, const void* w, long w_stride, int ldw, const xrt_packing* packing, void* out, int out_dtype,
                      int tile, long tiles, int n, int k, int coded_mode, const int* tile_group, int parts, void* stream);
int xrt_experts_combine(const float* sorted, const int* places, const int* chosen, const float* weights, long tokens, int top, int experts,
                        int width, int tile, int parts, float* out, void* stream);

// ---- a residual stream in several copies (csrc/streams.hip) ------------------------------------------------------------------
// streams: float32 [tokens][copies][width]. open: every copy is the token's row of x. read: out[r] = norm(sum over the copies s
// of in[s] * copy s of token rows[r] (or r)), the norm being u / sqrt(mean(u^2) + eps) * gain, or u itself with a null gain.
// write: all copies at once from the old ones, copy t <- sum over s of mix[s][t] * copy s + out_weights[t] * y (y float32
// [tokens][width]); with next_in the read of the new copies under next_in, gain and eps goes to `normed` in the same pass.
// in, mix and out_weights are float32 on the device.
#define XRT_MOST_STREAMS 8
int xrt_streams_open(const float* x, float* streams, long tokens, int width, int copies, void* stream);
int xrt_streams_read(const float* streams, int copies, const float* in, const void* gain, int gain_dtype, float eps, void* out,
                     int out_dtype, const int* rows, long n_rows, int width, void* stream);
int xrt_streams_write(float* streams, int copies, const float* mix, const float* out_weights, const float* y, long tokens, int width,
                      const float* next_in, const void* gain, int gain_dtype, float eps, void* normed, int normed_dtype, void* stream);

// ---- attention through a latent (csrc/latent.hip) ---------------------------------------------------------------------------
// The cache of such a layer has one key/value head whose keys are [latent (rank) | turned key part (rot_dim)] and whose values
// are the latent. complete: from float32 rows [latent | key part] (down_stride apart) the latent / rms(latent) * gain and the
// key part with its first rot_dims turned in pairs of neighbours by position * frequencies[pair], into the cache, and, with
// rows_out, once more as rows [tokens][rank + rot_dim] of the cache's element type (zeros for tokens of no sequence).
// queries: from float32 rows of heads x [plain (dim) | part to turn (rot_dim)] the plain parts to `plain` [tokens][heads][dim]
// and the turned parts to full[t][h][rank ..], rows full_stride apart, heads rank + rot_dim apart.
// linear_heads: out[t][h][n] = sum over k of a[t][h][k] * w[h][n][k]; rows of a and out a_stride and out_stride apart, heads
// a_head and out_head apart; all three of `dtype`, float32 sums (whose order depends on whether the step has up to 16 rows or more and on
// the sizes, on nothing else: a row's result never depends on the rows around it).
int xrt_latent_complete(const float* down, long down_stride, int dtype, long tokens, int rank, int rot_dim, int rot_dims,
                        const void* gain, int gain_dtype, float eps, const float* frequencies, const int* positions, const int* slots,
                        void* k_cache, void* v_cache, const int* block_table, int table_stride, int n_blocks, void* rows_out, void* stream);
// causal_softmax: scores float32 [rows][keys], row m being the query at position first_position + m / heads of head m % heads;
// rounded and rest (bfloat16, same shape) get the weight of every key at or before the query, exp(score * scale) over the sum
// of those and exp(sinks[head]) (sinks float32 [heads], or null), as the rounded number and what the rounding left; 0 elsewhere.
// transpose: dst[c][r] = src[r][c] for r < rows, c < cols; rows of src src_stride apart, dst [cols][rows].
int xrt_causal_softmax(const float* scores, long rows, long keys, int heads, int first_position, float scale, const float* sinks,
                       void* rounded, void* rest, void* stream);
int xrt_transpose(const void* src, long src_stride, int dtype, long rows, int cols, void* dst, void* stream);
int xrt_latent_queries(const float* q, long q_stride, int dtype, long tokens, int heads, int dim, int rot_dim, int rot_dims,
                       const float* frequencies, const int* positions, void* plain, void* full, long full_stride, int rank, void* stream);
int xrt_linear_heads(const void* a, long a_stride, long a_head, const void* w, int dtype, void* out, long out_stride, long out_head,
                     long rows, int heads, int n, int k, void* stream);

// ---- many heads on one key/value head with large keys, on the matrix cores (csrc/attention_latent.hip) ------------------------
// Causal attention of the step's tokens (queries alone in q, rows q_stride apart, n_heads x head_dim each) over a cache with one
// key/value head, keys of head_dim and values of value_dim numbers (multiples of 32 up to 512: `accepts`), bfloat16; with
// sink_scores (float32 [n_heads], or null) the softmax's denominator also holds exp(sink_scores[head]). out: rows of
// n_heads x value_dim. max_context: the longest sequence after this step; the workspace holds `xrt_attention_latent_workspace` floats.
int xrt_attention_latent_accepts(int dtype, int n_kv_heads, int head_dim, int value_dim);
long xrt_attention_latent_workspace(long tokens, int n_heads, int value_dim, int max_context);
int xrt_attention_latent(const void* q, long q_stride, long tokens, int n_heads, int head_dim, int value_dim, const void* k_cache,
                         const void* v_cache, const int* block_table, int table_stride, int n_blocks, const int* positions,
                         const int* slots, void* out, float scale, const float* sink_scores, int max_context, float* workspace,
                         long workspace_floats, void* stream);

#ifdef __cplusplus
}
#endif
