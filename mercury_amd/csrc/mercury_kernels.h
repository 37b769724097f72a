// C interface of the gfx950 kernel libraries.  This file is the one declaration of every
// entry point: the host core's table of function pointers and the ctypes signatures of the
// Python side are both derived from it (a line "// @library NAME" says which library the
// declarations after it belong to; mk_last_error and mk_abi_version are in both).
// Pointers are device pointers unless a comment says otherwise; `stream` is a hipStream_t.
// Functions validate their arguments on the host against what the kernel and its grid
// assume, return 0 on success and non-zero after recording a message for mk_last_error().
// Dtype codes: 0 = float32, 1 = bfloat16.
#pragma once

#include <hip/hip_runtime.h>

#define MK_ABI_VERSION 38

// Gate activations of a gated feed-forward: SILU is silu(g) * u; SWISH_CLAMP is
// g' * sigmoid(alpha * g') * (u' + beta) with g' = min(g, limit), u' = clamp(u, -limit, limit);
// GELU_TANH is 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))) * u.
enum { MK_ACT_SILU = 0, MK_ACT_SWISH_CLAMP = 1, MK_ACT_GELU_TANH = 2 };
// Activations of one operand: the square of relu; 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))).
enum { MK_UNARY_RELU2 = 0, MK_UNARY_GELU_TANH = 1 };
// Gates of one number per column on a mixer's output: z sigmoid(z), or sigmoid(z).
enum { MK_GATE_SILU = 0, MK_GATE_SIGMOID = 1 };
// Values mixed across layers (mk_qk_prepare): none; this layer leaves its values of the step's
// tokens in a buffer; this layer's values become (1 - lambda) v + lambda * what was left.
enum { MK_VMIX_NONE = 0, MK_VMIX_LEAVE = 1, MK_VMIX_BLEND = 2 };

#ifdef __cplusplus
extern "C" {
#endif

const char* mk_last_error();
int mk_abi_version();

// @library core: float32 arithmetic, float32 or bfloat16 storage

// out[t, :] = table[ids[t], :] * scale as float32 (the residual stream starts here).
int mk_embed(const int* ids, const void* table, int dtype, float* out, int tokens, int hidden,
             int vocab, float scale, hipStream_t stream);

// The residual stream of a step of few tokens in fixed point: 64-bit integers in units of
// 2^-32, into which projections add their results with integer atomics (the sum is the same
// in whatever order they arrive, and nothing has to add partial results up afterwards).
// mk_embed_fixed starts it; mk_rmsnorm_fixed normalises rows of it as mk_rmsnorm does rows of
// h; mk_fixed_add adds `count` float32 partial sums p[k * stride + i], i < n, into it.
int mk_embed_fixed(const int* ids, const void* table, int dtype, long long* out, int tokens,
                   int hidden, int vocab, float scale, hipStream_t stream);
int mk_rmsnorm_fixed(const long long* h64, const void* weight, int weight_dtype, float eps,
                     const int* rows, void* out, int out_dtype, int out_rows, int hidden,
                     hipStream_t stream);
int mk_fixed_add(long long* h64, const float* partials, int count, long long stride, long long n,
                 hipStream_t stream);

// logits[i] = cap * tanh(logits[i] / cap) for i < count, in place.
int mk_logit_cap(float* logits, long long count, float cap, hipStream_t stream);

// Per-request state of fixed size: rows of `state` [slots, width] (float32), a sequence's row
// being slots[token_seq[t]].  mk_state_store: every token at absolute position `at_position`
// writes its row of x [tokens, width] into its sequence's slot.  mk_state_load: every token's
// row of out is its sequence's row of the state.
int mk_state_store(const void* x, int dtype, float* state, const int* slots, const int* token_seq,
                   const int* positions, int at_position, int tokens, int width,
                   hipStream_t stream);
int mk_state_load(const float* state, const int* slots, const int* token_seq, void* out, int dtype,
                  int tokens, int width, hipStream_t stream);

// RMSNorm of rows of the float32 residual stream h, optionally after adding `num_partials`
// partial sums [p, row, hidden] (stride between partials in elements) into h.  `rows`, when
// not null, lists the rows of h to normalise; out row i then comes from h row rows[i].
int mk_rmsnorm(float* h, const float* partials, int num_partials, long long partial_stride,
               const void* weight, int weight_dtype, float eps, const int* rows, void* out,
               int out_dtype, int out_rows, int hidden, hipStream_t stream);

// The same with a say in the rounding: `once` != 0 rounds x * rstd * weight once, to the
// output type; 0 rounds the normalised value before the weight multiplies it, as mk_rmsnorm.
int mk_rmsnorm_rounding(float* h, const float* partials, int num_partials,
                        long long partial_stride, const void* weight, int weight_dtype, float eps,
                        const int* rows, void* out, int out_dtype, int out_rows, int hidden,
                        int once, hipStream_t stream);

// out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i].
int mk_silu_mul(const void* gate_up, void* out, int dtype, int tokens, int inter,
                hipStream_t stream);

// Rotary encoding of the q and k heads of qkv [T, row_stride] (q in place) and the write of
// rotated k into the paged key cache [pages, n_kv, page_size, d] and of raw v into the value
// cache, which is transposed within a page: [pages, n_kv, d, page_size].  The first `rot`
// dims of a head turn, pair j being dims (j, j + rot/2), or (2j, 2j + 1) when `interleaved`.
int mk_rope_kv_write(void* qkv, int dtype, int row_stride, const float* cos_table,
                     const float* sin_table, int table_positions, const int* positions,
                     const int* token_seq, const int* block_table, int table_stride,
                     void* k_cache, void* v_cache, int page_size, int n_q, int n_kv, int d,
                     int rot, int interleaved, int write_kv, int tokens, hipStream_t stream);

// y = x W^T (+ bias) with float32 FMA.  accumulate: y (float32) += instead of =.
int mk_linear_generic(const void* x, const void* w, int dtype, const void* bias, int bias_dtype,
                      void* out, int out_dtype, int accumulate, int M, int N, int K, int lda,
                      int ldo, hipStream_t stream);

// Causal grouped-query attention over the paged cache for any mix of prompt portions and
// decoded tokens; window = 0 means all earlier keys.  score_cap > 0: the scaled score becomes
// cap * tanh(score / cap); distance_slopes (float32 [n_q], or null): slope[head] * (query
// position - key position) is subtracted from it.
int mk_attention_generic(const void* q, int q_stride, void* out, int out_stride,
                         const void* k_cache, const void* v_cache, int dtype,
                         const int* positions, const int* token_seq, const int* block_table,
                         int table_stride, int page_size, int n_q, int n_kv, int d, float scale,
                         int window, float score_cap, const float* distance_slopes, int tokens,
                         hipStream_t stream);

// mk_rope_kv_write for a projection that arrives as float32 partial sums [p, T, width] of a
// K-split product: the slices are added in order (with the bias) before the rotation; q goes
// to q_out [T, n_q d].
int mk_qkv_finish(const float* partials, int num_partials, long long partial_stride,
                  const void* bias, int bias_dtype, void* q_out, int dtype,
                  const float* cos_table, const float* sin_table, int table_positions,
                  const int* positions, const int* token_seq, const int* block_table,
                  int table_stride, void* k_cache, void* v_cache, int page_size, int n_q,
                  int n_kv, int d, int rot, int write_kv, int tokens, hipStream_t stream);

// out[i] = mean + std * normal(key, i) for i < n, rounded to the dtype: the values the host
// core's fill computes for the same key (random_normal.h), so random weights are the same
// numbers wherever they are drawn.
int mk_fill_normal(void* out, int dtype, long long n, unsigned long long key, float mean,
                   float std, hipStream_t stream);

// mk_attention_generic with keys of width d and values of width dv (the value cache is
// [pages, n_kv, dv, page_size]); the output rows hold n_q heads of dv.  sinks (float32 [n_q],
// or null): exp(sink[head]) is added once to the softmax's denominator, unscaled, with no key
// or value behind it.  keep_first (with a window): the sequence's first keep_first keys stay
// visible to queries whose window has passed them.
int mk_attention_generic_kv(const void* q, int q_stride, void* out, int out_stride,
                            const void* k_cache, const void* v_cache, int dtype,
                            const int* positions, const int* token_seq, const int* block_table,
                            int table_stride, int page_size, int n_q, int n_kv, int d, int dv,
                            float scale, int window, int keep_first, float score_cap,
                            const float* distance_slopes, const float* sinks, int tokens,
                            hipStream_t stream);

// `batch` independent products y_b = x_b W_b^T in one launch: x_b = x + b * x_batch (rows lda
// apart), W_b = w + b * w_batch ([N, K]), y_b = out + b * o_batch (rows ldo apart); offsets in
// elements.  A matrix of its own per head over the head's own columns of x.
int mk_linear_batched_generic(const void* x, const void* w, int dtype, void* out, int out_dtype,
                              int M, int N, int K, int lda, int ldo, int batch, long long x_batch,
                              long long w_batch, long long o_batch, hipStream_t stream);

// Attention through a shared latent, the per-token side.  down [T, down_stride] (float32)
// holds a token's [query latent (q_rank) | key/value latent (kv_rank) | rotated key part
// (rot)].  The query latent is RMS-normed (q_norm_w) into q_latent [T, q_rank]; the key/value
// latent is RMS-normed (kv_norm_w) and, with the rotated part turned by the token's position
// (the first rot_dims dims of it, pairs (2i, 2i + 1) when interleaved, else (i, i + rot_dims /
// 2); angle tables [positions, rot_dims / 2]), written to the paged cache as one key row
// [kv_rank + rot] of one shared head, the normed latent once more as that head's value,
// transposed within the page ([pages, value_width, page_size]).  Key rows are key_width >=
// kv_rank + rot wide, the value has value_width >= kv_rank rows; what lies beyond is written
// as zeros.  q_rank = 0: no query latent.
int mk_latent_prepare(const float* down, int down_stride, int q_rank, int kv_rank, int rot,
                      const void* q_norm_w, const void* kv_norm_w, int norm_dtype, float eps,
                      const float* cos_table, const float* sin_table, int table_positions,
                      int rot_dims, int interleaved, const int* positions, const int* token_seq,
                      const int* block_table, int table_stride, void* q_latent, void* k_cache,
                      void* v_cache, int key_width, int value_width, int dtype, int page_size,
                      int write_kv, int tokens, hipStream_t stream);

// q [T, heads, dim + rot] -> out[t, head, out_offset .. out_offset + rot) of rows
// [heads, out_width]: every head's rotated part, turned by the token's position, and zeros
// behind it up to out_width.
int mk_latent_query_tail(const void* q, int dtype, int heads, int dim, int rot,
                         const float* cos_table, const float* sin_table, int table_positions,
                         int rot_dims, int interleaved, const int* positions, void* out,
                         int out_width, int out_offset, int tokens, hipStream_t stream);

// Routing: scores = softmax(logits [T, experts], float32); ids / weights [T, top]: the `top`
// largest scores' experts (ties: the lower index) and score * scale, the scores divided by
// the chosen ones' sum first when `renormalize`.
int mk_route_topk(const float* logits, int experts, int top, float scale, int renormalize,
                  int* ids, float* weights, int tokens, hipStream_t stream);

// Experts token by token: act [T * top, ff] = gate_act(Wg[e] x_t, Wu[e] x_t) for
// w [experts, 2 ff, K] = [gate | up]; then y [T, N] (float32) += sum_j weights[t, j] *
// Wd[e_j] act[(t, j)] for w [experts, N, ff], j ascending.
int mk_expert_gated(const void* x, const void* w, int dtype, const int* ids, void* act,
                    int tokens, int top, int ff, int K, int kind, float limit, float alpha,
                    float beta, hipStream_t stream);
int mk_expert_down(const void* act, const void* w, int dtype, const int* ids, const float* weights,
                   float* y, int tokens, int top, int ff, int N, hipStream_t stream);

// act[t, :] *= sigmoid(x[t, :] . w) in place: a feed-forward's activations (`dtype`, [T, inter])
// scaled by a gate of one number per token, the dot product and the sigmoid in float32.
int mk_row_gate(void* act, const void* x, const void* w, int dtype, int tokens, int inter,
                int hidden, hipStream_t stream);

// out[t, i] = gate_act(gate_up[t, i], gate_up[t, I + i]) for an activation MK_ACT_*.
int mk_gate_act(const void* gate_up, void* out, int dtype, int tokens, int inter, int kind,
                float limit, float alpha, float beta, hipStream_t stream);

// h[i] += mult * (y[i] + sum_k a[k * stride + i] + sum_k b[k * stride + i]) for i < n; y may
// be null.  mk_fill_zero: p[i] = 0 by a kernel (a captured graph records no memset node).
// Pairs (token, choice) grouped by expert: rows [pairs] lists the pair indices expert by
// expert (in no particular order within an expert), offsets [experts + 1] where each expert's
// group starts.  One workgroup.  mk_expert_combine: y[t, :] += sum_j pairs_out[t * top + j, :],
// j ascending.
int mk_route_group(const int* ids, int pairs, int experts, int* rows, int* offsets,
                   hipStream_t stream);
int mk_expert_combine(const float* pairs_out, float* y, int tokens, int top, int N,
                      hipStream_t stream);

int mk_scaled_add(float* h, const float* y, const float* a, int na, const float* b, int nb,
                  long long stride, float mult, long long n, hipStream_t stream);
int mk_fill_zero(float* p, long long n, hipStream_t stream);

// Queries and keys between their projection and the cache, from a float32 row
// [q: n_q d | k: n_kv d | v: n_kv dv] per token (the last part absent when `values_are_keys`:
// the values are then the keys as projected, before anything below).  In this order: RMS norms
// over the whole q part and the whole k part with weights q_norm [n_q d] and k_norm [n_kv d]
// (both null: none); q times 1 + temp_coef * ln(floor((p + 1) / temp_every) + 1) at position p
// (temp_every 0: none); the first `rot` dims of every head turned as in mk_rope_kv_write.
// q goes to q_out [T, n_q d] of `dtype`, k and v into the paged cache (values [pages, n_kv, dv,
// page_size]) when write_kv.
// maps > 1: a head of d dims is `maps` score maps of d / maps dims side by side, each turned in
// its own first `rot` dims; q_out is then [T, n_q maps, d], query (head, map) holding its
// map's dims in their place and zeros elsewhere, so that its product with a whole key row is
// the map's score.
// head_norm != 0: the norms run over every head by itself, q_norm and k_norm being weights of d
// entries shared by the heads.  v_mode (MK_VMIX_*): the values before they are cached are left
// in v_carry [T, n_kv dv] (float32), or blended with what lies there,
// (1 - v_lambda) v + v_lambda v_carry.
int mk_qk_prepare(const float* qkv, int row_stride, void* q_out, int dtype, const void* q_norm,
                  const void* k_norm, int norm_dtype, float eps, float temp_coef, int temp_every,
                  const float* cos_table, const float* sin_table, int table_positions, int rot,
                  int interleaved, const int* positions, const int* token_seq,
                  const int* block_table, int table_stride, void* k_cache, void* v_cache,
                  int page_size, int n_q, int n_kv, int d, int dv, int values_are_keys,
                  int write_kv, int maps, int head_norm, float* v_carry, int v_mode,
                  float v_lambda, int tokens, hipStream_t stream);

// out[t, i] = a[t, i] * sigmoid(gate[t * gate_stride + i]), i < width; a and out of `dtype`
// (they may be the same), the gate float32 columns of a projection.
int mk_gate_mul(const void* a, int dtype, const float* gate, int gate_stride, void* out,
                int tokens, int width, hipStream_t stream);

// The residual stream as a sublayer reads it: h[i] += its `count` partial sums
// partials[k * stride + i], and out[i] = h[i] in `dtype`, i < n.
int mk_stream_cast(float* h, const float* partials, int count, long long stride, void* out,
                   int dtype, long long n, hipStream_t stream);

// out[i] = act(x[i]) for an activation MK_UNARY_*; x of in_dtype (float32, or the output's),
// the result rounded once to `dtype`.
int mk_unary_act(const void* x, int in_dtype, void* out, int dtype, long long n, int kind,
                 hipStream_t stream);

// h[t, :] += mult * (rmsnorm(a[t, :]) * wa + rmsnorm(b[t, :]) * wb), with a = ya + its `na`
// partial sums pa[k * stride + .] (ya may be null) and b likewise (no b at all: yb null and
// nb 0); plain weights, eps inside the root.
int mk_normed_sum(float* h, const float* ya, const float* pa, int na, const void* wa,
                  const float* yb, const float* pb, int nb, const void* wb, int weight_dtype,
                  float eps, float mult, long long stride, int tokens, int hidden,
                  hipStream_t stream);

// h[t, :] += scale .* (rmsnorm(y[t, :] + its `count` partial sums p[k * stride + .]) * weight):
// a sublayer's output normed before it enters the stream, times a stored vector per channel
// (`scale`, float32 or null).  x_out (or null): the new h once more, in x_dtype, for a sublayer
// that reads the stream itself.
int mk_norm_scale_add(float* h, const float* y, const float* partials, int count,
                      long long stride, const void* weight, int weight_dtype, const float* scale,
                      float eps, int tokens, int hidden, void* x_out, int x_dtype,
                      hipStream_t stream);

// Differential attention's tail.  a [T, heads, 2, dv] (`dtype`) holds two maps' outputs per
// head; o = a1 - lambda * a2 is divided by its root mean square over dv (eps inside the root),
// multiplied by out_scale and, when gate is not null, by sigmoid(gate[t * gate_stride + head])
// (float32); out [T, heads dv] of `dtype`.
int mk_diff_heads(const void* a, void* out, int dtype, const float* gate, int gate_stride,
                  float lambda, float eps, float out_scale, int tokens, int heads, int dv,
                  hipStream_t stream);

// out[t, :] = [a[t, :] | b[t, :]] in `dtype`; mk_copy_f32: dst[i] = src[i] by a kernel.
int mk_concat_cast(const float* a, const float* b, void* out, int dtype, int tokens, int hidden,
                   hipStream_t stream);
int mk_copy_f32(float* dst, const float* src, long long n, hipStream_t stream);

// A state-space mixer's pieces.  Per-request state lies in rows of `slot_stride` floats, a
// sequence's row being slots[seq]; cu_q [S + 1] are the prefix sums of the step's tokens.
// mk_causal_conv_silu: out[t, c] = silu(bias[c] + sum_j w[c, j] u_(t - taps + 1 + j)[c]) for the
// `channels` columns of proj from col0 on, inputs before the step's first token coming from
// `carried` ([taps - 1, channels] per slot, oldest first), which then takes the sequence's last
// taps - 1 inputs.
int mk_causal_conv_silu(const float* proj, int row_stride, int col0, int channels, int taps,
                        const void* w, const void* bias, int weight_dtype, float* carried,
                        long long slot_stride, const int* slots, const int* token_seq,
                        const int* cu_q, float* out, int tokens, int num_seqs, hipStream_t stream);
// mk_ssm_scan: per head S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T, S being N x P,
// y_t = (S_t^T C_t + D x_t) * silu(z_t), dt_t = softplus(raw_t + dt_bias); rows of xbc are
// [x: heads P | B: groups N | C: groups N], z and raw dt are columns z_col and dt_col of proj;
// y_out [T, heads P].  The state is read from and written to the sequence's slot, laid out
// as the kernel's lanes hold it: mk_ssm_state_floats says how many floats that takes (-1: sizes
// it does not run).
int mk_ssm_scan(const float* xbc, int xbc_stride, const float* proj, int proj_stride, int z_col,
                int dt_col, const void* dt_bias, const void* a_log, const void* d_skip,
                int weight_dtype, float* state, long long slot_stride, const int* slots,
                const int* cu_q, int heads, int P, int N, int groups, float* y_out, int tokens,
                int num_seqs, int total_chunks, float* workspace, hipStream_t stream);
// A step with a sequence of more than mk_ssm_chunk_tokens() tokens runs the recurrence in
// chunks side by side: total_chunks is then the sum over the sequences of ceil(tokens /
// chunk), `workspace` mk_ssm_scan_workspace(...) floats of scratch memory; else 0 and null.
int mk_ssm_chunk_tokens();
long long mk_ssm_scan_workspace(int total_chunks, int heads, int P, int N);
long long mk_ssm_state_floats(int heads, int P, int N);
// Retention: per head S_t = decay S_(t-1) + k_t v_t^T (S is dim x vdim, float32), o_t = S_t^T q_t.
// q, k, v are columns q_col, k_col, v_col of the float32 rows of proj ([heads dim], [heads dim],
// [heads vdim]); the first `rot` dims of every q and k head turn by the tabulated angles of the
// token's position (dim j with j + rot / 2), and k is multiplied by k_scale after the turn.
// The state of a sequence is its slot's row of `state` ([heads, dim, vdim], rows slot_stride
// floats apart), read at the step's start and left for the next; out [T, heads vdim] float32.
// total_chunks > 0: every sequence runs as ceil(tokens / mk_retention_chunk_tokens()) chunks
// side by side (total_chunks of them in the step) over a workspace of
// mk_retention_scan_workspace(...) floats; 0: token by token from the slot's state.
int mk_retention_chunk_tokens(void);
long long mk_retention_scan_workspace(int total_chunks, int heads, int dim, int vdim);
int mk_retention_scan(const float* proj, int proj_stride, int q_col, int k_col, int v_col,
                      const float* decay, float k_scale, const float* cos_table,
                      const float* sin_table, int table_positions, int rot, const int* positions,
                      const int* cu_q, const int* slots, float* state, long long slot_stride,
                      int heads, int dim, int vdim, float* out, int tokens, int num_seqs,
                      int total_chunks, float* workspace, hipStream_t stream);
// out[t, head, :] = y[t, head, :] / rms(y[t, head, :]) * weight[head dv + .] *
// gate(gate[t * gate_stride + head dv + .]): a norm per head (weight float32 [heads dv], or null
// for none), then a gate MK_GATE_* (float32 columns of a projection).
int mk_head_norm_gate(const float* y, void* out, int dtype, const float* gate, int gate_stride,
                      float eps, int tokens, int heads, int dv, const float* weight,
                      int gate_kind, hipStream_t stream);

// A matrix memory with input and forget gates and a running maximum (the mLSTM cell), per head:
//   m_t = max(f_t + m_(t-1), i_t),  S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T,
//   n_t likewise with k_t alone,  o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6),
// S, n and m zero before the sequence.  q (times q_scale), k, v and the raw gates a_t, b_t are
// columns of the float32 rows of proj ([heads dim] at q_col and k_col, [heads vdim] at v_col,
// [heads] at i_col and f_col); i_t = cap tanh(a_t / cap), f_t = logsigmoid(cap tanh(b_t / cap))
// (gate_cap <= 0: no bound).  A sequence's state is its slot's row of `state`
// (mk_mlstm_state_floats(...) floats, rows slot_stride apart), read at the step's start and left
// for the next; out [T, heads vdim] float32.
// total_chunks > 0: every sequence runs as ceil(tokens / mk_mlstm_chunk_tokens()) chunks side by
// side (total_chunks of them in the step) over a workspace of mk_mlstm_scan_workspace(...)
// floats; 0: token by token from the slot's state.
long long mk_mlstm_state_floats(int heads, int dim, int vdim);
int mk_mlstm_chunk_tokens(void);
long long mk_mlstm_scan_workspace(int total_chunks, int tokens, int heads, int dim, int vdim);
int mk_mlstm_scan(const float* proj, int proj_stride, int q_col, int k_col, int v_col, int i_col,
                  int f_col, float q_scale, float gate_cap, const int* cu_q, const int* slots,
                  float* state, long long slot_stride, int heads, int dim, int vdim, float* out,
                  int tokens, int num_seqs, int total_chunks, float* workspace,
                  hipStream_t stream);
// out[t, part] = y[t, part] / rms(y[t, part]) * weight[part], the row in `parts` equal parts.
int mk_group_rmsnorm(const float* y, void* out, int dtype, const void* weight, int weight_dtype,
                     float eps, int tokens, int width, int parts, hipStream_t stream);

// @library mfma: bfloat16 kernels on the matrix cores

// y = x W^T for 1 <= M <= 16 rows of x, K split into `slices` (ask mk_linear_skinny_slices
// for a good count): out is float32 [slices, M, N], to be summed over the slices.
int mk_linear_skinny_slices(int M, int N, int K);
int mk_linear_skinny(const void* x, const void* w, float* out, int M, int N, int K, int slices,
                     hipStream_t stream);

// out[M, N] (float32) += x W^T (+ bias) for 1 <= M <= 16, all of K in each workgroup;
// mk_linear_skinny_unsplit says whether that is the faster form for the shape.
int mk_linear_skinny_unsplit(int M, int N, int K);
int mk_linear_skinny_acc(const void* x, const void* w, const void* bias, int bias_dtype,
                         float* out, int M, int N, int K, hipStream_t stream);

// h64[M, N] (the fixed-point residual stream, see mk_embed_fixed) += x W^T (+ bias) for
// 1 <= M <= 16, K in `slices` slices as mk_linear_skinny takes them.
int mk_linear_skinny_fixed(const void* x, const void* w, const void* bias, int bias_dtype,
                           long long* h64, int M, int N, int K, int slices, hipStream_t stream);

// act[M, inter] (bfloat16) = silu(x Wg^T) * (x Wu^T) for w = [Wg | Wu] stacked [2 inter, K],
// 1 <= M <= 16.
int mk_gated_skinny(const void* x, const void* w, void* act, int M, int inter, int K,
                    hipStream_t stream);
// The same with the gate activation MK_ACT_* `kind` (limit, alpha, beta: its constants).
int mk_gated_skinny_act(const void* x, const void* w, void* act, int M, int inter, int K, int kind,
                        float limit, float alpha, float beta, hipStream_t stream);

// The gated and the q/k/v projection of at most 16 rows on x = rmsnorm(h64) * norm_w, which
// every workgroup makes for itself from the fixed-point residual stream h64 [M, K] (the norm
// needs no kernel of its own); K at most mk_skinny_normed_max_k(M).
int mk_skinny_normed_max_k(int M);
int mk_gated_skinny_normed(const long long* h64, const void* norm_w, int norm_dtype, float eps,
                           const void* w, void* act, int M, int inter, int K, hipStream_t stream);
int mk_qkv_skinny_normed(const long long* h64, const void* norm_w, int norm_dtype, float eps,
                         const void* w, const void* bias, int bias_dtype, void* q_out,
                         const float* cos_table, const float* sin_table, int table_positions,
                         const int* positions, const int* token_seq, const int* block_table,
                         int table_stride, void* k_cache, void* v_cache, int page_size, int n_q,
                         int n_kv, int d, int rotate, int M, int K, hipStream_t stream);

// The q/k/v projection of 1 <= M <= 64 tokens, w = [(n_q + 2 n_kv) d, K], with bias, rotation
// of q and k over the whole head (rotate != 0), q [M, n_q d] out and k, v written to the
// paged cache; n_kv = 0 projects the queries only.  d must be a multiple of 32.
int mk_qkv_skinny(const void* x, const void* w, const void* bias, int bias_dtype, void* q_out,
                  const float* cos_table, const float* sin_table, int table_positions,
                  const int* positions, const int* token_seq, const int* block_table,
                  int table_stride, void* k_cache, void* v_cache, int page_size, int n_q,
                  int n_kv, int d, int rotate, int M, int K, hipStream_t stream);

// The q/k/v projection as mk_qkv_skinny, for any M, tiled through LDS; config: a tile
// configuration, -1 for the one estimated fastest.
int mk_qkv_tiled(const void* x, const void* w, const void* bias, int bias_dtype, void* q_out,
                 const float* cos_table, const float* sin_table, int table_positions,
                 const int* positions, const int* token_seq, const int* block_table,
                 int table_stride, void* k_cache, void* v_cache, int page_size, int n_q,
                 int n_kv, int d, int rotate, int M, int K, int config, hipStream_t stream);

// The gated projection for any M, tiled through LDS; config: a tile configuration, -1 for the
// one estimated fastest.
int mk_gated_tiled_config(int M, int inter, int K);
int mk_gated_tiled(const void* x, const void* w, void* act, int M, int inter, int K, int config,
                   hipStream_t stream);
int mk_gated_tiled_act(const void* x, const void* w, void* act, int M, int inter, int K, int config,
                       int kind, float limit, float alpha, float beta, hipStream_t stream);

// Many small products in one launch: y_b = x_b W_b^T for b < batch, x_b = x + b * x_batch (rows
// lda apart), W_b = w + b * w_batch ([N, K]), y_b = out + b * o_batch (rows ldo apart), offsets
// in elements, everything bfloat16; K, lda and the offsets multiples of 8.
int mk_linear_batched_mfma(const void* x, const void* w, void* out, int M, int N, int K, int lda,
                           int ldo, int batch, long long x_batch, long long w_batch,
                           long long o_batch, hipStream_t stream);

// Experts over the tokens routed to them.  rows [T * top] lists the (token, choice) pairs
// grouped by expert, offsets [experts + 1] where each expert's group starts, max_rows bounds a
// group's size.  gated: act[pair, :] (bfloat16 [T * top, ff]) = activation(Wg[e] x[pair / top],
// Wu[e] x[pair / top]) for w [experts, 2 ff, K].  down: y[pair, :] (float32 [T * top, N]) =
// weights[pair] * Wd[e] act[pair, :] for w [experts, N, ff].
int mk_expert_gated_mfma(const void* x, const void* w, void* act, const int* rows,
                         const int* offsets, int experts, int max_rows, int top, int ff, int K,
                         int kind, float limit, float alpha, float beta, hipStream_t stream);
int mk_expert_down_mfma(const void* act, const void* w, float* y, const int* rows,
                        const int* offsets, const float* weights, int experts, int max_rows, int ff,
                        int N, hipStream_t stream);

// Attention of `heads` query heads over one shared key/value head with keys of dk (a multiple
// of 32) and values of dv dims (a multiple of 16): q [T, heads, dk], out [T, heads, dv], keys
// [pages, page, dk], values transposed within the page [pages, dv, page].  Tiles of 16 rows,
// row f of a sequence = token f / heads, head f % heads (tile_seq / tile_row0 as for
// mk_attention_mfma with one group of `heads`).  num_parts > 1 splits every tile's keys into
// that many parts (at most mk_attention_latent_max_parts()) whose results part_o
// [tiles, parts, dv, 16] / part_ml [tiles, parts, 2, 16] a second kernel merges.  tile_rows 64
// (keys unsplit): tiles of 64 rows, one a workgroup, whose wavefronts share every block of
// keys through LDS: for prompt portions.  window > 0: a row at position p sees the keys
// (p - window, p] only.  sinks (float32 [heads], or null): exp(sink[head]) stands once more in
// the denominator of the head's rows, unscaled.
// Key and value widths come from a list of compiled shapes: mk_attention_latent_widths gives
// the widths a cache must have for keys of at least dk and values of at least dv dims (host
// pointers; returns 0 when no shape holds them), padded with zeros.
int mk_attention_latent_widths(int dk, int dv, int* key_width, int* value_width);
int mk_attention_latent_supported(int dk, int dv, int page_size);
int mk_attention_latent_max_parts(void);
int mk_attention_latent(const void* q, void* out, const void* k_cache, const void* v_cache,
                        const int* tile_seq, const int* tile_row0, int num_tiles, int tile_rows,
                        const int* cu_q,
                        const int* kv_len, const int* block_table, int table_stride, int page_size,
                        int heads, int dk, int dv, float scale, int num_parts, float* part_o,
                        float* part_ml, int window, const float* sinks, hipStream_t stream);

// y = x W^T (+ bias) for any M, tiled through LDS; output bfloat16 or float32, or float32
// accumulated into `out`.  config: a tile configuration, 0 .. mk_linear_tiled_configs() - 1
// (mk_linear_tiled_config picks the one estimated fastest for the shape and the bytes the
// epilogue moves per element of y; -1 does the same).
// mk_linear_tiled_partials: the same product as float32 partial sums out[slices, M, N] over
// slices of K, for few rows of x over a long K (mk_linear_tiled_slices: how many slices pay;
// any count that the 64-wide stages of K divide into is taken).
int mk_linear_tiled_slices(int M, int N, int K);
int mk_linear_tiled_partials(const void* x, const void* w, float* out, int M, int N, int K,
                             int slices, hipStream_t stream);
int mk_linear_tiled_configs(void);
int mk_linear_tiled_config(int M, int N, int K, int out_bytes);
int mk_linear_tiled(const void* x, const void* w, const void* bias, int bias_dtype, void* out,
                    int out_dtype, int accumulate, int M, int N, int K, int ldo, int config,
                    hipStream_t stream);

// Whether mk_attention_mfma takes this head size and page size.
int mk_attention_mfma_supported(int head_dim, int page_size);

// The most rows per tile (16, 32 or 64) mk_attention_mfma takes for this head size.
int mk_attention_mfma_max_rows(int head_dim);

// The same attention on the matrix cores.  The caller cuts the step into tiles of
// rows_per_tile rows (row f of a sequence = token f / G, head kvh * G + f % G):
// tile_seq / tile_row0 name each tile's sequence and first row.  cu_q [S+1] are the prefix sums of the sequences' token
// counts, kv_len [S] their lengths once this step's tokens are written.  With num_splits > 1
// the keys are split, split_blocks blocks of 32 keys per split (0: each tile's own range in
// num_splits equal parts), and part_o [tiles, n_kv, splits, rows_per_tile, d] /
// part_ml [.., rows_per_tile, 2] hold the partial results.  staged != 0: the tiles are of
// 4 * rows_per_tile rows, one per workgroup, whose wavefronts share the keys and values
// through LDS, `staged` (1, 2 or 4, at most what mk_attention_mfma_staged returns) groups of
// four wavefronts taking the key blocks in turn; for many rows per sequence, keys unsplit.
// staged = 8: the prompt kernel built on 32 x 32 x 16 products (wavefronts of 32 rows, blocks
// of 64 keys; tiles of 128 rows, rows_per_tile = 32), where mk_attention_mfma_wide says so.
// tile_seq = tile_row0 = null: no tile list, tile t is the one new token of sequence t
// (decoding; tiles of 16 rows, at most 16 heads a group, no window, split_blocks 0): part s of
// num_splits is then the blocks s, s + num_splits, ... of the keys, and the kernel asks for
// nothing before the block table.
// mk_attention_mfma_check: what mk_attention_mfma checks of its arguments before it launches,
// without the launch (0: it would take them; else mk_last_error() says why not).
int mk_attention_mfma_staged(int head_dim, int rows_per_tile);
int mk_attention_mfma_wide(int head_dim);
// The same kernel on tiles of 64 rows (two wavefronts a key group; staged = 8 * chains + 4):
// which numbers of chains exist at this head size (bit n - 1).
int mk_attention_mfma_wide_half(int head_dim);
// Which of these instantiations, as its `staged` code, measured fastest for a step of `wg128`
// workgroups of 128 rows or `wg64` of 64 (key/value heads counted) whose longest sequence is
// `blocks32` blocks of 32 keys, most of them this step's own or not (`fresh`); 0: none, the
// 16-row kernels are faster.
int mk_attention_mfma_wide_choice(int head_dim, int wg128, int wg64, int blocks32, int fresh);
int mk_attention_mfma_check(int q_stride, int out_stride, int num_tiles, int page_size, int n_q,
                            int n_kv, int d, float scale, int window, int rows_per_tile,
                            int staged, int num_splits, int split_blocks, int has_workspace);
int mk_attention_mfma(const void* q, int q_stride, void* out, int out_stride,
                      const void* k_cache, const void* v_cache, const int* tile_seq,
                      const int* tile_row0, int num_tiles, const int* cu_q, const int* kv_len,
                      const int* block_table, int table_stride, int page_size, int n_q, int n_kv,
                      int d, float scale, int window, int rows_per_tile, int staged,
                      int num_splits, int split_blocks, float* part_o, float* part_ml,
                      hipStream_t stream);

// out [M, N] (bfloat16) = act(x W^T) for an activation of one operand MK_UNARY_*, applied to the
// float32 sums in the tiled kernel's epilogue.  config -1: by the sizes.
int mk_linear_tiled_act(const void* x, const void* w, void* out, int M, int N, int K, int act,
                        int config, hipStream_t stream);

// mk_attention_mfma in tiles of 16 rows with a say in the score: score_cap > 0 bounds the
// scaled score to cap * tanh(score / cap); sinks (float32 [n_q], or null) adds exp(sink[head])
// once to the softmax's denominator.  tile_seq / tile_row0 null: every sequence brings one
// token (see mk_attention_mfma).  staged: 0, or 1, 2, 4 key groups of workgroups of four
// wavefronts that share a sequence's keys through LDS (the tile list then in steps of 64 rows).
int mk_attention_mfma_scored(const void* q, int q_stride, void* out, int out_stride,
                             const void* k_cache, const void* v_cache, const int* tile_seq,
                             const int* tile_row0, int num_tiles, const int* cu_q,
                             const int* kv_len, const int* block_table, int table_stride,
                             int page_size, int n_q, int n_kv, int d, float scale, int window,
                             int staged, int num_splits, int split_blocks, float score_cap,
                             const float* sinks, float* part_o, float* part_ml,
                             hipStream_t stream);
// The same, leaving the parts of split keys unmerged (see mk_attention_mfma_parts).
int mk_attention_mfma_parts_scored(const void* q, int q_stride, const void* k_cache,
                                   const void* v_cache, const int* tile_seq, const int* tile_row0,
                                   int num_tiles, const int* cu_q, const int* kv_len,
                                   const int* block_table, int table_stride, int page_size,
                                   int n_q, int n_kv, int d, float scale, int window,
                                   int num_splits, int split_blocks, float score_cap,
                                   const float* sinks, float* part_o, float* part_ml,
                                   hipStream_t stream);

// Decoding with split keys, in two kernels instead of three.  mk_attention_mfma_parts is
// mk_attention_mfma without the merge of the key splits: the partial results stay in part_o /
// part_ml, mk_attention_mfma_parts_written(...) of them per (tile, kv head) (a workgroup's four
// wavefronts may have added four parts up already).  mk_attention_out then merges them and
// multiplies by the output matrix w_o [N, n_q d] in one kernel, for steps of one token per
// sequence (tile = token, M of them): out[slice, M, N] are float32 partial sums over slices of
// heads_per_slice query heads each (mk_attention_out_heads_per_slice: how many, for slices
// stored or, with `atomic`, added into the fixed-point stream; 0 where the sizes are not taken; mk_attention_out_max_parts: the most partial results per (tile, kv head)
// it takes), to be added up by whoever consumes the projection; or, with `out` null, the
// result is added into the fixed-point residual stream fixed_out [M, N] (see mk_embed_fixed).
// wide: 128 rows of w_o per workgroup instead of 64.
int mk_attention_mfma_parts_written(int rows_per_tile, int num_splits, int d);
int mk_attention_mfma_parts(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                            const int* tile_seq, const int* tile_row0, int num_tiles,
                            const int* cu_q, const int* kv_len, const int* block_table,
                            int table_stride, int page_size, int n_q, int n_kv, int d, float scale,
                            int window, int rows_per_tile, int num_splits, int split_blocks,
                            float* part_o, float* part_ml, hipStream_t stream);
int mk_attention_out_heads_per_slice(int n_q, int n_kv, int d, int M, int N, int atomic);
int mk_attention_out_max_parts(int M, int heads_per_slice);
int mk_attention_out(const float* part_o, const float* part_ml, int parts, const void* w_o,
                     float* out, long long* fixed_out, int M, int N, int n_q, int n_kv, int d,
                     int heads_per_slice, int wide, hipStream_t stream);

// Two-map (differential) attention with its tail, bfloat16 on the matrix cores: a head's key
// row holds two score maps of map_dim dims side by side, query (head, map) lies a key row wide
// in q [T, q_stride] at (head * 2 + map) * 2 map_dim with its own map's dims filled; both maps
// are softmax attentions over the same values (dv wide) inside `window` (0: every earlier key)
// beside the sequence's first `keep_first` keys; out [T, heads, dv] =
// (a1 - lambda a2) / rms * out_scale * sigmoid(gate[t * gate_stride + head]) (gate float32 or
// null).  positions [T] and cu_q [S + 1] describe the step; its longest sequence brings
// max_q_len tokens.  mk_attention_maps_supported: whether the sizes are compiled.
// splits > 1 (a step in which every sequence brings one token): that many workgroups share a
// (sequence, head)'s key blocks and leave parts in `parts` (mk_attention_maps_parts floats),
// which a second kernel merges in their order.
int mk_attention_maps_supported(int map_dim, int dv, int page_size);
long long mk_attention_maps_parts(int num_seqs, int heads, int dv, int splits);
int mk_attention_maps(const void* q, int q_stride, void* out, const void* k_cache,
                      const void* v_cache, const float* gate, int gate_stride,
                      const int* positions, const int* cu_q, const int* block_table,
                      int table_stride, int page_size, int heads, int kv_heads, int map_dim,
                      int dv, float scale, int window, int keep_first, float lambda, float eps,
                      float out_scale, int num_seqs, int max_q_len, int splits, float* parts,
                      hipStream_t stream);

// @library core

// parts: optional scratch of rows * 64 * 8 bytes; with it, few rows of a large vocabulary
// are searched by 64 workgroups per row.
int mk_argmax(const float* logits, int rows, int vocab, long long row_stride, int* out,
              void* parts, hipStream_t stream);

// mk_argmax without a buffer of the caller's, and without any allocation: the partial results
// live in a device array inside the library (one per GPU, kept until the process ends), of
// mk_argmax_static_max_rows() rows; more rows are refused.  This entry point has no
// counterpart in the reference: it is for callers that cannot allocate (code under HIP graph
// capture, serving loops and harnesses that forbid hipMalloc).  Calls that overlap on one GPU
// share the array and race; calls on one stream, one after the other, are safe.  The first
// call on a device asks the runtime where the array lies; mk_argmax_static_init() does only
// that, for the current device, so that a caller can have it done before a stream capture
// begins.  Both may be called from several threads.
int mk_argmax_static_max_rows(void);
int mk_argmax_static_init(void);
int mk_argmax_static(const float* logits, int rows, int vocab, long long row_stride, int* out,
                     hipStream_t stream);

// One token per row: the argmax where temperature <= 0, else an inverse-CDF draw with the
// row's uniform number from softmax(logits / temperature) restricted to the nucleus top_p
// (top_ps null: no row restricts it, and the threshold search is skipped).  scratch:
// mk_sample_scratch_bytes(rows, top_ps != null) bytes, 256-byte aligned.
long long mk_sample_scratch_bytes(int rows, int nucleus);
int mk_sample(const float* logits, int rows, int vocab, long long row_stride,
              const float* temperatures, const float* top_ps, const float* uniforms,
              void* scratch, int* out, hipStream_t stream);

#ifdef __cplusplus
}
#endif
