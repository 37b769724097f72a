// The launch sequences of the built-in operations: which kernels run a projection, a q/k/v
// projection, an attention or a gated projection of given sizes, and with which arguments.
// There is one copy of each: the program's operations (builtin.cc) and the Python faces of the
// kernels (bindings.cc, what the kernel tests and parts from outside call) both come here.
//
// Every function takes the operation context of op_abi.h for its stream, its compute dtype
// and its temporaries; with the context `dry` it allocates and launches nothing.
#pragma once

#include <hip/hip_runtime_api.h>

#include "../host/op_abi.h"
#include "dispatch.h"

namespace mercury {

struct Launch {
  mk_op_context* ctx;
  explicit Launch(mk_op_context* c) : ctx(c) {}
  bool dry() const { return ctx->dry != 0; }
  hipStream_t stream() const { return (hipStream_t)ctx->stream; }
  int dtype() const { return ctx->dtype; }
  int elem() const { return element_size(ctx->dtype); }
  void* alloc(size_t bytes) const { return ctx->alloc(ctx->arena, bytes); }
};

// out[t, :] = table[ids[t], :] * scale as float32.
void embed(Launch& l, const int* ids, const void* table, int table_dtype, float* out, int tokens,
           int hidden, int vocab, float scale);

// RMSNorm of rows of h (all, or those `rows` lists) into `out` (allocated when null), after
// adding `pending_count` partial sums [p, tokens, hidden] into h.
void* rmsnorm(Launch& l, float* h, int tokens, int hidden, const float* pending, int pending_count,
              const void* weight, int weight_dtype, float eps, const int* rows, int out_rows,
              void* out = nullptr, bool round_once = false);

// The residual stream of a step of few tokens in fixed point (op_abi.h): its start, the norm
// of rows of it, and a norm left for the projection behind it to fold in.
void embed_fixed(Launch& l, const int* ids, const void* table, int table_dtype, long long* out,
                 int tokens, int hidden, int vocab, float scale);
void* rmsnorm_fixed(Launch& l, const long long* h64, int hidden, const void* weight,
                    int weight_dtype, float eps, const int* rows, int out_rows);
struct NormFold {
  const long long* h64 = nullptr;
  const void* weight = nullptr;
  int weight_dtype = 0;
  float eps = 0.f;
};
// h64 += x W^T (+ bias).
void project_into_fixed(Launch& l, const void* x, int m, const void* w, int n, int k,
                        const void* bias, int bias_dtype, long long* h64);

void* silu_mul(Launch& l, const void* gate_up, int tokens, int inter, void* out = nullptr);

// The activation of a gated feed-forward with its constants (MK_ACT_* of mercury_kernels.h):
// silu(g) * u, or g' * sigmoid(alpha g') * (u' + beta) on g' = min(g, limit) and
// u' = clamp(u, -limit, limit).
struct GateAct {
  int kind = 0;
  float limit = 0.f, alpha = 1.f, beta = 0.f;
  bool silu() const { return kind == 0; }
};
void* gate_activation(Launch& l, const void* gate_up, int tokens, int inter, const GateAct& act,
                      void* out = nullptr);

// h += mult * (y + the partial sums a [na, n] and b [nb, n]); y may be null.
void scaled_add(Launch& l, float* h, const float* y, const float* a, int na, const float* b, int nb,
                long long n, float mult);
float* zeros(Launch& l, long long n);

// logits <- cap * tanh(logits / cap), in place.
void logit_cap(Launch& l, float* logits, long long count, float cap);

// Overrides of the choices, for tests: kernel 0 auto, 1 the float32-arithmetic kernel, 2 the
// matrix-core kernels; tile_config -1 auto.
struct LinearForce {
  int kernel = 0;
  int tile_config = -1;
};

// y = x W^T (+ bias) into `out` (allocated when null) of out_dtype; with `accumulate`, added
// into the float32 `out`.
void* linear(Launch& l, const void* x, int m, const void* w, int n, int k, const void* bias,
             int bias_dtype, void* out, int out_dtype, bool accumulate, LinearForce force = {});

// Float32 partial sums [slices, m, n] of x W^T over slices of K.
float* linear_partials(Launch& l, const void* x, int m, const void* w, int n, int k, int& slices);

// h += x W^T (+ bias), or, where that streams the weights faster, partial sums left for the
// next norm to add (pending / pending_count; none when the product went into h).
void project_into_stream(Launch& l, const void* x, int m, const void* w, int n, int k,
                         const void* bias, int bias_dtype, float* h, const float*& pending,
                         int& pending_count);

// How a position encoding transforms q and k: rotation by tabulated angles over the first
// `rotary_dim` dims of a head, pairing dim j with j + rotary_dim/2 ("half") or 2j with 2j+1
// ("interleaved"); rotary_dim 0 is no transformation.
struct PositionDesc {
  int rotary_dim = 0;
  const float* cos = nullptr;
  const float* sin = nullptr;
  int table_positions = 0;
  int interleaved = 0;
};

// The per-token and per-sequence arrays the cache-touching kernels read.
struct StepArrays {
  const int *positions = nullptr, *token_seq = nullptr, *cu_q = nullptr, *kv_len = nullptr;
  const int* table = nullptr;    // the cache group's block table [S, table_stride]
  int table_stride = 0;
};

struct QkvArgs {
  const void *w = nullptr, *bias = nullptr;
  int bias_dtype = 0;
  int n_q = 0, n_kv = 0, head_dim = 0;
  PositionDesc pos;
  void *k_cache = nullptr, *v_cache = nullptr;
  int page_size = 1;
  bool writes = true;            // false: only the queries are projected (w holds n_q heads)
};

struct Queries {
  const void* q;
  int stride;
};

// kind: -1 by the sizes, else a QkvKind; tile_config for the tiled kernel.
struct QkvForce {
  int kind = -1;
  int tile_config = -1;
};

// q, k, v = x W^T + bias, q and k rotated, k and v written to the paged cache; the rotated
// queries come back (rows of `stride` elements).
// With `fold`, x is rmsnorm(fold->h64) * fold->weight and `x` is ignored: the projection makes
// it itself where its kernel can, else the norm runs first.
Queries qkv_project(Launch& l, const void* x, int m, int k, const QkvArgs& a, const StepArrays& s,
                    QkvForce force = {}, const NormFold* fold = nullptr);

// What some makes of attention do to q and k between projection and cache, beyond a rotation:
// RMS norms over the whole q and the whole k projection (weights q_norm [n_q d], k_norm
// [n_kv d]), a query temperature 1 + coef * ln(floor((p + 1) / every) + 1), values that are
// the keys as projected (no v rows in w), values of another width than the keys.
struct QkPrep {
  const void *q_norm = nullptr, *k_norm = nullptr;
  int norm_dtype = 0;
  float eps = 0.f;
  float temp_coef = 0.f;
  int temp_every = 0;
  int values_are_keys = 0;
  int value_dim = 0;            // 0: as wide as the keys
  // A head of `maps` score maps side by side (each turned by itself): the queries come back
  // as n_q * maps rows a key row wide, every one zero outside its own map.
  int maps = 1;
  // Further columns of the stacked projection behind q, k, v that belong to the caller (a
  // gate's logits): projected in the same product, left alone here.
  int extra_cols = 0;
  // The norms run over every head by itself, q_norm and k_norm being [head_dim] weights the
  // heads share.
  int head_norm = 0;
  // Values mixed across layers (MK_VMIX_*): this layer leaves its values of the step's tokens in
  // the step's carried buffer, or caches (1 - v_lambda) v + v_lambda * what lies there.
  int v_mode = 0;
  float v_lambda = 0.f;
  bool active() const {
    return q_norm != nullptr || temp_every > 0 || values_are_keys != 0 || value_dim > 0 ||
           maps > 1 || extra_cols > 0 || v_mode != 0;
  }
};
// qkv_project for such an attention: the projection in float32, then one kernel for all of
// the above, the rotation and the cache write.
// `raw`, when not null, receives the float32 projection and `raw_stride` its row width (the
// extra columns start behind q, k and v).
Queries qkv_prepared(Launch& l, const void* x, int m, int k, const QkvArgs& a, const QkPrep& prep,
                     const StepArrays& s, const float** raw = nullptr, int* raw_stride = nullptr);

// Rotation and cache write of an already projected qkv [m, row_stride] (q rotated in place).
void rope_kv_write(Launch& l, void* qkv, int row_stride, int m, const QkvArgs& a,
                   const StepArrays& s);

// The same for a projection that arrives as partial sums [slices, m, width]; the rotated q
// goes to a new [m, n_q d] tensor of out_dtype.
void* qkv_finish(Launch& l, const float* parts, int slices, int m, const QkvArgs& a,
                 const StepArrays& s, int out_dtype);

struct AttendArgs {
  int n_q = 0, n_kv = 0, head_dim = 0, page_size = 0, window = 0;
  int keep_first = 0;    // with a window: the sequence's first keys stay visible past it
  int value_dim = 0;     // 0: values as wide as keys
  int v_dim() const { return value_dim > 0 ? value_dim : head_dim; }
  float scale = 0.f;
  const void *k_cache = nullptr, *v_cache = nullptr;
  // What only the float32-arithmetic kernel computes: a bound cap * tanh(score / cap) on the
  // score, and a penalty slope[head] * distance subtracted from it.  With either, that kernel
  // runs whatever the dtype.
  float score_cap = 0.f;
  const float* distance_slopes = nullptr;
  // exp(sinks[head]) once more in the softmax's denominator (float32 [n_q])
  const float* sinks = nullptr;
  bool plain_scores() const {
    return score_cap <= 0.f && distance_slopes == nullptr && sinks == nullptr;
  }
};

struct AttendForce {
  int kernel = 0;
  int tile_rows = -1, staged = -1, splits = 0, split_blocks = 0;
};

AttentionPlan plan_for(int dtype, const AttendArgs& a, const mk_step_view& step,
                       const AttendForce& force = {});

// Causal grouped-query attention of every token of the step over its sequence's cached keys;
// [m, n_q d] of the compute dtype into `out` (allocated when null).
void* attend(Launch& l, const Queries& q, const AttendArgs& a, const StepArrays& s,
             const mk_step_view& step, AttendForce force = {}, void* out = nullptr);

// The attention and its output projection into the residual stream h [m, hidden] (+ bias), as
// project_into_stream does it (pending / pending_count: partial sums left for the next norm).
// Decoding with the keys split over workgroups takes two kernels instead of three: the
// attention leaves its partial results, and one kernel merges them and multiplies by w_o
// (`fold`: -1 where the sizes allow and it pays, 0 never, 1 wherever the sizes allow).  With
// h_fixed the residual stream is that one (h is ignored) and nothing is left pending.
void attend_and_project(Launch& l, const Queries& q, const AttendArgs& a, const StepArrays& s,
                        const mk_step_view& step, const void* w_o, const void* b_o, int b_o_dtype,
                        int hidden, float* h, const float*& pending, int& pending_count,
                        AttendForce force = {}, int fold = -1, long long* h_fixed = nullptr);

// Two maps per head combined: a [m, heads, 2, dv] -> [m, heads dv] in the compute dtype,
// Two maps a head attended, combined, normed and gated in one matrix-core kernel (see
// mk_attention_maps), or null where that kernel does not serve the step: another dtype than
// bfloat16, the library not loaded, sizes it is not compiled for, a score that is not plain.
// `a` describes the maps as heads (n_q = heads * 2, as `attend` takes it).
void* attend_maps(Launch& l, const Queries& q, const AttendArgs& a, const StepArrays& s,
                  const mk_step_view& step, const float* gate, int gate_stride, float lambda,
                  float eps, float out_scale);
// a .* sigmoid(gate): [m, width] of the compute dtype times the sigmoid of float32 columns
// (rows gate_stride apart), into a new tensor.
void* gate_mul(Launch& l, const void* a, int m, int width, const float* gate, int gate_stride);
// The residual stream itself as a sublayer's input: h += pending, x = h in the compute dtype.
void* stream_cast(Launch& l, float* h, int tokens, int hidden, const float* pending,
                  int pending_count);
// (a1 - lambda a2) / rms * out_scale * sigmoid(gate) (see mk_diff_heads).
void* diff_heads(Launch& l, const void* a, int m, int heads, int dv, const float* gate,
                 int gate_stride, float lambda, float eps, float out_scale);

// h += scale .* (rmsnorm(y + its partial sums) * weight) (see mk_norm_scale_add).
// With `x_out` the new h also goes there, in the compute dtype.
void norm_scale_add(Launch& l, float* h, const float* y, const float* partials, int count,
                    const void* weight, int weight_dtype, const float* scale, float eps,
                    int tokens, int hidden, void* x_out = nullptr);

// Retention: one projection [q | k | v | gate] in float32, the decayed recurrence per head from
// the state earlier steps left (queries and keys turned, keys scaled), a norm per head, the
// gate silu(gate columns), the output projection into h.  `state` holds [heads, dim, vdim]
// floats per slot.
struct RetentionArgs {
  const void* w_in = nullptr;      // [2 heads dim + 2 heads vdim, hidden]
  const void* w_out = nullptr;     // [hidden, heads vdim]
  const float* decay = nullptr;    // [heads]
  int heads = 0, dim = 0, vdim = 0;
  float k_scale = 1.f, eps = 0.f;
  PositionDesc pos;
  float* state = nullptr;
  long long slot_floats = 0;
  int in_width() const { return 2 * heads * dim + 2 * heads * vdim; }
};
void retention(Launch& l, const void* x, int m, int hidden, const RetentionArgs& a,
               const mk_step_view& step, float* h, const float*& pending, int& pending_count);

// A matrix memory with gates (the mLSTM cell, see mk_mlstm_scan): one projection
// [q | k | v | gate | i | f] in float32 with a bias on its last 2 heads columns, the recurrence
// per head from the state earlier steps left, a norm per head with a weight over all heads'
// columns, the gate sigmoid(gate columns), the output projection into h.
struct MlstmArgs {
  const void* w_in = nullptr;      // [2 heads dim + 2 heads vdim + 2 heads, hidden]
  const void* b_in = nullptr;      // [the same rows], zero but for the gates' rows
  int b_in_dtype = 0;
  const void* w_out = nullptr;     // [hidden, heads vdim]
  const float* norm = nullptr;     // [heads vdim]
  int heads = 0, dim = 0, vdim = 0;
  float q_scale = 1.f, gate_cap = 0.f, eps = 0.f;
  float* state = nullptr;
  long long slot_floats = 0;
  int in_width() const { return 2 * heads * dim + 2 * heads * vdim + 2 * heads; }
};
void mlstm(Launch& l, const void* x, int m, int hidden, const MlstmArgs& a,
           const mk_step_view& step, float* h, const float*& pending, int& pending_count);

// act = silu(x Wg^T) * (x Wu^T) for w = [Wg | Wu] stacked [2 inter, k].  tile_config: -2 by the
// sizes, else the tiled kernel with that configuration (-1: its own choice).
// `fold` as for qkv_project.
void* gated(Launch& l, const void* x, int m, int k, const void* w_gate_up, int inter,
            int tile_config = -2, const NormFold* fold = nullptr, const GateAct& act = {});

// h += act(x Wu^T) Wd^T for an activation of one operand (MK_UNARY_*), or partial sums left as
// project_into_stream leaves them.
void unary_mlp(Launch& l, const void* x, int m, int hidden, const void* w_up, const void* w_down,
               int inter, int act, float* h, const float*& pending, int& pending_count);

// A state-space mixer: in-projection [z | x | B | C | dt] in float32, the short convolution
// over x, B, C with its carried inputs, the recurrence from the state earlier steps left, the
// gate, the norm in groups, the output projection into h.  `state` holds, per slot of
// `slot_floats` floats, the carried inputs followed by the recurrent state.
struct StateSpaceArgs {
  const void* w_in = nullptr;      // [2 inner + 2 groups N + heads, hidden]
  const void *conv_w = nullptr, *conv_b = nullptr;   // [channels, taps], [channels]
  const void *dt_bias = nullptr, *a_log = nullptr, *d_skip = nullptr;   // [heads]
  const void* norm = nullptr;      // [inner]
  int vector_dtype = 0;
  const void* w_out = nullptr;     // [hidden, inner]
  int heads = 0, vdim = 0, state_size = 0, groups = 0, taps = 0, norm_groups = 1;
  float eps = 0.f;
  float* state = nullptr;
  long long slot_floats = 0;
  int inner() const { return heads * vdim; }
  int channels() const { return heads * vdim + 2 * groups * state_size; }
  int in_width() const { return 2 * heads * vdim + 2 * groups * state_size + heads; }
  long long carried_floats() const { return (long long)(taps - 1) * channels(); }
};
void state_space(Launch& l, const void* x, int m, int hidden, const StateSpaceArgs& a,
                 const mk_step_view& step, float* h, const float*& pending, int& pending_count);

// h += mult * (rmsnorm(a) wa + rmsnorm(b) wb), a = ya + its partial sums (see mk_normed_sum).
void normed_sum(Launch& l, float* h, const float* ya, const float* pa, int na, const void* wa,
                const float* yb, const float* pb, int nb, const void* wb, int weight_dtype,
                float eps, float mult, int tokens, int hidden);

// h <- [h | kept] W^T: the stream re-entered through a projection of itself beside a stream
// kept from earlier in the step.
void stream_mix(Launch& l, float* h, const float* kept, int m, int hidden, const void* w);
void copy_stream(Launch& l, float* dst, const float* src, long long n);

// y[t, head, :] = W[head] x[t, head, :] for every head: x rows `lda` apart with head `head`
// at x + head * x_head, W [heads, n, k], y rows `ldo` apart with the head at out + head * o_head
// (elements).  `out` is allocated as [m, heads * n] when null (then ldo = heads * n, o_head = n).
void* linear_per_head(Launch& l, const void* x, int m, int heads, int lda, int x_head,
                      const void* w, int n, int k, void* out, int ldo, int o_head);

// Attention through a low-rank latent shared by the heads.  Per token the cache holds one key
// row [c | r] (c the normed latent of kv_rank, r the rotated key part of `rot`) and c once
// more as the value; a query head h scores (W_uk[h]^T q_h) . c + rot(q_rot_h) . r, and its
// output is W_uv[h] applied to the attention's weighted sum of latents.
struct LatentArgs {
  const void* w_down = nullptr;    // [q_rank + kv_rank + rot + gate_cols, hidden]: query latent, c, r, gate
  const void *q_norm = nullptr, *kv_norm = nullptr;
  int norm_dtype = 0;
  float eps = 0.f;
  const void* w_uq = nullptr;      // [heads (dim + rot), q_rank]
  const void* w_uk_t = nullptr;    // [heads, kv_rank, dim]: W_uk per head, transposed
  const void* w_uv = nullptr;      // [heads, vdim, kv_rank]
  int heads = 0, dim = 0, rot = 0, vdim = 0, q_rank = 0, kv_rank = 0;
  // q_rank 0: the queries come straight from the input, w_uq being [heads (dim + rot), hidden].
  // gate_cols: further rows of w_down whose float32 products belong to the caller (a gate).
  int gate_cols = 0;
  int window = 0;                  // > 0: a query sees itself and the window - 1 tokens before it
  const float* sinks = nullptr;    // [heads]: exp(sink) once more in the softmax's denominator
  PositionDesc pos;                // over the first pos.rotary_dim dims of the rotated parts
  void *k_cache = nullptr, *v_cache = nullptr;
  int page_size = 1;
  bool writes = true;
  // rows as the cache holds them: padded to a shape the matrix-core attention takes
  int key_width() const {
    int k, v;
    latent_cache_widths(kv_rank + rot, kv_rank, k, v);
    return k;
  }
  int value_width() const {
    int k, v;
    latent_cache_widths(kv_rank + rot, kv_rank, k, v);
    return v;
  }
};
// Down-projection, norms, rotation and cache write, query up-projection; the queries come back
// as rows [heads, kv_rank + rot] = [absorbed | rotated].
// `raw` / `raw_stride`, when not null, receive the float32 down-projection (the gate's
// columns are its last gate_cols).
Queries latent_queries(Launch& l, const void* x, int m, int hidden, const LatentArgs& a,
                       const StepArrays& s, const float** raw = nullptr, int* raw_stride = nullptr);
// The attention over the cached latents: [m, heads, value_width()] weighted sums of them.
struct LatentPlan {
  bool mfma = false;
  int parts = 1, num_tiles = 0;
  int tile_rows = 16;      // 64: a workgroup's wavefronts share the keys through LDS (prompts)
};
LatentPlan latent_plan(int dtype, const LatentArgs& a, const mk_step_view& step);
void* latent_attend(Launch& l, const Queries& q, const LatentArgs& a, float scale,
                    const StepArrays& s, const mk_step_view& step);
// [m, heads, value_width()] weighted sums of latents -> [m, heads vdim] values.
void* latent_values(Launch& l, const void* summed, int m, const LatentArgs& a);

// Routed experts: router logits in float32, the `top` of softmax, and
// y += sum_j weight_j * down_ej(act(gate_ej x, up_ej x)); y float32 [m, hidden].
struct ExpertArgs {
  const void* w_router = nullptr;    // [experts, hidden]
  const void* w_gate_up = nullptr;   // [experts, 2 ff, hidden]
  const void* w_down = nullptr;      // [experts, hidden, ff]
  int experts = 0, top = 0, ff = 0;
  float scale = 1.f;
  int renormalize = 0;
  GateAct act;
  // A shared expert every token runs, added beside the chosen ones (null: none): a gated
  // feed-forward [2 shared_ff, hidden] / [hidden, shared_ff] with an activation of its own,
  // multiplied by sigmoid(x . shared_gate) when shared_gate [hidden] is there.
  const void *shared_gate_up = nullptr, *shared_down = nullptr, *shared_gate = nullptr;
  int shared_ff = 0;
  GateAct shared_act;
};
// The shared expert's down-projection goes into y or is left as partial sums (pending).
void routed_experts(Launch& l, const void* x, int m, int hidden, const ExpertArgs& a, float* y,
                    const float*& pending, int& pending_count);

}  // namespace mercury
