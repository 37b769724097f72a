// The operation kinds the package's own parts lower themselves to, each a parameter block
// and a run function over the launch sequences of launch.h.  They are registered like any
// kind from outside would be (OpRegistry); the program walk knows none of them.
#pragma once

#include "launch.h"

namespace mercury {

// "embed": h = table[token_ids] * scale.
struct EmbedParams {
  const void* table = nullptr;
  int table_dtype = 0, vocab = 0;
  float scale = 1.f;
};

// "norm": x = rmsnorm(h + pending) * weight; with select_rows, of the step's wanted rows only
// (what an output head reads).
struct NormParams {
  const void* weight = nullptr;
  int weight_dtype = 0;
  float eps = 0.f;
  int select_rows = 0;
  int round_once = 0;     // x * rstd * weight rounded once, not the normalised value first
};

// "attention": q/k/v projection, position encoding, cache write, softmax attention over the
// cache, output projection into h (or left as partial sums).
struct AttentionParams {
  QkvArgs qkv;
  const void *w_o = nullptr, *b_o = nullptr;
  int b_o_dtype = 0;
  int group = 0;          // which of the step's block tables
  int window = 0;
  float scale = 0.f;
  float score_cap = 0.f;                    // > 0: the score is bounded to cap * tanh(. / cap)
  const float* distance_slopes = nullptr;   // [n_q]: slope * distance is subtracted from it
  const float* sinks = nullptr;             // [n_q]: exp(sink) once more in the denominator
  QkPrep prep;                              // norms over q and k, query temperature, v = k
  int keep_first = 0;                       // with a window: the first keys stay visible past it
  // Differential attention (prep.maps == 2): every head has two score maps over the same
  // values; o = a1 - lambda a2, divided by its root mean square over the head (eps), times
  // out_scale.  head_gate: the stacked projection ends in one gate column per head, and the
  // head's output is multiplied by its sigmoid (with or without two maps).
  float diff_lambda = 0.f, diff_eps = 0.f, diff_scale = 1.f;
  int head_gate = 0;
  // out_gate: the stacked projection ends in one gate column per column of the heads side by
  // side (n_q value_dim of them), and the attention's output is multiplied by their sigmoid
  // before the output projection.
  int out_gate = 0;
};

// "stream_cast": x = h + pending in the compute dtype: a sublayer that reads the residual
// stream itself, with no norm before it.
struct StreamCastParams {
  int unused = 0;
};

// "mlstm": a matrix memory with gates per head and request (launch.h), its output projection
// into h (or left as partial sums).
struct MlstmParams {
  MlstmArgs args;
};

// "retention": a decayed outer-product state per head and request (launch.h), its output
// projection into h (or left as partial sums).
struct RetentionParams {
  RetentionArgs args;
};

// "post_norm": one sublayer whose output is RMS-normed over the model width and multiplied,
// channel by channel, by a stored vector before it enters the stream:
// h += scale .* (rmsnorm(f(x)) * weight).  Laid out as "parallel": this header, then the
// sublayer's parameter block at `offset`.
struct PostNormParams {
  float eps = 0.f;
  int weight_dtype = 0;
  const void* weight = nullptr;
  const float* scale = nullptr;     // float32 [hidden], or null
  int gives_x = 0;                  // the new stream goes out as x too, in the compute dtype,
                                    // for an operation behind this one that reads the stream itself
  mk_op_run_fn run = nullptr;
  mk_op_tiles_fn tiles = nullptr;
  int flags = 0;
  int offset = 0;
};

// "unary_mlp": h += act(x Wu^T) Wd^T for an activation of one operand (or left as partial sums).
struct UnaryMlpParams {
  const void *w_up = nullptr, *w_down = nullptr;
  int inter = 0;
  int act = 0;
};

// "state_space": a state-space mixer over per-request state (launch.h), its output projection
// into h (or left as partial sums).
struct StateSpaceParams {
  StateSpaceArgs args;
};

// "normed_sum": mixers side by side on the same x; each one's output is RMS-normed over the
// model width with a plain weight of its own, and h += mult * their sum.  Laid out as
// "parallel": this header, then the sublayers' parameter blocks at `offset`.
constexpr int kNormedSumMax = 2;
struct NormedSumParams {
  float mult = 1.f, eps = 0.f;
  int count = 0;
  int weight_dtype = 0;
  struct Sub {
    mk_op_run_fn run = nullptr;
    mk_op_tiles_fn tiles = nullptr;
    int flags = 0;
    int offset = 0;
    const void* weight = nullptr;
  } sub[kNormedSumMax];
};

// "keep_stream": the residual stream as it stands is kept for the rest of the step.
// "stream_mix": h <- [h | kept] W^T, W [hidden, 2 hidden].
struct StreamMixParams {
  const void* weight = nullptr;
};

// "gated_mlp": h += (act(x Wg^T) * (x Wu^T)) Wd^T (or left as partial sums).
struct GatedMlpParams {
  const void *w_gate_up = nullptr, *w_down = nullptr;
  int inter = 0;
  GateAct act;
};

// "latent_attention": attention through a low-rank latent shared by the heads (launch.h),
// its output projection into h (or left as partial sums).
struct LatentAttentionParams {
  LatentArgs latent;
  const void* w_o = nullptr;   // [hidden, heads vdim]
  int group = 0;               // which of the step's block tables
  float scale = 0.f;
  // the down-projection ends in heads vdim gate columns whose sigmoid multiplies the heads'
  // values before the output projection
  int out_gate = 0;
};

// "routed_experts": h += sum over a token's chosen experts (launch.h).
struct RoutedExpertsParams {
  ExpertArgs experts;
};

// "parallel": sublayers that read the same x, their outputs summed, scaled and added:
// h += mult * (f_0(x) + f_1(x) ...).  Each sublayer is an operation of a registered kind that
// adds its output into h; here it gets a zeroed buffer in h's place.  The block is this header
// followed by the sublayers' parameter blocks at `offset` bytes from its start.
constexpr int kParallelMax = 4;
struct ParallelParams {
  float mult = 1.f;
  int count = 0;
  struct Sub {
    mk_op_run_fn run = nullptr;
    mk_op_tiles_fn tiles = nullptr;
    int flags = 0;
    int offset = 0;
  } sub[kParallelMax];
};

// "head": logits = x W^T (+ bias), optionally capped to cap * tanh(. / cap).
struct HeadParams {
  const void *weight = nullptr, *bias = nullptr;
  int bias_dtype = 0;
  float cap = 0.f;
};

void register_builtin_ops();

}  // namespace mercury
