#include "builtin.h"

#include <cstdio>
#include <cstring>
#include <exception>

#include "../host/program.h"
#include "kernels.h"

namespace mercury {

namespace {

// Run `body`; a thrown error becomes the non-zero return and the context's message.
template <typename F>
int guarded(mk_op_context* ctx, F body) {
  try {
    body();
    return 0;
  } catch (const std::exception& e) {
    std::snprintf(ctx->error, sizeof ctx->error, "%s", e.what());
    return 1;
  }
}

StepArrays arrays_of(const mk_step_view& s, int group) {
  if (group < 0 || group >= s.num_groups) {
    throw KernelError("the step has no block table for cache group " + std::to_string(group));
  }
  StepArrays a;
  a.positions = s.positions;
  a.token_seq = s.token_seq;
  a.cu_q = s.cu_q;
  a.kv_len = s.kv_len;
  a.table = s.tables[group];
  a.table_stride = s.widths[group];
  return a;
}

int run_embed(const void* params, mk_op_context* ctx) {
  return guarded(ctx, [&] {
    const EmbedParams& p = *static_cast<const EmbedParams*>(params);
    Launch l(ctx);
    if (ctx->stream_fixed) {
      embed_fixed(l, ctx->step->token_ids, p.table, p.table_dtype, ctx->h_fixed,
                  ctx->step->num_tokens, ctx->hidden, p.vocab, p.scale);
      return;
    }
    embed(l, ctx->step->token_ids, p.table, p.table_dtype, ctx->h, ctx->step->num_tokens,
          ctx->hidden, p.vocab, p.scale);
  });
}

// The x an operation reads in a step in fixed point: a norm left for it to fold in (x is
// null then), or an x that exists.
const NormFold* fold_of(const mk_op_context* ctx, NormFold& fold) {
  if (!ctx->stream_fixed || ctx->x != nullptr || ctx->norm_weight == nullptr) return nullptr;
  fold.h64 = ctx->h_fixed;
  fold.weight = ctx->norm_weight;
  fold.weight_dtype = ctx->norm_weight_dtype;
  fold.eps = ctx->norm_eps;
  return &fold;
}

int run_norm(const void* params, mk_op_context* ctx) {
  return guarded(ctx, [&] {
    const NormParams& p = *static_cast<const NormParams*>(params);
    const mk_step_view& s = *ctx->step;
    Launch l(ctx);
    const int rows = p.select_rows ? s.num_rows : s.num_tokens;
    if (ctx->stream_fixed) {
      if (ctx->pending_count > 0) throw KernelError("partial sums beside a stream in fixed point");
      ctx->out_x_rows = rows;
      ctx->out_x_live = 1;
      if (p.select_rows) {   // few rows for a head that reads an x that exists
        ctx->out_x = rmsnorm_fixed(l, ctx->h_fixed, ctx->hidden, p.weight, p.weight_dtype, p.eps,
                                   s.logit_rows, rows);
      } else {               // left to the projection behind
        ctx->out_norm_weight = p.weight;
        ctx->out_norm_weight_dtype = p.weight_dtype;
        ctx->out_norm_eps = p.eps;
      }
      return;
    }
    ctx->out_x = rmsnorm(l, ctx->h, s.num_tokens, ctx->hidden, ctx->pending, ctx->pending_count,
                         p.weight, p.weight_dtype, p.eps, p.select_rows ? s.logit_rows : nullptr,
                         rows, nullptr, p.round_once != 0);
    ctx->out_x_rows = rows;
    ctx->out_x_live = 1;
  });
}

AttendArgs attend_args(const AttentionParams& p) {
  AttendArgs a;
  a.n_q = p.qkv.n_q;
  a.n_kv = p.qkv.n_kv;
  a.head_dim = p.qkv.head_dim;
  a.page_size = p.qkv.page_size;
  a.window = p.window;
  a.scale = p.scale;
  a.k_cache = p.qkv.k_cache;
  a.v_cache = p.qkv.v_cache;
  a.score_cap = p.score_cap;
  a.distance_slopes = p.distance_slopes;
  a.sinks = p.sinks;
  a.value_dim = p.prep.value_dim;
  a.keep_first = p.keep_first;
  // two maps a head: each is a query of its own over the same keys and values
  if (p.prep.maps > 1) a.n_q = p.qkv.n_q * p.prep.maps;
  return a;
}

int run_attention(const void* params, mk_op_context* ctx) {
  return guarded(ctx, [&] {
    const AttentionParams& p = *static_cast<const AttentionParams*>(params);
    const mk_step_view& s = *ctx->step;
    if (ctx->x_rows != s.num_tokens) throw KernelError("attention reads an x of every token");
    Launch l(ctx);
    const StepArrays arrays = arrays_of(s, p.group);
    NormFold fold;
    if (p.prep.active() && ctx->stream_fixed) {
      throw KernelError("attention: norms over q and k, a query temperature or values that are "
                        "keys do not run on a stream in fixed point");
    }
    if (p.out_gate) {
      // a sigmoid gate on every column of the heads' outputs, its logits the last columns of
      // the stacked projection
      if (p.prep.maps != 1 || p.head_gate) throw KernelError("attention: one gate, and one map a head with it");
      const float* raw = nullptr;
      int raw_stride = 0;
      const Queries q = qkv_prepared(l, ctx->x, s.num_tokens, ctx->hidden, p.qkv, p.prep, arrays,
                                     &raw, &raw_stride);
      const AttendArgs a = attend_args(p);
      const int inner = p.qkv.n_q * a.v_dim();
      const void* attended = attend(l, q, a, arrays, s);
      const void* gated = gate_mul(l, attended, s.num_tokens, inner,
                                   raw ? raw + (raw_stride - inner) : nullptr, raw_stride);
      project_into_stream(l, gated, s.num_tokens, p.w_o, ctx->hidden, inner, p.b_o, p.b_o_dtype,
                          ctx->h, ctx->out_pending, ctx->out_pending_count);
      return;
    }
    if (p.prep.maps > 1 || p.head_gate) {
      // maps combined, normed per head and gated between the attention and its projection
      if (p.prep.maps != 1 && p.prep.maps != 2) throw KernelError("attention: one or two maps a head");
      const float* raw = nullptr;
      int raw_stride = 0;
      const Queries q = qkv_prepared(l, ctx->x, s.num_tokens, ctx->hidden, p.qkv, p.prep, arrays,
                                     &raw, &raw_stride);
      const AttendArgs a = attend_args(p);
      const float* gate = p.head_gate && raw ? raw + (raw_stride - p.prep.extra_cols) : nullptr;
      if (p.prep.maps == 1) throw KernelError("attention: a gate per head comes with two maps");
      // bfloat16 at sizes the matrix cores take: one kernel attends both maps and finishes the
      // head; else the float32-arithmetic attention over the maps as heads, then the tail
      const void* heads = attend_maps(l, q, a, arrays, s, gate, raw_stride, p.diff_lambda,
                                      p.diff_eps, p.diff_scale);
      if (!heads) {
        const void* attended = attend(l, q, a, arrays, s);
        heads = diff_heads(l, attended, s.num_tokens, p.qkv.n_q, a.v_dim(), gate, raw_stride,
                           p.diff_lambda, p.diff_eps, p.diff_scale);
      }
      project_into_stream(l, heads, s.num_tokens, p.w_o, ctx->hidden, p.qkv.n_q * a.v_dim(), p.b_o,
                          p.b_o_dtype, ctx->h, ctx->out_pending, ctx->out_pending_count);
      return;
    }
    const Queries q = p.prep.active()
        ? qkv_prepared(l, ctx->x, s.num_tokens, ctx->hidden, p.qkv, p.prep, arrays)
        : qkv_project(l, ctx->x, s.num_tokens, ctx->hidden, p.qkv, arrays, {}, fold_of(ctx, fold));
    attend_and_project(l, q, attend_args(p), arrays, s, p.w_o, p.b_o, p.b_o_dtype, ctx->hidden,
                       ctx->h, ctx->out_pending, ctx->out_pending_count, {}, -1, ctx->h_fixed);
  });
}

int tiles_attention(const void* params, const mk_step_shape* shape, mk_tile_need* out) {
  const AttentionParams& p = *static_cast<const AttentionParams*>(params);
  mk_step_view view;
  std::memset(&view, 0, sizeof view);
  view.num_seqs = shape->num_seqs;
  view.counts = shape->counts;
  view.max_q_len = shape->max_q_len;
  view.max_kv_len = shape->max_kv_len;
  const AttentionPlan plan = plan_for(shape->dtype, attend_args(p), view);
  if (!plan.mfma) return 0;
  out->group = p.qkv.n_q * (p.prep.maps > 1 ? p.prep.maps : 1) / p.qkv.n_kv;
  out->tile_rows = plan.tile_rows;
  return 1;
}

int run_gated_mlp(const void* params, mk_op_context* ctx) {
  return guarded(ctx, [&] {
    const GatedMlpParams& p = *static_cast<const GatedMlpParams*>(params);
    const int m = ctx->step->num_tokens;
    if (ctx->x_rows != m) throw KernelError("the gated projection reads an x of every token");
    Launch l(ctx);
    NormFold fold;
    const void* act = gated(l, ctx->x, m, ctx->hidden, p.w_gate_up, p.inter, -2, fold_of(ctx, fold),
                            p.act);
    if (ctx->stream_fixed) {
      project_into_fixed(l, act, m, p.w_down, ctx->hidden, p.inter, nullptr, kF32, ctx->h_fixed);
      return;
    }
    project_into_stream(l, act, m, p.w_down, ctx->hidden, p.inter, nullptr, kF32, ctx->h,
                        ctx->out_pending, ctx->out_pending_count);
  });
}

int run_latent_attention(const void* params, mk_op_context* ctx) {
  return guarded(ctx, [&] {
    const LatentAttentionParams& p = *static_cast<const LatentAttentionParams*>(params);
    const LatentArgs& a = p.latent;
    const mk_step_view& s = *ctx->step;
    if (ctx->x_rows != s.num_tokens) throw KernelError("attention reads an x of every token");
    Launch l(ctx);
    const StepArrays arrays = arrays_of(s, p.group);
    const float* raw = nullptr;
    int raw_stride = 0;
    const Queries q = latent_queries(l, ctx->x, s.num_tokens, ctx->hidden, a, arrays, &raw, &raw_stride);
    const void* summed = latent_attend(l, q, a, p.scale, arrays, s);
    const void* values = latent_values(l, summed, s.num_tokens, a);
    if (p.out_gate) {
      const int inner = a.heads * a.vdim;
      if (a.gate_cols != inner) throw KernelError("latent attention: a gate column per value column");
      values = gate_mul(l, values, s.num_tokens, inner, raw ? raw + (raw_stride - inner) : nullptr,
                        raw_stride);
    }
    project_into_stream(l, values, s.num_tokens, p.w_o, ctx->hidden, a.heads * a.vdim, nullptr, kF32,
                        ctx->h, ctx->out_pending, ctx->out_pending_count);
  });
}

int tiles_latent_attention(const void* params, const mk_step_shape* shape, mk_tile_need* out) {
  const LatentAttentionParams& p = *static_cast<const LatentAttentionParams*>(params);
  mk_step_view view;
  std::memset(&view, 0, sizeof view);
  view.num_seqs = shape->num_seqs;
  view.counts = shape->counts;
  view.max_q_len = shape->max_q_len;
  view.max_kv_len = shape->max_kv_len;
  const LatentPlan plan = latent_plan(shape->dtype, p.latent, view);
  if (!plan.mfma) return 0;
  out->group = p.latent.heads;
  out->tile_rows = plan.tile_rows;
  return 1;
}

int run_routed_experts(const void* params, mk_op_context* ctx) {
  return guarded(ctx, [&] {
    const RoutedExpertsParams& p = *static_cast<const RoutedExpertsParams*>(params);
    const int m = ctx->step->num_tokens;
    if (ctx->x_rows != m) throw KernelError("the experts read an x of every token");
    Launch l(ctx);
    routed_experts(l, ctx->x, m, ctx->hidden, p.experts, ctx->h, ctx->out_pending,
                   ctx->out_pending_count);
  });
}

int run_stream_cast(const void*, mk_op_context* ctx) {
  return guarded(ctx, [&] {
    Launch l(ctx);
    const int tokens = ctx->step->num_tokens;
    ctx->out_x = stream_cast(l, ctx->h, tokens, ctx->hidden, ctx->pending, ctx->pending_count);
    ctx->out_x_rows = tokens;
    ctx->out_x_live = 1;
  });
}

int run_mlstm(const void* params, mk_op_context* ctx) {
  return guarded(ctx, [&] {
    const MlstmParams& p = *static_cast<const MlstmParams*>(params);
    const mk_step_view& s = *ctx->step;
    if (ctx->x_rows != s.num_tokens) throw KernelError("the mixer reads an x of every token");
    Launch l(ctx);
    mlstm(l, ctx->x, s.num_tokens, ctx->hidden, p.args, s, ctx->h, ctx->out_pending,
          ctx->out_pending_count);
  });
}

int run_retention(const void* params, mk_op_context* ctx) {
  return guarded(ctx, [&] {
    const RetentionParams& p = *static_cast<const RetentionParams*>(params);
    const mk_step_view& s = *ctx->step;
    if (ctx->x_rows != s.num_tokens) throw KernelError("the mixer reads an x of every token");
    Launch l(ctx);
    retention(l, ctx->x, s.num_tokens, ctx->hidden, p.args, s, ctx->h, ctx->out_pending,
              ctx->out_pending_count);
  });
}

// The sublayer adds into a zeroed buffer in the stream's place; what it leaves as partial sums
// is added to that buffer inside the kernel that norms, scales and adds.
int run_post_norm(const void* params, mk_op_context* ctx) {
  const PostNormParams& p = *static_cast<const PostNormParams*>(params);
  const int tokens = ctx->step->num_tokens;
  float* const h = ctx->h;
  float* y = nullptr;
  {
    const int code = guarded(ctx, [&] {
      Launch l(ctx);
      y = zeros(l, (long long)tokens * ctx->hidden);
    });
    if (code) return code;
  }
  ctx->h = y;
  ctx->out_x = nullptr;
  ctx->out_x_rows = ctx->out_x_live = 0;
  ctx->out_pending = nullptr;
  ctx->out_pending_count = 0;
  const int ran = p.run(static_cast<const char*>(params) + p.offset, ctx);
  ctx->h = h;
  if (ran) return ran;
  const float* parts = ctx->out_pending;
  const int count = ctx->out_pending_count;
  ctx->out_x = nullptr;
  ctx->out_x_rows = ctx->out_x_live = 0;
  ctx->out_pending = nullptr;
  ctx->out_pending_count = 0;
  ctx->out_logits_ready = 0;
  return guarded(ctx, [&] {
    Launch l(ctx);
    void* x = p.gives_x ? l.alloc((size_t)tokens * ctx->hidden * l.elem()) : nullptr;
    norm_scale_add(l, h, y, parts, count, p.weight, p.weight_dtype, p.scale, p.eps, tokens,
                   ctx->hidden, x);
    if (p.gives_x) {
      ctx->out_x = x;
      ctx->out_x_rows = tokens;
      ctx->out_x_live = 1;
    }
  });
}

int tiles_post_norm(const void* params, const mk_step_shape* shape, mk_tile_need* out) {
  const PostNormParams& p = *static_cast<const PostNormParams*>(params);
  return p.tiles ? p.tiles(static_cast<const char*>(params) + p.offset, shape, out) : 0;
}

int run_unary_mlp(const void* params, mk_op_context* ctx) {
  return guarded(ctx, [&] {
    const UnaryMlpParams& p = *static_cast<const UnaryMlpParams*>(params);
    const int m = ctx->step->num_tokens;
    if (ctx->x_rows != m) throw KernelError("the feed-forward reads an x of every token");
    Launch l(ctx);
    unary_mlp(l, ctx->x, m, ctx->hidden, p.w_up, p.w_down, p.inter, p.act, ctx->h,
              ctx->out_pending, ctx->out_pending_count);
  });
}

int run_state_space(const void* params, mk_op_context* ctx) {
  return guarded(ctx, [&] {
    const StateSpaceParams& p = *static_cast<const StateSpaceParams*>(params);
    const mk_step_view& s = *ctx->step;
    if (ctx->x_rows != s.num_tokens) throw KernelError("the mixer reads an x of every token");
    Launch l(ctx);
    state_space(l, ctx->x, s.num_tokens, ctx->hidden, p.args, s, ctx->h, ctx->out_pending,
                ctx->out_pending_count);
  });
}

// Every sublayer adds into a zeroed buffer of its own in the stream's place; what it leaves as
// partial sums is added to that buffer inside the kernel that norms and sums.
int run_normed_sum(const void* params, mk_op_context* ctx) {
  const NormedSumParams& p = *static_cast<const NormedSumParams*>(params);
  const int tokens = ctx->step->num_tokens;
  const long long n = (long long)tokens * ctx->hidden;
  float* const h = ctx->h;
  float* y[kNormedSumMax] = {nullptr};
  const float* parts[kNormedSumMax] = {nullptr};
  int counts[kNormedSumMax] = {0};
  if (p.count < 1 || p.count > kNormedSumMax) {
    std::snprintf(ctx->error, sizeof ctx->error, "normed_sum: %d sublayers", p.count);
    return 1;
  }
  // one fill for the buffers of all sublayers (each a multiple of 64 floats apart)
  const long long pitch = (n + 63) / 64 * 64;
  {
    float* all = nullptr;
    const int code = guarded(ctx, [&] {
      Launch l(ctx);
      all = zeros(l, pitch * p.count);
    });
    if (code) return code;
    for (int i = 0; i < p.count; ++i) y[i] = all ? all + pitch * i : nullptr;
  }
  for (int i = 0; i < p.count; ++i) {
    ctx->h = y[i];
    ctx->out_x = nullptr;
    ctx->out_x_rows = ctx->out_x_live = 0;
    ctx->out_pending = nullptr;
    ctx->out_pending_count = 0;
    const int ran = p.sub[i].run(static_cast<const char*>(params) + p.sub[i].offset, ctx);
    ctx->h = h;
    if (ran) return ran;
    parts[i] = ctx->out_pending;
    counts[i] = ctx->out_pending_count;
  }
  ctx->out_x = nullptr;
  ctx->out_x_rows = ctx->out_x_live = 0;
  ctx->out_pending = nullptr;
  ctx->out_pending_count = 0;
  ctx->out_logits_ready = 0;
  return guarded(ctx, [&] {
    Launch l(ctx);
    normed_sum(l, h, y[0], parts[0], counts[0], p.sub[0].weight, p.count > 1 ? y[1] : nullptr,
               parts[1], counts[1], p.count > 1 ? p.sub[1].weight : nullptr, p.weight_dtype, p.eps,
               p.mult, tokens, ctx->hidden);
  });
}

int tiles_normed_sum(const void* params, const mk_step_shape* shape, mk_tile_need* out) {
  const NormedSumParams& p = *static_cast<const NormedSumParams*>(params);
  for (int i = 0; i < p.count; ++i) {
    if (p.sub[i].tiles &&
        p.sub[i].tiles(static_cast<const char*>(params) + p.sub[i].offset, shape, out) > 0) {
      return 1;
    }
  }
  return 0;
}

int run_keep_stream(const void*, mk_op_context* ctx) {
  return guarded(ctx, [&] {
    Launch l(ctx);
    if (!l.dry() && !ctx->kept) throw KernelError("keep_stream: the step has no room to keep a stream");
    const long long n = (long long)ctx->step->num_tokens * ctx->hidden;
    if (ctx->pending_count > 0) scaled_add(l, ctx->h, nullptr, ctx->pending, ctx->pending_count, nullptr, 0, n, 1.f);
    copy_stream(l, ctx->kept, ctx->h, (long long)ctx->step->num_tokens * ctx->hidden);
  });
}

int run_stream_mix(const void* params, mk_op_context* ctx) {
  return guarded(ctx, [&] {
    const StreamMixParams& p = *static_cast<const StreamMixParams*>(params);
    Launch l(ctx);
    if (!l.dry() && !ctx->kept) throw KernelError("stream_mix: no stream was kept in this step");
    const long long n = (long long)ctx->step->num_tokens * ctx->hidden;
    // what the projection before left as partial sums belongs to the stream first
    if (ctx->pending_count > 0) scaled_add(l, ctx->h, nullptr, ctx->pending, ctx->pending_count, nullptr, 0, n, 1.f);
    stream_mix(l, ctx->h, ctx->kept, ctx->step->num_tokens, ctx->hidden, p.weight);
  });
}

int run_parallel(const void* params, mk_op_context* ctx) {
  const ParallelParams& p = *static_cast<const ParallelParams*>(params);
  const long long n = (long long)ctx->step->num_tokens * ctx->hidden;
  float* const h = ctx->h;
  // A factor of one needs no buffer: the sublayers add into the stream itself, and what they
  // leave as partial sums is passed on (the first) or added here (any further ones).
  const bool direct = p.mult == 1.f;
  float* y = nullptr;
  if (!direct) {
    const int code = guarded(ctx, [&] {
      Launch l(ctx);
      y = zeros(l, n);
    });
    if (code) return code;
  }
  const float* parts[kParallelMax] = {nullptr};
  int counts[kParallelMax] = {0};
  for (int i = 0; i < p.count; ++i) {
    ctx->h = direct ? h : y;
    ctx->out_x = nullptr;
    ctx->out_x_rows = ctx->out_x_live = 0;
    ctx->out_pending = nullptr;
    ctx->out_pending_count = 0;
    const int code = p.sub[i].run(static_cast<const char*>(params) + p.sub[i].offset, ctx);
    ctx->h = h;
    if (code) return code;
    parts[i] = ctx->out_pending;
    counts[i] = ctx->out_pending_count;
  }
  ctx->out_x = nullptr;
  ctx->out_x_rows = ctx->out_x_live = 0;
  ctx->out_pending = nullptr;
  ctx->out_pending_count = 0;
  ctx->out_logits_ready = 0;
  return guarded(ctx, [&] {
    Launch l(ctx);
    int first = -1, second = -1;
    for (int i = 0; i < p.count; ++i) {
      if (!counts[i]) continue;
      if (first < 0) first = i;
      else if (second < 0) second = i;
      else scaled_add(l, direct ? h : y, nullptr, parts[i], counts[i], nullptr, 0, n, 1.f);
    }
    if (direct) {
      if (second >= 0) scaled_add(l, h, nullptr, parts[second], counts[second], nullptr, 0, n, 1.f);
      if (first >= 0) {
        ctx->out_pending = parts[first];
        ctx->out_pending_count = counts[first];
      }
      return;
    }
    // partial sums of at most two sublayers go into the sum directly
    scaled_add(l, h, y, first < 0 ? nullptr : parts[first], first < 0 ? 0 : counts[first],
               second < 0 ? nullptr : parts[second], second < 0 ? 0 : counts[second], n, p.mult);
  });
}

int tiles_parallel(const void* params, const mk_step_shape* shape, mk_tile_need* out) {
  const ParallelParams& p = *static_cast<const ParallelParams*>(params);
  for (int i = 0; i < p.count; ++i) {
    if (p.sub[i].tiles &&
        p.sub[i].tiles(static_cast<const char*>(params) + p.sub[i].offset, shape, out) > 0) {
      return 1;
    }
  }
  return 0;
}

int run_head(const void* params, mk_op_context* ctx) {
  return guarded(ctx, [&] {
    const HeadParams& p = *static_cast<const HeadParams*>(params);
    const int rows = ctx->step->num_rows;
    if (rows == 0) return;
    if (ctx->x_rows != rows) throw KernelError("the head reads an x of the wanted rows");
    Launch l(ctx);
    linear(l, ctx->x, rows, p.weight, ctx->vocab, ctx->hidden, p.bias, p.bias_dtype, ctx->logits,
           kF32, false);
    if (p.cap > 0.f) logit_cap(l, ctx->logits, (long long)rows * ctx->vocab, p.cap);
    ctx->out_logits_ready = 1;
  });
}

}  // namespace

void register_builtin_ops() {
  OpRegistry& r = OpRegistry::instance();
  r.add(OpKind{"embed", &run_embed, nullptr, MK_OP_FIXED_STREAM});
  r.add(OpKind{"norm", &run_norm, nullptr, MK_OP_FOLDS_PENDING | MK_OP_FIXED_STREAM});
  r.add(OpKind{"attention", &run_attention, &tiles_attention, MK_OP_READS_X | MK_OP_FIXED_STREAM});
  // The same operations under names that are not flagged for the fixed-point stream: a norm
  // that rounds once and an attention that norms q and k, scales its queries, takes its keys
  // as values or has sinks keep their whole program on the float32 stream.
  r.add(OpKind{"norm_once", &run_norm, nullptr, MK_OP_FOLDS_PENDING});
  r.add(OpKind{"attention_prepared", &run_attention, &tiles_attention, MK_OP_READS_X});
  r.add(OpKind{"gated_mlp", &run_gated_mlp, nullptr, MK_OP_READS_X | MK_OP_FIXED_STREAM});
  r.add(OpKind{"latent_attention", &run_latent_attention, &tiles_latent_attention, MK_OP_READS_X});
  r.add(OpKind{"routed_experts", &run_routed_experts, nullptr, MK_OP_READS_X});
  r.add(OpKind{"parallel", &run_parallel, &tiles_parallel, MK_OP_READS_X});
  r.add(OpKind{"unary_mlp", &run_unary_mlp, nullptr, MK_OP_READS_X});
  r.add(OpKind{"state_space", &run_state_space, nullptr, MK_OP_READS_X});
  r.add(OpKind{"normed_sum", &run_normed_sum, &tiles_normed_sum, MK_OP_READS_X});
  r.add(OpKind{"retention", &run_retention, nullptr, MK_OP_READS_X});
  r.add(OpKind{"mlstm", &run_mlstm, nullptr, MK_OP_READS_X});
  r.add(OpKind{"stream_cast", &run_stream_cast, nullptr, MK_OP_FOLDS_PENDING});
  r.add(OpKind{"post_norm", &run_post_norm, &tiles_post_norm, MK_OP_READS_X});
  r.add(OpKind{"keep_stream", &run_keep_stream, nullptr, MK_OP_KEPT_STREAM | MK_OP_FOLDS_PENDING});
  r.add(OpKind{"stream_mix", &run_stream_mix, nullptr, MK_OP_KEPT_STREAM | MK_OP_FOLDS_PENDING});
  r.add(OpKind{"head", &run_head, nullptr, MK_OP_READS_X | MK_OP_FIXED_STREAM});
  r.fixed_stream_tokens = &fixed_stream_tokens;
}

}  // namespace mercury
