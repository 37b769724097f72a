#include "launch.h"

#include <algorithm>
#include <string>
#include <vector>

#include "kernels.h"

namespace mercury {

void embed(Launch& l, const int* ids, const void* table, int table_dtype, float* out, int tokens,
           int hidden, int vocab, float scale) {
  if (l.dry() || tokens == 0) return;
  check_core(need_core().mk_embed(ids, table, table_dtype, out, tokens, hidden, vocab, scale,
                                  l.stream()), "embed");
}

void* rmsnorm(Launch& l, float* h, int tokens, int hidden, const float* pending, int pending_count,
              const void* weight, int weight_dtype, float eps, const int* rows, int out_rows,
              void* out, bool round_once) {
  if (!out) out = l.alloc((size_t)out_rows * hidden * l.elem());
  if (l.dry() || out_rows == 0) return out;
  check_core(need_core().mk_rmsnorm_rounding(h, pending, pending_count, (long long)tokens * hidden,
                                             weight, weight_dtype, eps, rows, out, l.dtype(),
                                             out_rows, hidden, round_once ? 1 : 0, l.stream()),
             "rmsnorm");
  return out;
}

void embed_fixed(Launch& l, const int* ids, const void* table, int table_dtype, long long* out,
                 int tokens, int hidden, int vocab, float scale) {
  if (l.dry() || tokens == 0) return;
  check_core(need_core().mk_embed_fixed(ids, table, table_dtype, out, tokens, hidden, vocab, scale,
                                        l.stream()), "embed");
}

void* rmsnorm_fixed(Launch& l, const long long* h64, int hidden, const void* weight,
                    int weight_dtype, float eps, const int* rows, int out_rows) {
  void* out = l.alloc((size_t)out_rows * hidden * l.elem());
  if (l.dry() || out_rows == 0) return out;
  check_core(need_core().mk_rmsnorm_fixed(h64, weight, weight_dtype, eps, rows, out, l.dtype(),
                                          out_rows, hidden, l.stream()), "rmsnorm");
  return out;
}

void project_into_fixed(Launch& l, const void* x, int m, const void* w, int n, int k,
                        const void* bias, int bias_dtype, long long* h64) {
  if (m == 0) return;
  const int bd = bias ? bias_dtype : kF32;
  if (mfma_eligible(l.dtype(), l.dtype(), m, k) && m <= 16) {
    if (l.dry()) return;
    const KernelTable& t = need_mfma();
    check_mfma(t.mk_linear_skinny_fixed(x, w, bias, bd, h64, m, n, k,
                                        t.mk_linear_skinny_slices(m, n, k), l.stream()),
               "project_into_fixed");
    return;
  }
  // whatever kernel takes the product, into a buffer, and that into the stream
  float* y = (float*)linear(l, x, m, w, n, k, bias, bias_dtype, nullptr, kF32, false);
  if (l.dry()) return;
  check_core(need_core().mk_fixed_add(h64, y, 1, (long long)m * n, (long long)m * n, l.stream()),
             "project_into_fixed");
}

void* silu_mul(Launch& l, const void* gate_up, int tokens, int inter, void* out) {
  if (!out) out = l.alloc((size_t)tokens * inter * l.elem());
  if (l.dry() || tokens == 0) return out;
  check_core(need_core().mk_silu_mul(gate_up, out, l.dtype(), tokens, inter, l.stream()), "silu_mul");
  return out;
}

void* gate_activation(Launch& l, const void* gate_up, int tokens, int inter, const GateAct& act,
                      void* out) {
  if (!out) out = l.alloc((size_t)tokens * inter * l.elem());
  if (l.dry() || tokens == 0) return out;
  check_core(need_core().mk_gate_act(gate_up, out, l.dtype(), tokens, inter, act.kind, act.limit,
                                     act.alpha, act.beta, l.stream()), "gate_activation");
  return out;
}

void scaled_add(Launch& l, float* h, const float* y, const float* a, int na, const float* b, int nb,
                long long n, float mult) {
  if (l.dry() || n == 0) return;
  check_core(need_core().mk_scaled_add(h, y, a, na, b, nb, n, mult, n, l.stream()), "scaled_add");
}

float* zeros(Launch& l, long long n) {
  float* p = (float*)l.alloc((size_t)n * 4);
  if (l.dry() || n == 0) return p;
  check_core(need_core().mk_fill_zero(p, n, l.stream()), "zeros");
  return p;
}

void logit_cap(Launch& l, float* logits, long long count, float cap) {
  if (l.dry() || count == 0) return;
  check_core(need_core().mk_logit_cap(logits, count, cap, l.stream()), "logit_cap");
}

void* linear(Launch& l, const void* x, int m, const void* w, int n, int k, const void* bias,
             int bias_dtype, void* out, int out_dtype, bool accumulate, LinearForce force) {
  if (accumulate && (!out || out_dtype != kF32) && !l.dry()) {
    throw KernelError("linear: accumulation needs a float32 `out`");
  }
  if (!out) out = l.alloc((size_t)m * n * element_size(out_dtype));
  if (l.dry() || m == 0) return out;
  const int bd = bias ? bias_dtype : kF32;
  switch (choose_linear(l.dtype(), m, n, k, bias != nullptr, accumulate, out_dtype, force.kernel)) {
    case LinearKind::GENERIC:
      check_core(need_core().mk_linear_generic(x, w, l.dtype(), bias, bd, out, out_dtype,
                                               accumulate ? 1 : 0, m, n, k, k, n, l.stream()),
                 "linear");
      break;
    case LinearKind::SKINNY:
      check_mfma(need_mfma().mk_linear_skinny(x, w, (float*)out, m, n, k, 1, l.stream()), "linear");
      break;
    case LinearKind::SKINNY_ACC:
      check_mfma(need_mfma().mk_linear_skinny_acc(x, w, bias, bd, (float*)out, m, n, k, l.stream()),
                 "linear");
      break;
    default:
      check_mfma(need_mfma().mk_linear_tiled(x, w, bias, bd, out, out_dtype, accumulate ? 1 : 0, m,
                                             n, k, n, force.tile_config, l.stream()), "linear");
  }
  return out;
}

float* linear_partials(Launch& l, const void* x, int m, const void* w, int n, int k, int& slices) {
  if (!mfma_eligible(l.dtype(), l.dtype(), m, k)) {
    throw KernelError("linear_partials: bfloat16 operands with K a multiple of 8 are required");
  }
  const PartialsPlan plan = plan_partials(m, n, k);
  slices = plan.slices;
  float* out = (float*)l.alloc((size_t)plan.slices * m * n * 4);
  if (l.dry()) return out;
  const KernelTable& t = need_mfma();
  if (plan.skinny) {
    check_mfma(t.mk_linear_skinny(x, w, out, m, n, k, plan.slices, l.stream()), "linear_partials");
  } else {
    check_mfma(t.mk_linear_tiled_partials(x, w, out, m, n, k, plan.slices, l.stream()),
               "linear_partials");
  }
  return out;
}

void project_into_stream(Launch& l, const void* x, int m, const void* w, int n, int k,
                         const void* bias, int bias_dtype, float* h, const float*& pending,
                         int& pending_count) {
  pending = nullptr;
  pending_count = 0;
  if (m == 0) return;
  if (!bias && wants_partials(l.dtype(), l.dtype(), m, n, k)) {
    pending = linear_partials(l, x, m, w, n, k, pending_count);
    return;
  }
  // in a dry walk h is null: nothing to allocate here, nothing to launch
  if (l.dry()) return;
  linear(l, x, m, w, n, k, bias, bias_dtype, h, kF32, true);
}

namespace {
int kv_heads(const QkvArgs& a) { return a.writes ? a.n_kv : 0; }
int qkv_width(const QkvArgs& a) { return (a.n_q + 2 * kv_heads(a)) * a.head_dim; }
}  // namespace

void rope_kv_write(Launch& l, void* qkv, int row_stride, int m, const QkvArgs& a,
                   const StepArrays& s) {
  if (l.dry() || m == 0) return;
  check_core(need_core().mk_rope_kv_write(
                 qkv, l.dtype(), row_stride, a.pos.cos, a.pos.sin, a.pos.table_positions,
                 s.positions, s.token_seq, s.table, s.table_stride, a.writes ? a.k_cache : nullptr,
                 a.writes ? a.v_cache : nullptr, a.writes ? a.page_size : 1, a.n_q, kv_heads(a),
                 a.head_dim, a.pos.rotary_dim, a.pos.interleaved ? 1 : 0, a.writes ? 1 : 0, m,
                 l.stream()), "rope_kv_write");
}

void* qkv_finish(Launch& l, const float* parts, int slices, int m, const QkvArgs& a,
                 const StepArrays& s, int out_dtype) {
  if (a.pos.interleaved && a.pos.rotary_dim) {
    throw KernelError("rope: partial sums are finished in the half-split layout only");
  }
  void* q = l.alloc((size_t)m * a.n_q * a.head_dim * element_size(out_dtype));
  if (l.dry() || m == 0) return q;
  check_core(need_core().mk_qkv_finish(
                 parts, slices, (long long)m * qkv_width(a), a.bias, a.bias ? a.bias_dtype : kF32, q,
                 out_dtype, a.pos.cos, a.pos.sin, a.pos.table_positions, s.positions, s.token_seq,
                 s.table, s.table_stride, a.writes ? a.k_cache : nullptr,
                 a.writes ? a.v_cache : nullptr, a.writes ? a.page_size : 1, a.n_q, kv_heads(a),
                 a.head_dim, a.pos.rotary_dim, a.writes ? 1 : 0, m, l.stream()), "qkv_finish");
  return q;
}

Queries qkv_project(Launch& l, const void* x, int m, int k, const QkvArgs& a, const StepArrays& s,
                    QkvForce force, const NormFold* fold) {
  const int d = a.head_dim;
  const int width = qkv_width(a);
  const int page_size = a.writes ? a.page_size : 1;
  const int bd = a.bias ? a.bias_dtype : kF32;
  const PositionDesc& p = a.pos;
  const bool half = !(p.interleaved && p.rotary_dim);
  QkvKind kind = force.kind >= 0
      ? (QkvKind)force.kind
      : choose_qkv(l.dtype(), l.dtype(), m, width, k, d, p.rotary_dim, page_size, half);
  if ((kind == QkvKind::SKINNY || kind == QkvKind::TILED) &&
      !qkv_fusable(l.dtype(), l.dtype(), m, k, d, p.rotary_dim, page_size, half)) {
    throw KernelError("qkv_project: these operands cannot take the fused kernel");
  }
  const bool folded = fold && kind == QkvKind::SKINNY && m <= 16 && folds_norm(l.dtype(), m, k);
  if (fold && !folded) {
    x = rmsnorm_fixed(l, fold->h64, k, fold->weight, fold->weight_dtype, fold->eps, nullptr, m);
  }
  if (kind == QkvKind::SKINNY || kind == QkvKind::TILED) {
    void* q = l.alloc((size_t)m * a.n_q * d * 2);
    if (!l.dry() && m > 0) {
      const KernelTable& t = need_mfma();
      void* kc = a.writes ? a.k_cache : nullptr;
      void* vc = a.writes ? a.v_cache : nullptr;
      const int code = folded
          ? t.mk_qkv_skinny_normed(fold->h64, fold->weight, fold->weight_dtype, fold->eps, a.w,
                                   a.bias, bd, q, p.cos, p.sin, p.table_positions, s.positions,
                                   s.token_seq, s.table, s.table_stride, kc, vc, page_size, a.n_q,
                                   kv_heads(a), d, p.rotary_dim > 0, m, k, l.stream())
          : kind == QkvKind::SKINNY
          ? t.mk_qkv_skinny(x, a.w, a.bias, bd, q, p.cos, p.sin, p.table_positions, s.positions,
                            s.token_seq, s.table, s.table_stride, kc, vc, page_size, a.n_q,
                            kv_heads(a), d, p.rotary_dim > 0, m, k, l.stream())
          : t.mk_qkv_tiled(x, a.w, a.bias, bd, q, p.cos, p.sin, p.table_positions, s.positions,
                           s.token_seq, s.table, s.table_stride, kc, vc, page_size, a.n_q,
                           kv_heads(a), d, p.rotary_dim > 0, m, k, force.tile_config, l.stream());
      check_mfma(code, "qkv_project");
    }
    return {q, a.n_q * d};
  }
  if (kind == QkvKind::PARTIALS_FINISH) {
    int slices = 0;
    const float* parts = linear_partials(l, x, m, a.w, width, k, slices);
    return {qkv_finish(l, parts, slices, m, a, s, l.dtype()), a.n_q * d};
  }
  void* qkv = linear(l, x, m, a.w, width, k, a.bias, bd, nullptr, l.dtype(), false);
  rope_kv_write(l, qkv, width, m, a, s);
  return {qkv, width};
}

Queries qkv_prepared(Launch& l, const void* x, int m, int k, const QkvArgs& a, const QkPrep& prep,
                     const StepArrays& s, const float** raw, int* raw_stride) {
  const int d = a.head_dim, dv = prep.value_dim > 0 ? prep.value_dim : d;
  const int heads_kv = kv_heads(a);
  const int maps = prep.maps > 1 ? prep.maps : 1;
  const int width = a.n_q * d + heads_kv * d + (prep.values_are_keys ? 0 : heads_kv * dv) +
                    prep.extra_cols;
  const float* qkv = (const float*)linear(l, x, m, a.w, width, k, a.bias,
                                          a.bias ? a.bias_dtype : kF32, nullptr, kF32, false);
  if (raw) *raw = qkv;
  if (raw_stride) *raw_stride = width;
  void* q = l.alloc((size_t)m * a.n_q * maps * d * l.elem());
  if (l.dry() || m == 0) return {q, a.n_q * maps * d};
  if (prep.v_mode != 0 && (!l.ctx->carried || l.ctx->carried_width < heads_kv * dv)) {
    throw KernelError("attention: values mixed across layers need room in the step for " +
                      std::to_string(heads_kv * dv) + " floats a token");
  }
  const PositionDesc& p = a.pos;
  check_core(need_core().mk_qk_prepare(
                 qkv, width, q, l.dtype(), prep.q_norm, prep.k_norm, prep.norm_dtype, prep.eps,
                 prep.temp_coef, prep.temp_every, p.cos, p.sin, p.table_positions, p.rotary_dim,
                 p.interleaved ? 1 : 0, s.positions, s.token_seq, s.table, s.table_stride,
                 a.writes ? a.k_cache : nullptr, a.writes ? a.v_cache : nullptr,
                 a.writes ? a.page_size : 1, a.n_q, heads_kv, d, dv, prep.values_are_keys,
                 a.writes ? 1 : 0, maps, prep.head_norm, l.ctx->carried, prep.v_mode,
                 prep.v_lambda, m, l.stream()), "qk_prepare");
  return {q, a.n_q * maps * d};
}

AttentionPlan plan_for(int dtype, const AttendArgs& a, const mk_step_view& step,
                       const AttendForce& force) {
  if (a.distance_slopes != nullptr) {
    if (force.kernel == 2) {
      throw KernelError("attention: the matrix-core kernels do not bias the score by distance");
    }
    return AttentionPlan();     // the float32-arithmetic kernel
  }
  if (a.v_dim() != a.head_dim) {
    if (force.kernel == 2) {
      throw KernelError("attention: the matrix-core kernels keep values as wide as keys");
    }
    return AttentionPlan();
  }
  if (a.window > 0 && a.keep_first > 0) {
    if (force.kernel == 2) {
      throw KernelError("attention: the matrix-core kernels keep no first keys past a window");
    }
    return AttentionPlan();
  }
  const std::vector<int> counts(step.counts, step.counts + step.num_seqs);
  if (!a.plain_scores()) {
    // a bounded score or sinks: the matrix-core kernels of 16 rows a wavefront
    if (force.tile_rows > 16 || force.staged >= 8) {
      throw KernelError("attention: a bounded score or sinks run in tiles of 16 rows a wavefront");
    }
    return plan_attention(dtype, a.head_dim, a.page_size, a.n_q, a.n_kv, a.window, counts,
                          step.max_q_len, step.max_kv_len, force.kernel, force.tile_rows,
                          force.staged, force.splits, force.split_blocks, true);
  }
  return plan_attention(dtype, a.head_dim, a.page_size, a.n_q, a.n_kv, a.window, counts,
                        step.max_q_len, step.max_kv_len, force.kernel, force.tile_rows, force.staged,
                        force.splits, force.split_blocks);
}

namespace {
const mk_tile_list& tiles_for(const mk_step_view& step, int group, int tile_rows) {
  for (int i = 0; i < step.num_tile_lists; ++i) {
    const mk_tile_list& t = step.tile_lists[i];
    if (t.group == group && t.tile_rows == tile_rows) return t;
  }
  throw KernelError("the step carries no tile list for groups of " + std::to_string(group) +
                    " heads in tiles of " + std::to_string(tile_rows) + " rows");
}
}  // namespace

void* attend(Launch& l, const Queries& q, const AttendArgs& a, const StepArrays& s,
             const mk_step_view& step, AttendForce force, void* out) {
  const int m = step.num_tokens, d = a.head_dim;
  if (!out) out = l.alloc((size_t)m * a.n_q * a.v_dim() * l.elem());
  const AttentionPlan plan = plan_for(l.dtype(), a, step, force);
  if (!plan.mfma) {
    if (!l.dry() && m > 0) {
      check_core(need_core().mk_attention_generic_kv(
                     q.q, q.stride, out, a.n_q * a.v_dim(), a.k_cache, a.v_cache, l.dtype(),
                     s.positions, s.token_seq, s.table, s.table_stride, a.page_size, a.n_q, a.n_kv,
                     d, a.v_dim(), a.scale, a.window, a.window > 0 ? a.keep_first : 0, a.score_cap,
                     a.distance_slopes, a.sinks, m, l.stream()), "attention");
    }
    return out;
  }
  float *part_o = nullptr, *part_ml = nullptr;
  if (plan.splits > 1) {
    const size_t rows = (size_t)plan.num_tiles * a.n_kv * plan.splits * plan.rows;
    part_o = (float*)l.alloc(rows * d * 4);
    part_ml = (float*)l.alloc(rows * 2 * 4);
  }
  if (l.dry() || m == 0) return out;
  const mk_tile_list& tiles = tiles_for(step, a.n_q / a.n_kv, plan.tile_rows);
  if (!a.plain_scores()) {
    check_mfma(need_mfma().mk_attention_mfma_scored(
                   q.q, q.stride, out, a.n_q * d, a.k_cache, a.v_cache,
                   plan.direct ? nullptr : tiles.seq, plan.direct ? nullptr : tiles.row0,
                   tiles.count, s.cu_q, s.kv_len, s.table, s.table_stride, a.page_size, a.n_q,
                   a.n_kv, d, a.scale, a.window, plan.staged, plan.splits, plan.split_blocks,
                   a.score_cap, a.sinks, part_o, part_ml, l.stream()), "attention");
    return out;
  }
  check_mfma(need_mfma().mk_attention_mfma(
                 q.q, q.stride, out, a.n_q * d, a.k_cache, a.v_cache,
                 plan.direct ? nullptr : tiles.seq, plan.direct ? nullptr : tiles.row0,
                 tiles.count, s.cu_q, s.kv_len, s.table, s.table_stride, a.page_size, a.n_q, a.n_kv,
                 d, a.scale, a.window, plan.rows, plan.staged, plan.splits, plan.split_blocks,
                 part_o, part_ml, l.stream()), "attention");
  return out;
}

namespace {
// The merge of the key splits folded into the output projection repeats the merge once per
// 64 (or 128) rows of w_o; it pays while that repetition stays small beside what the two
// kernels it replaces cost (0.5B shapes, 8 decoded tokens: 11.5 us a layer against 14.6 as
// three kernels; 32B shapes, 64 tokens: 247 against 204, 100 MB of parts repeated).
constexpr long long kFoldMaxRepeatedBytes = 48ll << 20;
constexpr int kFoldWideFromHidden = 2048;
}  // namespace

void attend_and_project(Launch& l, const Queries& q, const AttendArgs& a, const StepArrays& s,
                        const mk_step_view& step, const void* w_o, const void* b_o, int b_o_dtype,
                        int hidden, float* h, const float*& pending, int& pending_count,
                        AttendForce force, int fold, long long* h_fixed) {
  const int m = step.num_tokens, d = a.head_dim;
  pending = nullptr;
  pending_count = 0;
  const AttentionPlan plan = plan_for(l.dtype(), a, step, force);
  int heads_per_slice = 0, written = 0;
  bool wide = false;
  const bool fixed = h_fixed != nullptr || (l.dry() && l.ctx->stream_fixed);
  if (fold != 0 && plan.mfma && plan.splits > 1 && !plan.staged && plan.rows == 16 &&
      step.max_q_len == 1 && plan.num_tiles == m && !b_o && a.n_q / a.n_kv <= 16) {
    const KernelTable& t = need_mfma();
    written = t.mk_attention_mfma_parts_written(plan.rows, plan.splits, d);
    heads_per_slice = t.mk_attention_out_heads_per_slice(a.n_q, a.n_kv, d, m, hidden, fixed ? 1 : 0);
    wide = hidden >= kFoldWideFromHidden;
    if (heads_per_slice &&
        (written < 2 || written > t.mk_attention_out_max_parts(m, heads_per_slice))) {
      heads_per_slice = 0;
    }
    if (heads_per_slice && fold < 0) {
      const long long part_bytes = (long long)m * a.n_q * written * (d * 4 + 8);
      const long long repeats = (hidden + (wide ? 127 : 63)) / (wide ? 128 : 64);
      if (part_bytes * repeats > kFoldMaxRepeatedBytes) heads_per_slice = 0;
    }
  }
  if (!heads_per_slice) {
    if (fold > 0) throw KernelError("attention: these sizes do not take the folded merge");
    const void* attended = attend(l, q, a, s, step, force);
    if (fixed) {
      project_into_fixed(l, attended, m, w_o, hidden, a.n_q * a.v_dim(), b_o, b_o_dtype, h_fixed);
    } else {
      project_into_stream(l, attended, m, w_o, hidden, a.n_q * a.v_dim(), b_o, b_o_dtype, h,
                          pending, pending_count);
    }
    return;
  }
  const size_t rows = (size_t)plan.num_tiles * a.n_kv * plan.splits * plan.rows;
  float* part_o = (float*)l.alloc(rows * d * 4);
  float* part_ml = (float*)l.alloc(rows * 2 * 4);
  const int slices = a.n_q / heads_per_slice;
  float* out = nullptr;
  if (!fixed) {
    out = (float*)l.alloc((size_t)slices * m * hidden * 4);
    pending = out;
    pending_count = slices;
  }
  if (l.dry() || m == 0) return;
  const KernelTable& t = need_mfma();
  const mk_tile_list& tiles = tiles_for(step, a.n_q / a.n_kv, plan.tile_rows);
  if (!a.plain_scores()) {
    check_mfma(t.mk_attention_mfma_parts_scored(
                   q.q, q.stride, a.k_cache, a.v_cache, plan.direct ? nullptr : tiles.seq,
                   plan.direct ? nullptr : tiles.row0, tiles.count, s.cu_q, s.kv_len, s.table,
                   s.table_stride, a.page_size, a.n_q, a.n_kv, d, a.scale, a.window, plan.splits,
                   plan.split_blocks, a.score_cap, a.sinks, part_o, part_ml, l.stream()),
               "attention");
  } else {
  check_mfma(t.mk_attention_mfma_parts(q.q, q.stride, a.k_cache, a.v_cache,
                                       plan.direct ? nullptr : tiles.seq,
                                       plan.direct ? nullptr : tiles.row0, tiles.count, s.cu_q, s.kv_len, s.table, s.table_stride,
                                       a.page_size, a.n_q, a.n_kv, d, a.scale, a.window, plan.rows,
                                       plan.splits, plan.split_blocks, part_o, part_ml, l.stream()),
             "attention");
  }
  check_mfma(t.mk_attention_out(part_o, part_ml, written, w_o, out, h_fixed, m, hidden, a.n_q, a.n_kv, d,
                                heads_per_slice, wide ? 1 : 0, l.stream()), "attention_out");
}

void* attend_maps(Launch& l, const Queries& q, const AttendArgs& a, const StepArrays& s,
                  const mk_step_view& step, const float* gate, int gate_stride, float lambda,
                  float eps, float out_scale) {
  const int heads = a.n_q / 2, map_dim = a.head_dim / 2;
  if (l.dtype() != kBF16 || !kernels().has_mfma() || !a.plain_scores() || a.distance_slopes ||
      a.n_q % 2 || a.head_dim % 2 || heads % a.n_kv ||
      !kernels().mk_attention_maps_supported(map_dim, a.v_dim(), a.page_size)) {
    return nullptr;
  }
  const int m = step.num_tokens;
  void* out = l.alloc((size_t)m * heads * a.v_dim() * l.elem());
  // a step of single tokens: the key blocks of a (sequence, head) go to as many workgroups as
  // leave each of their four wavefronts a block or two, while the chip has room for them
  int splits = 1;
  if (step.max_q_len == 1) {
    const int reach = a.window > 0 ? std::min(step.max_kv_len, a.window + a.keep_first + 32)
                                   : step.max_kv_len;
    const int blocks = (reach + 31) / 32;
    const int room = std::max(1, 2048 / std::max(1, step.num_seqs * heads));
    splits = std::max(1, std::min({8, (blocks + 7) / 8, room}));
  }
  float* parts = nullptr;
  if (splits > 1) {
    parts = (float*)l.alloc((size_t)kernels().mk_attention_maps_parts(step.num_seqs, heads,
                                                                      a.v_dim(), splits) * 4);
  }
  if (l.dry() || m == 0) return out;
  check_mfma(kernels().mk_attention_maps(
                 q.q, q.stride, out, a.k_cache, a.v_cache, gate, gate_stride, s.positions, s.cu_q,
                 s.table, s.table_stride, a.page_size, heads, a.n_kv, map_dim, a.v_dim(), a.scale,
                 a.window, a.window > 0 ? a.keep_first : 0, lambda, eps, out_scale, step.num_seqs,
                 step.max_q_len, splits, parts, l.stream()), "attention");
  return out;
}

void* gate_mul(Launch& l, const void* a, int m, int width, const float* gate, int gate_stride) {
  void* out = l.alloc((size_t)m * width * l.elem());
  if (l.dry() || m == 0) return out;
  check_core(need_core().mk_gate_mul(a, l.dtype(), gate, gate_stride, out, m, width, l.stream()),
             "gate_mul");
  return out;
}

void* stream_cast(Launch& l, float* h, int tokens, int hidden, const float* pending,
                  int pending_count) {
  void* out = l.alloc((size_t)tokens * hidden * l.elem());
  if (l.dry() || tokens == 0) return out;
  const long long n = (long long)tokens * hidden;
  check_core(need_core().mk_stream_cast(h, pending, pending_count, n, out, l.dtype(), n,
                                        l.stream()), "stream_cast");
  return out;
}

void* diff_heads(Launch& l, const void* a, int m, int heads, int dv, const float* gate,
                 int gate_stride, float lambda, float eps, float out_scale) {
  void* out = l.alloc((size_t)m * heads * dv * l.elem());
  if (l.dry() || m == 0) return out;
  check_core(need_core().mk_diff_heads(a, out, l.dtype(), gate, gate_stride, lambda, eps, out_scale,
                                       m, heads, dv, l.stream()), "diff_heads");
  return out;
}

void norm_scale_add(Launch& l, float* h, const float* y, const float* partials, int count,
                    const void* weight, int weight_dtype, const float* scale, float eps,
                    int tokens, int hidden, void* x_out) {
  if (l.dry() || tokens == 0) return;
  check_core(need_core().mk_norm_scale_add(h, y, partials, count, (long long)tokens * hidden,
                                           weight, weight_dtype, scale, eps, tokens, hidden,
                                           x_out, l.dtype(), l.stream()), "norm_scale_add");
}

void retention(Launch& l, const void* x, int m, int hidden, const RetentionArgs& a,
               const mk_step_view& step, float* h, const float*& pending, int& pending_count) {
  pending = nullptr;
  pending_count = 0;
  const int width = a.in_width(), qk = a.heads * a.dim, inner = a.heads * a.vdim;
  const float* proj = (const float*)linear(l, x, m, a.w_in, width, hidden, nullptr, kF32, nullptr,
                                           kF32, false);
  float* y = (float*)l.alloc((size_t)m * inner * 4);
  void* normed = l.alloc((size_t)m * inner * l.elem());
  // a step with a sequence longer than a chunk runs the recurrence in chunks side by side
  const KernelTable& core = need_core();
  const int chunk = core.mk_retention_chunk_tokens();
  int total_chunks = 0, longest = 0;
  for (int i = 0; i < step.num_seqs; ++i) {
    total_chunks += (step.counts[i] + chunk - 1) / chunk;
    longest = std::max(longest, step.counts[i]);
  }
  if (longest <= chunk) total_chunks = 0;
  float* scan_ws = nullptr;
  if (total_chunks) {
    const long long floats = core.mk_retention_scan_workspace(total_chunks, a.heads, a.dim, a.vdim);
    if (floats < 0) throw KernelError("retention: the recurrence does not run these sizes");
    scan_ws = (float*)l.alloc((size_t)floats * 4);
  }
  if (!l.dry() && m > 0) {
    const KernelTable& t = need_core();
    if (!a.state) throw KernelError("retention: no state tensor");
    check_core(t.mk_retention_scan(proj, width, 0, qk, 2 * qk, a.decay, a.k_scale, a.pos.cos,
                                   a.pos.sin, a.pos.table_positions, a.pos.rotary_dim,
                                   step.positions, step.cu_q, step.state_slots, a.state,
                                   a.slot_floats, a.heads, a.dim, a.vdim, y, m, step.num_seqs,
                                   total_chunks, scan_ws, l.stream()), "retention_scan");
    check_core(t.mk_head_norm_gate(y, normed, l.dtype(), proj + 2 * qk + inner, width, a.eps, m,
                                   a.heads, a.vdim, nullptr, MK_GATE_SILU, l.stream()),
               "head_norm_gate");
  }
  project_into_stream(l, normed, m, a.w_out, hidden, inner, nullptr, kF32, h, pending,
                      pending_count);
}

void mlstm(Launch& l, const void* x, int m, int hidden, const MlstmArgs& a,
           const mk_step_view& step, float* h, const float*& pending, int& pending_count) {
  pending = nullptr;
  pending_count = 0;
  const int width = a.in_width(), qk = a.heads * a.dim, inner = a.heads * a.vdim;
  const float* proj = (const float*)linear(l, x, m, a.w_in, width, hidden, a.b_in, a.b_in_dtype,
                                           nullptr, kF32, false);
  float* y = (float*)l.alloc((size_t)m * inner * 4);
  void* normed = l.alloc((size_t)m * inner * l.elem());
  // a step with a sequence longer than a chunk runs the recurrence in chunks side by side
  const KernelTable& core = need_core();
  const int chunk = core.mk_mlstm_chunk_tokens();
  int total_chunks = 0, longest = 0;
  for (int i = 0; i < step.num_seqs; ++i) {
    total_chunks += (step.counts[i] + chunk - 1) / chunk;
    longest = std::max(longest, step.counts[i]);
  }
  if (longest <= chunk) total_chunks = 0;
  float* scan_ws = nullptr;
  if (total_chunks) {
    const long long floats = core.mk_mlstm_scan_workspace(total_chunks, m, a.heads, a.dim, a.vdim);
    if (floats < 0) throw KernelError("mlstm: the recurrence does not run these sizes");
    scan_ws = (float*)l.alloc((size_t)floats * 4);
  }
  if (!l.dry() && m > 0) {
    const KernelTable& t = need_core();
    if (!a.state) throw KernelError("mlstm: no state tensor");
    const int gates = 2 * qk + 2 * inner;
    check_core(t.mk_mlstm_scan(proj, width, 0, qk, 2 * qk, gates, gates + a.heads, a.q_scale,
                               a.gate_cap, step.cu_q, step.state_slots, a.state, a.slot_floats,
                               a.heads, a.dim, a.vdim, y, m, step.num_seqs, total_chunks, scan_ws,
                               l.stream()),
               "mlstm_scan");
    check_core(t.mk_head_norm_gate(y, normed, l.dtype(), proj + 2 * qk + inner, width, a.eps, m,
                                   a.heads, a.vdim, a.norm, MK_GATE_SIGMOID, l.stream()),
               "head_norm_gate");
  }
  project_into_stream(l, normed, m, a.w_out, hidden, inner, nullptr, kF32, h, pending,
                      pending_count);
}

void* gated(Launch& l, const void* x, int m, int k, const void* w_gate_up, int inter,
            int tile_config, const NormFold* fold, const GateAct& act) {
  const bool fuses = fuses_gating(l.dtype(), l.dtype(), m, k, 2 * inter);
  const bool folded = fold && fuses && act.silu() && tile_config == -2 && m <= 16 &&
                      folds_norm(l.dtype(), m, k);
  if (fold && !folded) {
    x = rmsnorm_fixed(l, fold->h64, k, fold->weight, fold->weight_dtype, fold->eps, nullptr, m);
  }
  if (fuses) {
    void* out = l.alloc((size_t)m * inter * 2);
    if (l.dry() || m == 0) return out;
    const KernelTable& t = need_mfma();
    if (folded) {
      check_mfma(t.mk_gated_skinny_normed(fold->h64, fold->weight, fold->weight_dtype, fold->eps,
                                          w_gate_up, out, m, inter, k, l.stream()),
                 "gated_projection");
      return out;
    }
    const bool skinny = gated_is_skinny(m) && tile_config == -2;
    check_mfma(skinny ? t.mk_gated_skinny_act(x, w_gate_up, out, m, inter, k, act.kind, act.limit,
                                              act.alpha, act.beta, l.stream())
                      : t.mk_gated_tiled_act(x, w_gate_up, out, m, inter, k,
                                             tile_config == -2 ? -1 : tile_config, act.kind,
                                             act.limit, act.alpha, act.beta, l.stream()),
               "gated_projection");
    return out;
  }
  if (tile_config != -2) throw KernelError("gated_projection: operands not eligible");
  void* gate_up = linear(l, x, m, w_gate_up, 2 * inter, k, nullptr, kF32, nullptr, l.dtype(), false);
  return act.silu() ? silu_mul(l, gate_up, m, inter) : gate_activation(l, gate_up, m, inter, act);
}

void unary_mlp(Launch& l, const void* x, int m, int hidden, const void* w_up, const void* w_down,
               int inter, int act, float* h, const float*& pending, int& pending_count) {
  pending = nullptr;
  pending_count = 0;
  // many rows on the matrix cores: the activation in the product's epilogue
  if (mfma_eligible(l.dtype(), l.dtype(), m, hidden) && kernels().has_mfma() && !gated_is_skinny(m)) {
    void* acted = l.alloc((size_t)m * inter * l.elem());
    if (!l.dry()) {
      check_mfma(need_mfma().mk_linear_tiled_act(x, w_up, acted, m, inter, hidden, act, -1,
                                                 l.stream()), "linear_act");
    }
    project_into_stream(l, acted, m, w_down, hidden, inter, nullptr, kF32, h, pending,
                        pending_count);
    return;
  }
  // the product in float32, so that the activation's result is rounded once
  void* up = linear(l, x, m, w_up, inter, hidden, nullptr, kF32, nullptr, kF32, false);
  void* acted = l.alloc((size_t)m * inter * l.elem());
  if (!l.dry() && m > 0) {
    check_core(need_core().mk_unary_act(up, kF32, acted, l.dtype(), (long long)m * inter, act,
                                        l.stream()), "unary_act");
  }
  project_into_stream(l, acted, m, w_down, hidden, inter, nullptr, kF32, h, pending,
                      pending_count);
}

void state_space(Launch& l, const void* x, int m, int hidden, const StateSpaceArgs& a,
                 const mk_step_view& step, float* h, const float*& pending, int& pending_count) {
  pending = nullptr;
  pending_count = 0;
  const int inner = a.inner(), channels = a.channels(), width = a.in_width();
  const float* proj = (const float*)linear(l, x, m, a.w_in, width, hidden, nullptr, kF32, nullptr,
                                           kF32, false);
  float* xbc = (float*)l.alloc((size_t)m * channels * 4);
  float* y = (float*)l.alloc((size_t)m * inner * 4);
  void* normed = l.alloc((size_t)m * inner * l.elem());
  // a step with a sequence longer than a chunk runs the recurrence in chunks side by side
  const KernelTable& core = need_core();
  const int chunk = core.mk_ssm_chunk_tokens();
  int total_chunks = 0, longest = 0;
  for (int i = 0; i < step.num_seqs; ++i) {
    total_chunks += (step.counts[i] + chunk - 1) / chunk;
    longest = std::max(longest, step.counts[i]);
  }
  if (longest <= chunk) total_chunks = 0;
  float* scan_ws = nullptr;
  if (total_chunks) {
    const long long floats = core.mk_ssm_scan_workspace(total_chunks, a.heads, a.vdim, a.state_size);
    if (floats < 0) throw KernelError("state_space: the recurrence does not run these sizes");
    scan_ws = (float*)l.alloc((size_t)floats * 4);
  }
  if (!l.dry() && m > 0) {
    const KernelTable& t = need_core();
    if (!a.state) throw KernelError("state_space: no state tensor");
    check_core(t.mk_causal_conv_silu(proj, width, inner, channels, a.taps, a.conv_w, a.conv_b,
                                     a.vector_dtype, a.state, a.slot_floats, step.state_slots,
                                     step.token_seq, step.cu_q, xbc, m, step.num_seqs, l.stream()),
               "causal_conv");
    check_core(t.mk_ssm_scan(xbc, channels, proj, width, 0, inner + channels, a.dt_bias, a.a_log,
                             a.d_skip, a.vector_dtype, a.state + a.carried_floats(), a.slot_floats,
                             step.state_slots, step.cu_q, a.heads, a.vdim, a.state_size, a.groups,
                             y, m, step.num_seqs, total_chunks, scan_ws, l.stream()), "ssm_scan");
    check_core(t.mk_group_rmsnorm(y, normed, l.dtype(), a.norm, a.vector_dtype, a.eps, m, inner,
                                  a.norm_groups, l.stream()), "group_rmsnorm");
  }
  project_into_stream(l, normed, m, a.w_out, hidden, inner, nullptr, kF32, h, pending,
                      pending_count);
}

void normed_sum(Launch& l, float* h, const float* ya, const float* pa, int na, const void* wa,
                const float* yb, const float* pb, int nb, const void* wb, int weight_dtype,
                float eps, float mult, int tokens, int hidden) {
  if (l.dry() || tokens == 0) return;
  check_core(need_core().mk_normed_sum(h, ya, pa, na, wa, yb, pb, nb, wb, weight_dtype, eps, mult,
                                       (long long)tokens * hidden, tokens, hidden, l.stream()),
             "normed_sum");
}

void stream_mix(Launch& l, float* h, const float* kept, int m, int hidden, const void* w) {
  void* both = l.alloc((size_t)m * 2 * hidden * l.elem());
  if (l.dry() || m == 0) return;
  check_core(need_core().mk_concat_cast(h, kept, both, l.dtype(), m, hidden, l.stream()),
             "concat_cast");
  linear(l, both, m, w, hidden, 2 * hidden, nullptr, kF32, h, kF32, false);
}

void copy_stream(Launch& l, float* dst, const float* src, long long n) {
  if (l.dry() || n == 0) return;
  check_core(need_core().mk_copy_f32(dst, src, n, l.stream()), "copy");
}

void* linear_per_head(Launch& l, const void* x, int m, int heads, int lda, int x_head,
                      const void* w, int n, int k, void* out, int ldo, int o_head) {
  if (!out) {
    out = l.alloc((size_t)m * heads * n * l.elem());
    ldo = heads * n;
    o_head = n;
  }
  if (l.dry() || m == 0) return out;
  // the matrix-core kernel wants 16-byte pieces of rows: K, the row pitch and the heads' offsets
  // multiples of 8 elements
  if (l.dtype() == kBF16 && kernels().has_mfma() && k % 8 == 0 && lda % 8 == 0 && x_head % 8 == 0 &&
      ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0) {
    check_mfma(need_mfma().mk_linear_batched_mfma(x, w, out, m, n, k, lda, ldo, heads, x_head,
                                                  (long long)n * k, o_head, l.stream()),
               "linear_per_head");
    return out;
  }
  check_core(need_core().mk_linear_batched_generic(x, w, l.dtype(), out, l.dtype(), m, n, k, lda,
                                                   ldo, heads, x_head, (long long)n * k, o_head,
                                                   l.stream()), "linear_per_head");
  return out;
}

Queries latent_queries(Launch& l, const void* x, int m, int hidden, const LatentArgs& a,
                       const StepArrays& s, const float** raw, int* raw_stride) {
  const int down_width = a.q_rank + (a.writes ? a.kv_rank + a.rot : 0) + a.gate_cols;
  const int per_head = a.dim + a.rot, width = a.key_width();
  // the latents in float32: the norms read them
  const float* down = (const float*)linear(l, x, m, a.w_down, down_width, hidden, nullptr, kF32,
                                           nullptr, kF32, false);
  if (raw) *raw = down;
  if (raw_stride) *raw_stride = down_width;
  void* q_latent = a.q_rank > 0 ? l.alloc((size_t)m * a.q_rank * l.elem()) : nullptr;
  if (!l.dry() && m > 0) {
    check_core(need_core().mk_latent_prepare(
                   down, down_width, a.q_rank, a.kv_rank, a.rot, a.q_norm, a.kv_norm, a.norm_dtype,
                   a.eps, a.pos.cos, a.pos.sin, a.pos.table_positions, a.pos.rotary_dim,
                   a.pos.interleaved, s.positions, s.token_seq, s.table, s.table_stride, q_latent,
                   a.writes ? a.k_cache : nullptr, a.writes ? a.v_cache : nullptr, a.key_width(),
                   a.value_width(), l.dtype(), a.writes ? a.page_size : 1, a.writes ? 1 : 0, m,
                   l.stream()), "latent_prepare");
  }
  const void* q = a.q_rank > 0
      ? linear(l, q_latent, m, a.w_uq, a.heads * per_head, a.q_rank, nullptr, kF32, nullptr,
               l.dtype(), false)
      : linear(l, x, m, a.w_uq, a.heads * per_head, hidden, nullptr, kF32, nullptr, l.dtype(), false);
  void* out = l.alloc((size_t)m * a.heads * width * l.elem());
  linear_per_head(l, q, m, a.heads, a.heads * per_head, per_head, a.w_uk_t, a.kv_rank, a.dim, out,
                  a.heads * width, width);
  if (!l.dry() && m > 0) {
    check_core(need_core().mk_latent_query_tail(
                   q, l.dtype(), a.heads, a.dim, a.rot, a.pos.cos, a.pos.sin, a.pos.table_positions,
                   a.pos.rotary_dim, a.pos.interleaved, s.positions, out, width, a.kv_rank, m,
                   l.stream()), "latent_query_tail");
  }
  return {out, a.heads * width};
}

namespace {
// Decoding with few tiles: the keys are cut into parts until about this many wavefronts run,
// a part being at least this many blocks of 32 keys.
constexpr int kLatentWaves = 1024;
constexpr int kLatentMinBlocks = 4;
}  // namespace

LatentPlan latent_plan(int dtype, const LatentArgs& a, const mk_step_view& step) {
  LatentPlan plan;
  if (dtype != kBF16 || !kernels().has_mfma()) return plan;
  const KernelTable& t = need_mfma();
  if (!t.mk_attention_latent_supported(a.key_width(), a.value_width(), a.page_size)) return plan;
  plan.mfma = true;
  const std::vector<int> counts(step.counts, step.counts + step.num_seqs);
  plan.num_tiles = count_tiles(counts, a.heads, 16);
  // (inside a window a tile walks the window's blocks and one more, whatever the length)
  const int reach = a.window > 0 ? std::min(step.max_kv_len, a.window + 31) : step.max_kv_len;
  const int blocks = (reach + 31) / 32;
  int parts = 1;
  if (plan.num_tiles > 0 && plan.num_tiles < kLatentWaves) {
    parts = std::min(kLatentWaves / plan.num_tiles, std::max(1, blocks / kLatentMinBlocks));
  }
  plan.parts = std::max(1, std::min(parts, t.mk_attention_latent_max_parts()));
  // Keys unsplit and some sequence with a tile of 64 rows to fill: prompt portions, whose
  // rows share their keys through LDS.
  if (plan.parts == 1 && (long long)step.max_q_len * a.heads >= 64) {
    plan.tile_rows = 64;
    plan.num_tiles = count_tiles(counts, a.heads, 64);
  }
  return plan;
}

void* latent_attend(Launch& l, const Queries& q, const LatentArgs& a, float scale,
                    const StepArrays& s, const mk_step_view& step) {
  const int m = step.num_tokens, dk = a.key_width(), dv = a.value_width();
  void* out = l.alloc((size_t)m * a.heads * dv * l.elem());
  const LatentPlan plan = latent_plan(l.dtype(), a, step);
  if (!plan.mfma) {
    if (!l.dry() && m > 0) {
      check_core(need_core().mk_attention_generic_kv(
                     q.q, q.stride, out, a.heads * dv, a.k_cache, a.v_cache, l.dtype(), s.positions,
                     s.token_seq, s.table, s.table_stride, a.page_size, a.heads, 1, dk, dv, scale,
                     a.window, 0, 0.f, nullptr, a.sinks, m, l.stream()), "latent_attention");
    }
    return out;
  }
  float *part_o = nullptr, *part_ml = nullptr;
  if (plan.parts > 1) {
    part_o = (float*)l.alloc((size_t)plan.num_tiles * plan.parts * dv * 16 * 4);
    part_ml = (float*)l.alloc((size_t)plan.num_tiles * plan.parts * 32 * 4);
  }
  if (l.dry() || m == 0) return out;
  const mk_tile_list& tiles = tiles_for(step, a.heads, plan.tile_rows);
  check_mfma(need_mfma().mk_attention_latent(q.q, out, a.k_cache, a.v_cache, tiles.seq, tiles.row0,
                                             tiles.count, plan.tile_rows, s.cu_q, s.kv_len, s.table,
                                             s.table_stride,
                                             a.page_size, a.heads, dk, dv, scale, plan.parts, part_o,
                                             part_ml, a.window, a.sinks, l.stream()),
             "latent_attention");
  return out;
}

void* latent_values(Launch& l, const void* summed, int m, const LatentArgs& a) {
  return linear_per_head(l, summed, m, a.heads, a.heads * a.value_width(), a.value_width(), a.w_uv,
                         a.vdim, a.kv_rank, nullptr, 0, 0);
}

namespace {
// The shared expert beside the routed ones: a gated feed-forward of every token, its
// activations times the token's gate, its down-projection into the same sum.
void shared_expert(Launch& l, const void* x, int m, int hidden, const ExpertArgs& a, float* y,
                   const float*& pending, int& pending_count) {
  if (!a.shared_gate_up) return;
  void* act = gated(l, x, m, hidden, a.shared_gate_up, a.shared_ff, -2, nullptr, a.shared_act);
  if (a.shared_gate && !l.dry() && m > 0) {
    check_core(need_core().mk_row_gate(act, x, a.shared_gate, l.dtype(), m, a.shared_ff, hidden,
                                       l.stream()), "row_gate");
  }
  project_into_stream(l, act, m, a.shared_down, hidden, a.shared_ff, nullptr, kF32, y, pending,
                      pending_count);
}
}  // namespace

void routed_experts(Launch& l, const void* x, int m, int hidden, const ExpertArgs& a, float* y,
                    const float*& pending, int& pending_count) {
  pending = nullptr;
  pending_count = 0;
  shared_expert(l, x, m, hidden, a, y, pending, pending_count);
  const float* logits = (const float*)linear(l, x, m, a.w_router, a.experts, hidden, nullptr, kF32,
                                             nullptr, kF32, false);
  int* ids = (int*)l.alloc((size_t)m * a.top * 4);
  float* weights = (float*)l.alloc((size_t)m * a.top * 4);
  void* act = l.alloc((size_t)m * a.top * a.ff * l.elem());
  // On the matrix cores the (token, choice) pairs are grouped by expert, so that an expert's
  // matrices are multiplied with all its tokens at once; every pair's down-projection lands in
  // a row of its own and the rows of a token are added in the order of its choices.
  const bool grouped = l.dtype() == kBF16 && kernels().has_mfma() && hidden % 8 == 0 &&
                       a.ff % 8 == 0 && a.experts <= 1024;
  int *rows = nullptr, *offsets = nullptr;
  float* pair_out = nullptr;
  if (grouped) {
    rows = (int*)l.alloc((size_t)m * a.top * 4);
    offsets = (int*)l.alloc((size_t)(a.experts + 1) * 4);
    pair_out = (float*)l.alloc((size_t)m * a.top * hidden * 4);
  }
  if (l.dry() || m == 0) return;
  const KernelTable& t = need_core();
  check_core(t.mk_route_topk(logits, a.experts, a.top, a.scale, a.renormalize, ids, weights, m,
                             l.stream()), "route");
  if (grouped) {
    const KernelTable& f = need_mfma();
    check_core(t.mk_route_group(ids, m * a.top, a.experts, rows, offsets, l.stream()), "route_group");
    check_mfma(f.mk_expert_gated_mfma(x, a.w_gate_up, act, rows, offsets, a.experts, m, a.top, a.ff,
                                      hidden, a.act.kind, a.act.limit, a.act.alpha, a.act.beta,
                                      l.stream()), "expert_gated");
    check_mfma(f.mk_expert_down_mfma(act, a.w_down, pair_out, rows, offsets, weights, a.experts, m,
                                     a.ff, hidden, l.stream()), "expert_down");
    check_core(t.mk_expert_combine(pair_out, y, m, a.top, hidden, l.stream()), "expert_combine");
    return;
  }
  check_core(t.mk_expert_gated(x, a.w_gate_up, l.dtype(), ids, act, m, a.top, a.ff, hidden,
                               a.act.kind, a.act.limit, a.act.alpha, a.act.beta, l.stream()),
             "expert_gated");
  check_core(t.mk_expert_down(act, a.w_down, l.dtype(), ids, weights, y, m, a.top, a.ff, hidden,
                              l.stream()), "expert_down");
}

}  // namespace mercury
