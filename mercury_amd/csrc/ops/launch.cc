#include "launch.h"

#include <string>

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
              void* out) {
  if (!out) out = l.alloc((size_t)out_rows * hidden * l.elem());
  if (l.dry() || out_rows == 0) return out;
  check_core(need_core().mk_rmsnorm(h, pending, pending_count, (long long)tokens * hidden, weight,
                                    weight_dtype, eps, rows, out, l.dtype(), out_rows, hidden,
                                    l.stream()), "rmsnorm");
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

AttentionPlan plan_for(int dtype, const AttendArgs& a, const mk_step_view& step,
                       const AttendForce& force) {
  if (!a.plain_scores()) {
    if (force.kernel == 2) {
      throw KernelError("attention: the matrix-core kernels neither cap nor bias the score");
    }
    return AttentionPlan();     // the float32-arithmetic kernel
  }
  const std::vector<int> counts(step.counts, step.counts + step.num_seqs);
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
  if (!out) out = l.alloc((size_t)m * a.n_q * d * l.elem());
  const AttentionPlan plan = plan_for(l.dtype(), a, step, force);
  if (!plan.mfma) {
    if (!l.dry() && m > 0) {
      check_core(need_core().mk_attention_generic(
                     q.q, q.stride, out, a.n_q * d, a.k_cache, a.v_cache, l.dtype(), s.positions,
                     s.token_seq, s.table, s.table_stride, a.page_size, a.n_q, a.n_kv, d, a.scale,
                     a.window, a.score_cap, a.distance_slopes, m, l.stream()), "attention");
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
      project_into_fixed(l, attended, m, w_o, hidden, a.n_q * d, b_o, b_o_dtype, h_fixed);
    } else {
      project_into_stream(l, attended, m, w_o, hidden, a.n_q * d, b_o, b_o_dtype, h, pending,
                          pending_count);
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
  check_mfma(t.mk_attention_mfma_parts(q.q, q.stride, a.k_cache, a.v_cache,
                                       plan.direct ? nullptr : tiles.seq,
                                       plan.direct ? nullptr : tiles.row0, tiles.count, s.cu_q, s.kv_len, s.table, s.table_stride,
                                       a.page_size, a.n_q, a.n_kv, d, a.scale, a.window, plan.rows,
                                       plan.splits, plan.split_blocks, part_o, part_ml, l.stream()),
             "attention");
  check_mfma(t.mk_attention_out(part_o, part_ml, written, w_o, out, h_fixed, m, hidden, a.n_q, a.n_kv, d,
                                heads_per_slice, wide ? 1 : 0, l.stream()), "attention_out");
}

void* gated(Launch& l, const void* x, int m, int k, const void* w_gate_up, int inter,
            int tile_config, const NormFold* fold) {
  const bool fuses = fuses_gating(l.dtype(), l.dtype(), m, k, 2 * inter);
  const bool folded = fold && fuses && tile_config == -2 && m <= 16 && folds_norm(l.dtype(), m, k);
  if (fold && !folded) {
    x = rmsnorm_fixed(l, fold->h64, k, fold->weight, fold->weight_dtype, fold->eps, nullptr, m);
  }
  if (fuses) {
    void* act = l.alloc((size_t)m * inter * 2);
    if (l.dry() || m == 0) return act;
    const KernelTable& t = need_mfma();
    if (folded) {
      check_mfma(t.mk_gated_skinny_normed(fold->h64, fold->weight, fold->weight_dtype, fold->eps,
                                          w_gate_up, act, m, inter, k, l.stream()),
                 "gated_projection");
      return act;
    }
    const bool skinny = gated_is_skinny(m) && tile_config == -2;
    check_mfma(skinny ? t.mk_gated_skinny(x, w_gate_up, act, m, inter, k, l.stream())
                      : t.mk_gated_tiled(x, w_gate_up, act, m, inter, k,
                                         tile_config == -2 ? -1 : tile_config, l.stream()),
               "gated_projection");
    return act;
  }
  if (tile_config != -2) throw KernelError("gated_projection: operands not eligible");
  void* gate_up = linear(l, x, m, w_gate_up, 2 * inter, k, nullptr, kF32, nullptr, l.dtype(), false);
  return silu_mul(l, gate_up, m, inter);
}

}  // namespace mercury
