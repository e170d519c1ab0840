#include "program.h"

#include <algorithm>

#include "kernels.h"

namespace mercury {

const StepView::Tiles& StepView::tiles_for(int group, int tile_rows) const {
  for (const Tiles& t : tiles) {
    if (t.group == group && t.tile_rows == tile_rows) return t;
  }
  throw KernelError("the step carries no attention tile list for groups of " +
                    std::to_string(group) + " heads in tiles of " + std::to_string(tile_rows) + " rows");
}

void* Arena::alloc(size_t bytes) {
  const size_t aligned = (bytes + 255) & ~(size_t)255;
  if (!dry_ && used_ + aligned > size_) {
    throw KernelError("the step's workspace is too small: an operation needs " +
                      std::to_string(used_ + aligned) + " bytes of an arena of " + std::to_string(size_));
  }
  void* p = dry_ ? nullptr : base_ + used_;
  used_ += aligned;
  peak_ = std::max(peak_, used_);
  return p;
}

namespace {

struct Ctx {
  const StepView& step;
  Arena* arena;
  hipStream_t stream;
  bool dry;
  int dtype, hidden;
  int elem() const { return element_size(dtype); }
};

// y = x W^T (+ bias) into a fresh [m, n] tensor of out_dtype.
void* linear_out(Ctx& c, const void* x, int m, const void* w, int n, int k, const void* bias,
                 int bias_dtype, int out_dtype, void* out = nullptr) {
  if (!out) out = c.arena->alloc((size_t)m * n * element_size(out_dtype));
  if (c.dry || m == 0) return out;
  const int bd = bias ? bias_dtype : kF32;
  switch (choose_linear(c.dtype, m, n, k, bias != nullptr, false, out_dtype)) {
    case LinearKind::GENERIC:
      check_core(need_core().mk_linear_generic(x, w, c.dtype, bias, bd, out, out_dtype, 0, m, n, k, k,
                                               n, c.stream), "linear");
      break;
    case LinearKind::SKINNY:
      check_mfma(need_mfma().mk_linear_skinny(x, w, (float*)out, m, n, k, 1, c.stream), "linear");
      break;
    default:
      check_mfma(need_mfma().mk_linear_tiled(x, w, bias, bd, out, out_dtype, 0, m, n, k, n, -1,
                                             c.stream), "linear");
  }
  return out;
}

// Float32 partial sums [slices, m, n] of x W^T over slices of K.
float* linear_partials(Ctx& c, const void* x, int m, const void* w, int n, int k, int& slices) {
  const PartialsPlan plan = plan_partials(m, n, k);
  slices = plan.slices;
  float* out = (float*)c.arena->alloc((size_t)plan.slices * m * n * 4);
  if (c.dry) return out;
  const KernelTable& t = need_mfma();
  if (plan.skinny) {
    check_mfma(t.mk_linear_skinny(x, w, out, m, n, k, plan.slices, c.stream), "linear_partials");
  } else {
    check_mfma(t.mk_linear_tiled_partials(x, w, out, m, n, k, plan.slices, c.stream), "linear_partials");
  }
  return out;
}

// h += x W^T (+ bias), or, where that streams the weights faster, partial sums left for the
// next norm to add.
void project_into_stream(Ctx& c, const void* x, int m, const void* w, int n, int k,
                         const void* bias, int bias_dtype, float* h, const float*& pending,
                         int& pending_count) {
  pending = nullptr;
  pending_count = 0;
  if (m == 0) return;
  if (!bias && wants_partials(c.dtype, c.dtype, m, n, k)) {
    pending = linear_partials(c, x, m, w, n, k, pending_count);
    return;
  }
  if (c.dry) return;
  const int bd = bias ? bias_dtype : kF32;
  switch (choose_linear(c.dtype, m, n, k, bias != nullptr, true, kF32)) {
    case LinearKind::GENERIC:
      check_core(need_core().mk_linear_generic(x, w, c.dtype, bias, bd, h, kF32, 1, m, n, k, k, n,
                                               c.stream), "linear");
      break;
    case LinearKind::SKINNY_ACC:
      check_mfma(need_mfma().mk_linear_skinny_acc(x, w, bias, bd, h, m, n, k, c.stream), "linear");
      break;
    default:
      check_mfma(need_mfma().mk_linear_tiled(x, w, bias, bd, h, kF32, 1, m, n, k, n, -1, c.stream),
                 "linear");
  }
}

void* rmsnorm(Ctx& c, float* h, const float* pending, int pending_count, const Op& op,
              const int* rows, int out_rows, void* out = nullptr) {
  if (!out) out = c.arena->alloc((size_t)out_rows * c.hidden * c.elem());
  if (c.dry || out_rows == 0) return out;
  check_core(need_core().mk_rmsnorm(h, pending, pending_count,
                                    (long long)c.step.num_tokens * c.hidden, op.norm_w,
                                    op.norm_w_dtype, op.eps, rows, out, c.dtype, out_rows, c.hidden,
                                    c.stream), "rmsnorm");
  return out;
}

struct Queries {
  const void* q;
  int stride;
};

Queries qkv_project(Ctx& c, const void* x, const Op& op) {
  const StepView& s = c.step;
  const int m = s.num_tokens, k = c.hidden, d = op.head_dim;
  const int heads_kv = op.writes ? op.n_kv : 0;
  const int width = (op.n_q + 2 * heads_kv) * d;
  const int page_size = op.writes ? op.page_size : 1;
  const int bd = op.b_qkv ? op.b_qkv_dtype : kF32;
  const int* table = s.tables.at((size_t)op.group);
  const int table_stride = s.widths.at((size_t)op.group);
  void* k_cache = op.writes ? op.k_cache : nullptr;
  void* v_cache = op.writes ? op.v_cache : nullptr;
  const PositionDesc& p = op.pos;
  const QkvKind kind = choose_qkv(c.dtype, c.dtype, m, width, k, d, p.rotary_dim, page_size,
                                  !p.interleaved);
  if (kind == QkvKind::SKINNY || kind == QkvKind::TILED) {
    void* q = c.arena->alloc((size_t)m * op.n_q * d * 2);
    if (!c.dry) {
      const KernelTable& t = need_mfma();
      const int code = kind == QkvKind::SKINNY
          ? t.mk_qkv_skinny(x, op.w_qkv, op.b_qkv, bd, q, p.cos, p.sin, p.table_positions,
                            s.positions, s.token_seq, table, table_stride, k_cache, v_cache,
                            page_size, op.n_q, heads_kv, d, p.rotary_dim > 0, m, k, c.stream)
          : t.mk_qkv_tiled(x, op.w_qkv, op.b_qkv, bd, q, p.cos, p.sin, p.table_positions,
                           s.positions, s.token_seq, table, table_stride, k_cache, v_cache,
                           page_size, op.n_q, heads_kv, d, p.rotary_dim > 0, m, k, -1, c.stream);
      check_mfma(code, "qkv_project");
    }
    return {q, op.n_q * d};
  }
  if (kind == QkvKind::PARTIALS_FINISH) {
    int slices = 0;
    const float* parts = linear_partials(c, x, m, op.w_qkv, width, k, slices);
    void* q = c.arena->alloc((size_t)m * op.n_q * d * c.elem());
    if (!c.dry) {
      check_core(need_core().mk_qkv_finish(parts, slices, (long long)m * width, op.b_qkv, bd, q,
                                           c.dtype, p.cos, p.sin, p.table_positions, s.positions,
                                           s.token_seq, table, table_stride, k_cache, v_cache,
                                           page_size, op.n_q, heads_kv, d, p.rotary_dim,
                                           op.writes ? 1 : 0, m, c.stream), "qkv_finish");
    }
    return {q, op.n_q * d};
  }
  void* qkv = linear_out(c, x, m, op.w_qkv, width, k, op.b_qkv, bd, c.dtype);
  if (!c.dry) {
    check_core(need_core().mk_rope_kv_write(qkv, c.dtype, width, p.cos, p.sin, p.table_positions,
                                            s.positions, s.token_seq, table, table_stride, k_cache,
                                            v_cache, page_size, op.n_q, heads_kv, d, p.rotary_dim,
                                            p.interleaved ? 1 : 0, op.writes ? 1 : 0, m, c.stream),
               "rope_kv_write");
  }
  return {qkv, width};
}

void* attention(Ctx& c, const Queries& q, const Op& op) {
  const StepView& s = c.step;
  const int m = s.num_tokens, d = op.head_dim;
  const int* table = s.tables.at((size_t)op.group);
  const int table_stride = s.widths.at((size_t)op.group);
  void* out = c.arena->alloc((size_t)m * op.n_q * d * c.elem());
  const AttentionPlan plan = plan_attention(c.dtype, d, op.page_size, op.n_q, op.n_kv, op.window,
                                            s.counts, s.max_q_len, s.max_kv_len);
  if (!plan.mfma) {
    if (!c.dry) {
      check_core(need_core().mk_attention_generic(q.q, q.stride, out, op.n_q * d, op.k_cache,
                                                  op.v_cache, c.dtype, s.positions, s.token_seq,
                                                  table, table_stride, op.page_size, op.n_q, op.n_kv,
                                                  d, op.scale, op.window, m, c.stream), "attention");
    }
    return out;
  }
  float *part_o = nullptr, *part_ml = nullptr;
  if (plan.splits > 1) {
    const size_t rows = (size_t)plan.num_tiles * op.n_kv * plan.splits * plan.rows;
    part_o = (float*)c.arena->alloc(rows * d * 4);
    part_ml = (float*)c.arena->alloc(rows * 2 * 4);
  }
  if (c.dry) return out;
  const StepView::Tiles& tiles = s.tiles_for(op.n_q / op.n_kv, plan.tile_rows);
  check_mfma(need_mfma().mk_attention_mfma(q.q, q.stride, out, op.n_q * d, op.k_cache, op.v_cache,
                                           tiles.seq, tiles.row0, tiles.count, s.cu_q, s.kv_len,
                                           table, table_stride, op.page_size, op.n_q, op.n_kv, d,
                                           op.scale, op.window, plan.rows, plan.staged, plan.splits,
                                           plan.split_blocks, part_o, part_ml, c.stream), "attention");
  return out;
}

void* gated(Ctx& c, const void* x, const Op& op) {
  const int m = c.step.num_tokens, k = c.hidden;
  void* act = nullptr;
  if (fuses_gating(c.dtype, c.dtype, m, k, 2 * op.inter)) {
    act = c.arena->alloc((size_t)m * op.inter * 2);
    if (c.dry) return act;
    const KernelTable& t = need_mfma();
    check_mfma(gated_is_skinny(m)
                   ? t.mk_gated_skinny(x, op.w_gate_up, act, m, op.inter, k, c.stream)
                   : t.mk_gated_tiled(x, op.w_gate_up, act, m, op.inter, k, -1, c.stream),
               "gated_projection");
    return act;
  }
  void* gate_up = linear_out(c, x, m, op.w_gate_up, 2 * op.inter, k, nullptr, kF32, c.dtype);
  act = c.arena->alloc((size_t)m * op.inter * c.elem());
  if (!c.dry && m > 0) {
    check_core(need_core().mk_silu_mul(gate_up, act, c.dtype, m, op.inter, c.stream), "silu_mul");
  }
  return act;
}

}  // namespace

std::vector<Program::TileNeed> Program::tile_needs(const std::vector<int>& counts, int max_q_len,
                                                   int max_kv_len) const {
  std::vector<TileNeed> out;
  for (const Op& op : ops_) {
    if (op.kind != OpKind::ATTENTION) continue;
    const AttentionPlan plan = plan_attention(dtype_, op.head_dim, op.page_size, op.n_q, op.n_kv,
                                              op.window, counts, max_q_len, max_kv_len);
    if (!plan.mfma) continue;
    const TileNeed need{op.n_q / op.n_kv, plan.tile_rows};
    bool known = false;
    for (const TileNeed& t : out) known = known || (t.group == need.group && t.tile_rows == need.tile_rows);
    if (!known) out.push_back(need);
  }
  return out;
}

void Program::walk(const StepView& step, char* workspace, size_t workspace_bytes, void* stream,
                   RunState& state, bool dry, WorkspaceNeed* need) const {
  auto round = [](size_t b) { return (b + 255) & ~(size_t)255; };
  const int elem = element_size(dtype_);
  const size_t h_bytes = round((size_t)step.num_tokens * hidden_ * 4);
  const size_t sel_bytes = round((size_t)step.num_rows * hidden_ * elem);
  const size_t logit_bytes = round((size_t)step.num_rows * vocab_ * 4);
  const size_t persistent = h_bytes + sel_bytes + logit_bytes;
  Arena arenas[2];
  if (dry) {
    arenas[0].reset(nullptr, 0, true);
    arenas[1].reset(nullptr, 0, true);
  } else {
    if (workspace_bytes < persistent) throw KernelError("the step's workspace is too small");
    const size_t each = ((workspace_bytes - persistent) / 2) & ~(size_t)255;
    arenas[0].reset(workspace + persistent, each, false);
    arenas[1].reset(workspace + persistent + each, each, false);
  }
  float* h = (float*)workspace;
  void* selected = workspace + h_bytes;
  float* logits = (float*)(workspace + h_bytes + sel_bytes);
  state.h = h;
  state.logits = nullptr;

  const void* x = nullptr;
  const float* pending = state.pending;
  int pending_count = state.pending_count;
  int i = state.begin;
  for (; i < (int)ops_.size(); ++i) {
    const Op& op = ops_[i];
    if (op.kind == OpKind::HOST) break;
    Arena& arena = arenas[i & 1];
    arena.rewind();
    Ctx c{step, &arena, (hipStream_t)stream, dry, dtype_, hidden_};
    switch (op.kind) {
      case OpKind::EMBED:
        if (!dry && step.num_tokens) {
          check_core(need_core().mk_embed(step.token_ids, op.table, op.table_dtype, h,
                                          step.num_tokens, hidden_, op.vocab, c.stream), "embed");
        }
        break;
      case OpKind::NORM:
        x = rmsnorm(c, h, pending, pending_count, op, nullptr, step.num_tokens);
        pending = nullptr;
        pending_count = 0;
        break;
      case OpKind::ATTENTION: {
        const Queries q = qkv_project(c, x, op);
        const void* attended = attention(c, q, op);
        project_into_stream(c, attended, step.num_tokens, op.w_o, hidden_, op.n_q * op.head_dim,
                            op.b_o, op.b_o_dtype, h, pending, pending_count);
        break;
      }
      case OpKind::GATED_MLP: {
        const void* act = gated(c, x, op);
        project_into_stream(c, act, step.num_tokens, op.w_down, hidden_, op.inter, nullptr, kF32, h,
                            pending, pending_count);
        break;
      }
      case OpKind::HEAD:
        if (step.num_rows > 0) {
          rmsnorm(c, h, pending, pending_count, op, step.logit_rows, step.num_rows, selected);
          linear_out(c, selected, step.num_rows, op.head_w, vocab_, hidden_, nullptr, kF32, kF32,
                     logits);
          state.logits = logits;
        }
        pending = nullptr;
        pending_count = 0;
        break;
      default:
        break;
    }
  }
  state.stopped_at = i;
  state.pending = pending;
  state.pending_count = pending_count;
  if (need) {
    need->persistent = persistent;
    need->arena = std::max(arenas[0].peak(), arenas[1].peak());
  }
}

WorkspaceNeed Program::measure(const StepView& step) const {
  WorkspaceNeed need;
  RunState state;
  int begin = 0;
  // every native stretch of the program, whatever a caller-run layer may hand over
  while (begin < (int)ops_.size()) {
    state.begin = begin;
    state.pending = nullptr;
    state.pending_count = 0;
    WorkspaceNeed part;
    walk(step, nullptr, 0, nullptr, state, true, &part);
    need.persistent = std::max(need.persistent, part.persistent);
    need.arena = std::max(need.arena, part.arena);
    begin = state.stopped_at + 1;
  }
  return need;
}

void Program::run(const StepView& step, char* workspace, size_t workspace_bytes, void* stream,
                  RunState& state) const {
  walk(step, workspace, workspace_bytes, stream, state, false, nullptr);
}

}  // namespace mercury
