#include "program.h"

#include <algorithm>
#include <cstring>

namespace mercury {

OpRegistry& OpRegistry::instance() {
  static OpRegistry registry;
  return registry;
}

void OpRegistry::add(const OpKind& kind) {
  if (kind.name.empty() || kind.name == "host") {
    throw KernelError("an operation kind needs a name of its own ('host' is the caller's)");
  }
  if (!kind.run) throw KernelError("operation kind '" + kind.name + "' has no run function");
  kinds_[kind.name] = kind;
}

const OpKind& OpRegistry::get(const std::string& name) const {
  auto it = kinds_.find(name);
  if (it == kinds_.end()) {
    std::string known;
    for (const auto& kv : kinds_) known += (known.empty() ? "" : ", ") + kv.first;
    throw KernelError("no operation kind '" + name + "' is registered; known: " + known);
  }
  return it->second;
}

std::vector<std::string> OpRegistry::names() const {
  std::vector<std::string> out;
  for (const auto& kv : kinds_) out.push_back(kv.first);
  return out;
}

StepView StepView::shape_only(const std::vector<int>& counts, int num_rows, int max_kv_len,
                              int num_groups) {
  StepView v;
  v.counts = counts;
  v.num_seqs = (int)counts.size();
  for (int c : counts) {
    v.num_tokens += c;
    v.max_q_len = std::max(v.max_q_len, c);
  }
  v.num_rows = num_rows;
  v.max_kv_len = max_kv_len;
  v.tables.assign((size_t)num_groups, nullptr);
  v.widths.assign((size_t)num_groups, 0);
  return v;
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

void Program::append(const std::string& kind, const void* params, size_t bytes) {
  Entry e;
  e.kind = OpRegistry::instance().get(kind);
  // Parameter blocks hold pointers and doubles: keep the copy 16-byte aligned whatever the
  // vector's allocator gives.
  e.params.resize(bytes + 16);
  e.offset = (16 - reinterpret_cast<uintptr_t>(e.params.data()) % 16) % 16;
  if (bytes) std::memcpy(e.params.data() + e.offset, params, bytes);
  entries_.push_back(std::move(e));
  // moving a vector keeps its buffer, so the offset computed above still holds
}

void Program::append_caller_step(int index, bool gives_x) {
  Entry e;
  e.kind.name = "host";
  e.caller_index = index;
  e.gives_x = gives_x;
  entries_.push_back(std::move(e));
}

std::string Program::kind_of(size_t i) const { return entries_.at(i).kind.name; }

bool Program::fixed_stream(int num_tokens) const {
  const OpRegistry& registry = OpRegistry::instance();
  if (num_tokens < 1 || entries_.empty()) return false;
  for (const Entry& e : entries_) {
    if (!e.kind.run || !(e.kind.flags & MK_OP_FIXED_STREAM)) return false;
  }
  if (registry.fixed_stream_limit >= 0) return num_tokens <= registry.fixed_stream_limit;
  return registry.fixed_stream_tokens && num_tokens <= registry.fixed_stream_tokens(dtype_, hidden_);
}

std::vector<Program::TileNeed> Program::tile_needs(const std::vector<int>& counts, int max_q_len,
                                                   int max_kv_len) const {
  std::vector<TileNeed> out;
  mk_step_shape shape;
  shape.dtype = dtype_;
  shape.num_seqs = (int)counts.size();
  shape.counts = counts.data();
  shape.max_q_len = max_q_len;
  shape.max_kv_len = max_kv_len;
  for (const Entry& e : entries_) {
    if (!e.kind.tiles) continue;
    mk_tile_need need{0, 0};
    if (e.kind.tiles(e.params.data() + e.offset, &shape, &need) <= 0) continue;
    bool known = false;
    for (const TileNeed& t : out) known = known || (t.group == need.group && t.tile_rows == need.tile_rows);
    if (!known) out.push_back(TileNeed{need.group, need.tile_rows});
  }
  return out;
}

namespace {
void* arena_alloc(void* arena, size_t bytes) { return static_cast<Arena*>(arena)->alloc(bytes); }
}  // namespace

void Program::walk(const StepView& step, char* workspace, size_t workspace_bytes, void* stream,
                   RunState& state, bool dry, WorkspaceNeed* need) const {
  auto round = [](size_t b) { return (b + 255) & ~(size_t)255; };
  const bool own = state.own_h != nullptr || state.own_stream;
  const bool fixed = !own && state.begin == 0 && state.x == nullptr && state.x_rows == 0 &&
                     fixed_stream(step.num_tokens);
  const size_t h_bytes = round((size_t)step.num_tokens * hidden_ * (fixed ? 8 : 4));
  const size_t logit_bytes = round((size_t)step.num_rows * vocab_ * 4);
  const size_t persistent = own ? 0 : h_bytes + logit_bytes;
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

  mk_step_view view;
  view.num_tokens = step.num_tokens;
  view.num_seqs = step.num_seqs;
  view.num_rows = step.num_rows;
  view.max_q_len = step.max_q_len;
  view.max_kv_len = step.max_kv_len;
  view.token_ids = step.token_ids;
  view.positions = step.positions;
  view.token_seq = step.token_seq;
  view.cu_q = step.cu_q;
  view.kv_len = step.kv_len;
  view.state_slots = step.state_slots;
  view.logit_rows = step.logit_rows;
  view.num_groups = (int)step.tables.size();
  view.tables = step.tables.data();
  view.widths = step.widths.data();
  view.counts = step.counts.data();
  view.num_tile_lists = (int)step.tiles.size();
  view.tile_lists = step.tiles.data();

  mk_op_context ctx;
  std::memset(&ctx, 0, sizeof ctx);
  ctx.step = &view;
  ctx.stream = stream;
  ctx.dry = dry ? 1 : 0;
  ctx.dtype = dtype_;
  ctx.hidden = hidden_;
  ctx.vocab = vocab_;
  ctx.h = dry || fixed ? nullptr : (own ? state.own_h : (float*)workspace);
  ctx.stream_fixed = fixed ? 1 : 0;
  ctx.h_fixed = dry || !fixed ? nullptr : (long long*)workspace;
  ctx.logits = dry ? nullptr : (own ? state.own_logits : (float*)(workspace + h_bytes));
  ctx.alloc = &arena_alloc;
  state.h = ctx.h;
  state.logits = nullptr;

  // What the entry before `begin` left (a caller-run step's hand-over, or nothing).
  const void* x = state.x;
  int x_rows = state.x_rows;
  bool x_live = state.x != nullptr || (dry && state.x_rows > 0);
  const float* pending = state.pending;
  int pending_count = state.pending_count;
  const void* norm_weight = nullptr;   // a norm left to the next operation (fixed point only)
  int norm_weight_dtype = 0;
  float norm_eps = 0.f;

  int i = state.begin;
  for (; i < (int)entries_.size(); ++i) {
    const Entry& e = entries_[i];
    if (!e.kind.run) break;
    if ((e.kind.flags & MK_OP_READS_X) && !x_live) {
      throw KernelError("operation " + std::to_string(i) + " ('" + e.kind.name +
                        "') reads x, but the operation before it left none: x lives for one "
                        "operation only");
    }
    if (pending_count > 0 && !(e.kind.flags & MK_OP_FOLDS_PENDING)) {
      throw KernelError("operation " + std::to_string(i) + " ('" + e.kind.name +
                        "') follows one that left partial sums, and does not add them up");
    }
    Arena& arena = arenas[i & 1];
    arena.rewind();
    ctx.arena = &arena;
    ctx.x = x_live ? x : nullptr;
    ctx.x_rows = x_live ? x_rows : 0;
    ctx.x_live = x_live ? 1 : 0;
    ctx.pending = pending;
    ctx.pending_count = pending_count;
    ctx.norm_weight = x_live ? norm_weight : nullptr;
    ctx.norm_weight_dtype = norm_weight_dtype;
    ctx.norm_eps = norm_eps;
    ctx.out_norm_weight = nullptr;
    ctx.out_norm_weight_dtype = 0;
    ctx.out_norm_eps = 0.f;
    ctx.out_x = nullptr;
    ctx.out_x_rows = 0;
    ctx.out_x_live = 0;
    ctx.out_pending = nullptr;
    ctx.out_pending_count = 0;
    ctx.out_logits_ready = 0;
    ctx.error[0] = 0;
    const int code = e.kind.run(e.params.data() + e.offset, &ctx);
    if (code != 0) {
      ctx.error[sizeof ctx.error - 1] = 0;
      throw KernelError("operation " + std::to_string(i) + " ('" + e.kind.name + "'): " +
                        (ctx.error[0] ? ctx.error : "failed without a message"));
    }
    x = ctx.out_x;
    x_rows = ctx.out_x_rows;
    x_live = ctx.out_x_live != 0;
    pending = ctx.out_pending;
    pending_count = ctx.out_pending_count;
    norm_weight = ctx.out_norm_weight;
    norm_weight_dtype = ctx.out_norm_weight_dtype;
    norm_eps = ctx.out_norm_eps;
    if (norm_weight && !fixed) {
      throw KernelError("operation " + std::to_string(i) + " ('" + e.kind.name +
                        "') left a norm undone outside a step in fixed point");
    }
    if (ctx.out_logits_ready) state.logits = ctx.logits;
  }
  state.stopped_at = i;
  state.x = x_live ? x : nullptr;
  state.x_rows = x_live ? x_rows : 0;
  state.pending = pending;
  state.pending_count = pending_count;
  if (need) {
    need->persistent = persistent;
    need->arena = std::max(arenas[0].peak(), arenas[1].peak());
  }
}

WorkspaceNeed Program::measure(const StepView& step, int given_x_rows, bool own_stream) const {
  WorkspaceNeed need;
  RunState state;
  state.own_stream = own_stream;
  int begin = 0;
  // every stretch between caller-run steps; behind such a step, x is there if it says so and
  // partial sums may or may not be (an operation that adds them up takes none as well)
  while (begin < (int)entries_.size()) {
    state.begin = begin;
    state.x = nullptr;
    state.x_rows = begin == 0 ? given_x_rows
                              : (entries_[begin - 1].gives_x ? step.num_tokens : 0);
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
