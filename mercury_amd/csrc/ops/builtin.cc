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
                         rows);
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
    const Queries q = qkv_project(l, ctx->x, s.num_tokens, ctx->hidden, p.qkv, arrays, {},
                                  fold_of(ctx, fold));
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
  out->group = p.qkv.n_q / p.qkv.n_kv;
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
    const void* act = gated(l, ctx->x, m, ctx->hidden, p.w_gate_up, p.inter, -2, fold_of(ctx, fold));
    if (ctx->stream_fixed) {
      project_into_fixed(l, act, m, p.w_down, ctx->hidden, p.inter, nullptr, kF32, ctx->h_fixed);
      return;
    }
    project_into_stream(l, act, m, p.w_down, ctx->hidden, p.inter, nullptr, kF32, ctx->h,
                        ctx->out_pending, ctx->out_pending_count);
  });
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
  r.add(OpKind{"gated_mlp", &run_gated_mlp, nullptr, MK_OP_READS_X | MK_OP_FIXED_STREAM});
  r.add(OpKind{"head", &run_head, nullptr, MK_OP_READS_X | MK_OP_FIXED_STREAM});
  r.fixed_stream_tokens = &fixed_stream_tokens;
}

}  // namespace mercury
