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
              void* out = nullptr);

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

// Rotation and cache write of an already projected qkv [m, row_stride] (q rotated in place).
void rope_kv_write(Launch& l, void* qkv, int row_stride, int m, const QkvArgs& a,
                   const StepArrays& s);

// The same for a projection that arrives as partial sums [slices, m, width]; the rotated q
// goes to a new [m, n_q d] tensor of out_dtype.
void* qkv_finish(Launch& l, const float* parts, int slices, int m, const QkvArgs& a,
                 const StepArrays& s, int out_dtype);

struct AttendArgs {
  int n_q = 0, n_kv = 0, head_dim = 0, page_size = 0, window = 0;
  float scale = 0.f;
  const void *k_cache = nullptr, *v_cache = nullptr;
  // What only the float32-arithmetic kernel computes: a bound cap * tanh(score / cap) on the
  // score, and a penalty slope[head] * distance subtracted from it.  With either, that kernel
  // runs whatever the dtype.
  float score_cap = 0.f;
  const float* distance_slopes = nullptr;
  bool plain_scores() const { return score_cap <= 0.f && distance_slopes == nullptr; }
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

// act = silu(x Wg^T) * (x Wu^T) for w = [Wg | Wu] stacked [2 inter, k].  tile_config: -2 by the
// sizes, else the tiled kernel with that configuration (-1: its own choice).
// `fold` as for qkv_project.
void* gated(Launch& l, const void* x, int m, int k, const void* w_gate_up, int inter,
            int tile_config = -2, const NormFold* fold = nullptr);

}  // namespace mercury
