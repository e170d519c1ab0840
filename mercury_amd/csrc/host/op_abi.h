/* The C interface of an operation of a step program.
 *
 * A program (program.h) is a list of operations; the host core walks it once per step and
 * knows nothing of what an operation computes.  An operation kind is a name, a `run` function
 * and, optionally, a `tiles` function; an operation is a kind plus a block of bytes (its
 * parameters: weight pointers, sizes, constants) that the program copies and hands back at
 * every call.  Kinds are registered at run time, by the built-in parts of the package and by
 * anybody else: a function pointer is all it takes (from C++, or from Python through ctypes).
 *
 * Registers.  Operations work on a few named values of the step:
 *   h        float32 [T, hidden]   the residual stream, alive for the whole step
 *   x        dtype   [x_rows, hidden]  what the previous operation normalised (or otherwise
 *                                  prepared) for this one to read
 *   pending  float32 [pending_count, T, hidden]  partial sums the previous operation left for
 *                                  this one to add into h
 *   logits   float32 [R, vocab]    the step's result; the operation that fills it says so
 * A step of a few tokens may keep the residual stream in fixed point instead: `h` is then NULL
 * and `h_fixed` holds it as 64-bit integers in units of 2^-32, into which operations add their
 * results with integer atomics (no partial sums are left, `pending` stays empty).  A norm may
 * then leave its work to the operation behind it: `x` is NULL though `x_live` is set, and
 * `norm_weight` / `norm_eps` say what x would have been (rmsnorm(h_fixed) * weight).  Only
 * programs whose every operation is of a kind flagged MK_OP_FIXED_STREAM are run this way.
 * x and pending live in the previous operation's arena, so they are alive for exactly one
 * operation: `x_live` / `pending_count` say whether the previous operation produced them.  An
 * operation that produces them for the next sets `out_*`.
 *
 * Memory.  `alloc` hands out 256-byte aligned device memory from the operation's arena; it is
 * valid until the operation after the next starts.  With `dry` set nothing may be launched:
 * the walk only adds up what the operations allocate, `alloc` returns NULL, and every device
 * pointer of the context is NULL; the operation must still make the same `alloc` calls and
 * set the same `out_*` fields, which is how a program is measured and checked before it runs.
 */
#ifndef MERCURY_OP_ABI_H
#define MERCURY_OP_ABI_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Row tiles of a step: the rows of a sequence are its (token, head-in-group) pairs,
 * `group` heads per token; tile i covers rows [row0[i], row0[i] + tile_rows) of sequence
 * seq[i].  Laid out by the step packer for every (group, tile_rows) an operation asked for. */
typedef struct mk_tile_list {
  int group, tile_rows, count;
  const int* seq;   /* device */
  const int* row0;  /* device */
} mk_tile_list;

typedef struct mk_step_view {
  int num_tokens, num_seqs, num_rows;
  int max_q_len, max_kv_len;
  /* device, int32 */
  const int *token_ids, *positions, *token_seq, *cu_q, *kv_len, *state_slots, *logit_rows;
  /* one block table per cache group: tables[g] is device int32 [num_seqs, widths[g]] */
  int num_groups;
  const int* const* tables;
  const int* widths;
  /* host: tokens per sequence */
  const int* counts;
  int num_tile_lists;
  const mk_tile_list* tile_lists;
} mk_step_view;

typedef struct mk_op_context {
  const mk_step_view* step;
  void* stream;            /* hipStream_t */
  int dry;
  int dtype;               /* 0 float32, 1 bfloat16: the model's compute dtype */
  int hidden, vocab;
  /* in */
  float* h;
  const void* x;
  int x_rows, x_live;
  const float* pending;
  int pending_count;
  float* logits;           /* room for [num_rows, vocab] float32 */
  /* out */
  const void* out_x;
  int out_x_rows, out_x_live;
  const float* out_pending;
  int out_pending_count;
  int out_logits_ready;
  /* the operation's arena */
  void* arena;
  void* (*alloc)(void* arena, size_t bytes);
  /* a message for a non-zero return */
  char error[512];
  /* the residual stream in fixed point (then h is NULL), and the norm the operation before
     left for this one to do (then x is NULL and x_live set); out_norm_*: the same for the
     operation behind this one, with out_x NULL and out_x_live set */
  int stream_fixed;        /* set in a dry walk too, where h_fixed is NULL like every pointer */
  long long* h_fixed;
  const void* norm_weight;
  int norm_weight_dtype;
  float norm_eps;
  const void* out_norm_weight;
  int out_norm_weight_dtype;
  float out_norm_eps;
} mk_op_context;

/* What the shape of a step is before it is packed: enough to say which tile lists an
 * operation will want. */
typedef struct mk_step_shape {
  int dtype;
  int num_seqs;
  const int* counts;
  int max_q_len, max_kv_len;
} mk_step_shape;

typedef struct mk_tile_need {
  int group, tile_rows;
} mk_tile_need;

/* 0 on success; otherwise ctx->error holds the reason. */
typedef int (*mk_op_run_fn)(const void* params, mk_op_context* ctx);
/* Writes at most one need to *out and returns how many (0 or 1). */
typedef int (*mk_op_tiles_fn)(const void* params, const mk_step_shape* shape, mk_tile_need* out);

/* Flags of an operation kind: what it expects of the operation before it. */
enum {
  MK_OP_READS_X = 1,        /* needs a live x */
  MK_OP_FOLDS_PENDING = 2,  /* adds live partial sums into h; without it, live partial sums
                               before this operation are an error (they would be lost) */
  MK_OP_FIXED_STREAM = 4    /* also works on a residual stream in fixed point (h_fixed) and
                               on an x left undone as a norm (norm_weight) */
};

#ifdef __cplusplus
}
#endif

#endif
