// Which kernel runs an operation of a given shape.  These decisions are pure functions of
// sizes and element types; the launch sequences (launch.cc) ask here, whoever calls them.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

#include "../host/row_tiles.h"

namespace mercury {

constexpr int kF32 = 0, kBF16 = 1;

inline int element_size(int dtype) { return dtype == kBF16 ? 2 : 4; }

// ---- projections

// bfloat16 operands with K a multiple of 8 and at least one row: what the matrix-core
// projections take.
bool mfma_eligible(int x_dtype, int w_dtype, int m, int k);

// Whether x W^T is best computed as float32 partial sums over slices of K that the consumer
// (a norm, or the rotation and cache write) adds up: few enough rows over a matrix large
// enough for bandwidth to matter that whole-K workgroups would leave compute units idle.
bool wants_partials(int x_dtype, int w_dtype, int m, int n, int k);

struct PartialsPlan {
  bool skinny = false;     // weights straight from HBM into the matrix cores (few rows)
  int slices = 1;
};
PartialsPlan plan_partials(int m, int n, int k);

enum class LinearKind { GENERIC = 0, SKINNY = 1, SKINNY_ACC = 2, TILED = 3 };
// force: 0 auto, 1 the float32-arithmetic kernel, 2 the matrix-core kernels.
LinearKind choose_linear(int x_dtype, int m, int n, int k, bool has_bias, bool accumulate,
                         int out_dtype, int force = 0);

// The gated projection act = silu(x Wg^T) * (x Wu^T) as one matrix-core kernel.
bool fuses_gating(int x_dtype, int w_dtype, int m, int k, int rows_of_w);
bool gated_is_skinny(int m);

enum class QkvKind { SKINNY = 0, TILED = 1, PARTIALS_FINISH = 2, LINEAR_ROPE = 3 };
// SKINNY / TILED: projection, bias, rotation and cache write in one kernel.  PARTIALS_FINISH:
// K-split partial sums, then a small kernel that adds them up, rotates and writes.
// LINEAR_ROPE: the projection (whole), then the rotation and cache-write kernel.
QkvKind choose_qkv(int x_dtype, int w_dtype, int m, int width, int k, int head_dim,
                   int rotary_dim, int page_size, bool half_layout);
bool qkv_fusable(int x_dtype, int w_dtype, int m, int k, int head_dim, int rotary_dim,
                 int page_size, bool half_layout);

// Up to how many tokens a step keeps its residual stream in fixed point (64-bit integers that
// projections add into with atomics, the norms folded into the projections behind them): a
// model of bfloat16 whose width the norm-folding projections take; 0 for never.
int fixed_stream_tokens(int dtype, int hidden);
// Whether the norm-folding projections take m rows of width k.
bool folds_norm(int dtype, int m, int k);

// ---- attention

struct AttentionPlan {
  bool mfma = false;
  int rows = 16;          // rows per wavefront tile
  int staged = 0;         // 0, or how many groups of four wavefronts share a workgroup's keys;
                          // 8, 16, 24: the kernel of 32-row wavefronts with one, two, three groups;
                          // 20, 36: the same on tiles of 64 rows with two and four groups
  int splits = 1;
  int split_blocks = 0;   // key blocks (of 32) per part; 0: every tile's own range in equal parts
  bool direct = false;    // decoding, one token per sequence: no tile list, part s of the keys is
                          // every splits-th block from s
  int tile_rows = 16;     // rows per entry of the tile list: rows, 4 * rows when staged, 2 * rows for 20 and 36
  int num_tiles = 0;
};

// counts: tokens per sequence this step.  overrides < 0 (or 0 for splits) leave the choice
// to the step's size.
AttentionPlan plan_attention(int dtype, int head_dim, int page_size, int n_q, int n_kv, int window,
                             const std::vector<int>& counts, int max_q_len, int max_kv_len,
                             int force = 0, int tile_rows = -1, int staged = -1,
                             int splits = 0, int split_blocks = 0);

// Why the matrix-core attention would refuse to run `plan` for these sizes ("" when it takes
// it): the kernel entry point's own argument checks, without the launch.
std::string plan_defect(const AttentionPlan& plan, int head_dim, int page_size, int n_q, int n_kv);

}  // namespace mercury
