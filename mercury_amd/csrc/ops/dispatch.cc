#include "dispatch.h"

#include <algorithm>

#include "kernels.h"

namespace mercury {

namespace {
// Thresholds, each with the measurement that set it.
constexpr int kSkinnyMaxRows = 64;
// K-split partial sums: the skinny kernel up to here, tiles beyond.
constexpr int kSkinnySplitMaxRows = 16;
// Larger matrices stream faster through the tiled kernel's ring of LDS buffers
// (5120 x 27648 at 8 rows: 57 against 50 us; 896 x 4864: 4.8 against 5.4).
constexpr int64_t kSkinnySplitMaxWeights = 20ll << 20;
// Head and gated projection: the skinny kernel below this many rows, tiles from here (the
// head, 152064 x 3584, at 1, 8, 16, 64 rows: skinny 188, 204, 238, 429 us; tiles 187, 191,
// 198, 221).
constexpr int kTiledMinRows = 8;
// A q/k/v matrix from this size on goes as partial sums and a finishing kernel (4608 x 3584 at
// 8, 16, 32, 64 rows: 14.0, 13.9, 15.4, 16.5 us against 15.2, 16.1, 21.1, 30.7 in the one
// skinny kernel; 1152 x 896 the other way round: 10.6 against 6.0).
constexpr int64_t kFusedQkvSplitWeights = 24ll << 20;
constexpr int kFusedQkvTiledRows = 256;
constexpr int kFusedQkvMinWorkgroups = 128;

constexpr int kAttentionTargetWaves = 1024;
constexpr int kAttentionStagedWorkgroups = 64;
constexpr int kAttentionStagedMaxWaves = 16384;
constexpr int kAttentionWideTileWaves = 400;
constexpr int kAttentionMinBlocksPerSplit = 2;
// Beyond this the merge of the parts costs more than the shorter chains save (one sequence
// of 16,384 tokens, 28 heads of 128: 25 us with 256 parts, 17 with 64 or 128).
constexpr int kAttentionMaxSplits = 128;

bool partials_by_skinny(int m, int n, int k) {
  return m <= kSkinnySplitMaxRows && (int64_t)n * k * 2 < kSkinnySplitMaxWeights;
}
}  // namespace

bool mfma_eligible(int x_dtype, int w_dtype, int m, int k) {
  return x_dtype == kBF16 && w_dtype == kBF16 && m > 0 && k % 8 == 0;
}

bool wants_partials(int x_dtype, int w_dtype, int m, int n, int k) {
  if (!mfma_eligible(x_dtype, w_dtype, m, k)) return false;
  const KernelTable& t = need_mfma();
  if (partials_by_skinny(m, n, k)) return !t.mk_linear_skinny_unsplit(m, n, k);
  return t.mk_linear_tiled_slices(m, n, k) > 1;
}

PartialsPlan plan_partials(int m, int n, int k) {
  const KernelTable& t = need_mfma();
  PartialsPlan plan;
  plan.skinny = partials_by_skinny(m, n, k);
  plan.slices = plan.skinny ? t.mk_linear_skinny_slices(m, n, k) : t.mk_linear_tiled_slices(m, n, k);
  return plan;
}

LinearKind choose_linear(int x_dtype, int m, int n, int k, bool has_bias, bool accumulate,
                         int out_dtype, int force) {
  (void)n;
  bool mfma = force == 2 || (force == 0 && x_dtype == kBF16 && k % 8 == 0);
  if (!mfma) return LinearKind::GENERIC;
  if (x_dtype != kBF16 || k % 8) {
    throw KernelError("linear: the matrix-core kernels take bfloat16 with K % 8 == 0");
  }
  if (m < kTiledMinRows && out_dtype == kF32 && !has_bias && !accumulate) return LinearKind::SKINNY;
  if (m <= kSkinnySplitMaxRows && accumulate) return LinearKind::SKINNY_ACC;
  return LinearKind::TILED;
}

bool fuses_gating(int x_dtype, int w_dtype, int m, int k, int rows_of_w) {
  return x_dtype == kBF16 && w_dtype == kBF16 && m > 0 && k % 8 == 0 && rows_of_w % 2 == 0;
}

bool gated_is_skinny(int m) { return m < kTiledMinRows; }

bool qkv_fusable(int x_dtype, int w_dtype, int m, int k, int head_dim, int rotary_dim,
                 int page_size, bool half_layout) {
  return mfma_eligible(x_dtype, w_dtype, m, k) && head_dim % 32 == 0 &&
         (rotary_dim == 0 || rotary_dim == head_dim) && (half_layout || rotary_dim == 0) &&
         page_size > 0 && (page_size & (page_size - 1)) == 0;
}

// Measured on the 0.5B shapes (896 wide), a layer's kernels in replayed graphs: q/k/v with the
// norm folded in 6.0 / 6.5 us at 1 / 8 tokens against 8.0 / 8.6 as norm and projection; gated
// projection with the norm folded in plus a down projection adding with atomics 13.0 / 15.0
// against 15.8 / 16.5; at 16 tokens every workgroup's copy of the rows (8 bytes a value)
// costs more than the norm kernel did (20.6 against 16.8).  Wider rows cost every workgroup
// more: at 1,536 and 2,048 (the 1.5B and 3B shapes) q/k/v still saves 1.6-1.9 us a layer up
// to 8 tokens, but the gated projection and its down projection only break even up to 4
// (27.8 against 27.8, 36.6 against 38.1 us) and lose at 8 (31.0 against 28.4, 39.6 against
// 38.7).
constexpr int kFixedStreamMaxTokens = 8;
constexpr int kFixedStreamNarrow = 1024, kFixedStreamMaxTokensWide = 4;

bool folds_norm(int dtype, int m, int k) {
  if (dtype != kBF16 || m < 1 || k % 8 != 0 || !kernels().has_mfma()) return false;
  return k <= kernels().mk_skinny_normed_max_k(m);
}

int fixed_stream_tokens(int dtype, int hidden) {
  const int most = hidden <= kFixedStreamNarrow ? kFixedStreamMaxTokens : kFixedStreamMaxTokensWide;
  return folds_norm(dtype, most, hidden) ? most : 0;
}

QkvKind choose_qkv(int x_dtype, int w_dtype, int m, int width, int k, int head_dim,
                   int rotary_dim, int page_size, bool half_layout) {
  const bool half = half_layout || rotary_dim == 0;
  auto unfused = [&]() {
    // the finishing kernel rotates in the half-split layout only
    return half && wants_partials(x_dtype, w_dtype, m, width, k) ? QkvKind::PARTIALS_FINISH
                                                                 : QkvKind::LINEAR_ROPE;
  };
  if (!qkv_fusable(x_dtype, w_dtype, m, k, head_dim, rotary_dim, page_size, half_layout)) {
    return unfused();
  }
  const bool partials = wants_partials(x_dtype, w_dtype, m, width, k);
  if (m <= kFusedQkvTiledRows && (int64_t)width * k * 2 >= kFusedQkvSplitWeights && partials) {
    return QkvKind::PARTIALS_FINISH;
  }
  if (m <= 16 || (m <= kSkinnyMaxRows && width / 32 >= kFusedQkvMinWorkgroups)) return QkvKind::SKINNY;
  // many rows: partial sums would be a second pass over [rows, width] in float32
  if (m > kFusedQkvTiledRows || !partials) return QkvKind::TILED;
  return QkvKind::PARTIALS_FINISH;
}

AttentionPlan plan_attention(int dtype, int head_dim, int page_size, int n_q, int n_kv, int window,
                             const std::vector<int>& counts, int max_q_len, int max_kv_len,
                             int force, int tile_rows, int staged_in, int splits_in,
                             int split_blocks_in) {
  AttentionPlan plan;
  plan.mfma = force == 2;
  if (force == 0 && dtype == kBF16) {
    plan.mfma = need_mfma().mk_attention_mfma_supported(head_dim, page_size) != 0;
  }
  if (!plan.mfma) return plan;
  if (dtype != kBF16) throw KernelError("attention: the matrix-core kernel takes bfloat16 only");
  const KernelTable& t = need_mfma();
  const int group = n_q / n_kv;
  // Tiles of 16 rows, the keys split when the tiles alone would leave most of the chip idle
  // (decoding); wider tiles, whose rows share every key fragment a wavefront loads, when
  // there are plenty (prompts).
  const int span = window ? std::min(max_kv_len, window + max_q_len) : max_kv_len;
  const int blocks = std::max(1, (span + 31) / 32);
  int rows = 16;
  long long total_rows = 0;
  for (int c : counts) total_rows += c;
  total_rows *= group;
  // 64-row tiles exist but run at one wavefront per SIMD; 32 rows measured fastest
  const int max_rows = std::min(32, t.mk_attention_mfma_max_rows(head_dim));
  // (never wider than the rows the longest sequence brings: a decoded token's heads are one
  // tile of 16 however many sequences there are)
  while (rows < max_rows && rows < (long long)max_q_len * group &&
         (total_rows / (rows * 2)) * n_kv >= kAttentionWideTileWaves) {
    rows *= 2;
  }
  if (tile_rows > 0) rows = tile_rows;
  int staged = staged_in;
  const bool split_forced = splits_in > 0;
  if (staged >= 8) rows = 32;
  // Prompts of a head size it takes go to the kernel of 32-row wavefronts and 64-key blocks,
  // in workgroups of 128 rows of one sequence or of 64, the keys in one to four chains:
  // whichever instantiation the kernel library measured fastest for a step of this many
  // workgroups and blocks (`staged` 8, 16, 24; 20, 36 for the tiles of 64 rows).
  if (staged < 0 && !split_forced && tile_rows <= 0 && (long long)max_q_len * group >= 64) {
    const long long wg128 = (total_rows / 128) * n_kv, wg64 = (total_rows / 64) * n_kv;
    if (wg64 < (1 << 24)) {
      const int code = t.mk_attention_mfma_wide_choice(head_dim, (int)wg128, (int)wg64, blocks,
                                                       2 * max_q_len > max_kv_len);
      const bool half = code % 8 != 0;
      const int exists = half ? t.mk_attention_mfma_wide_half(head_dim) : t.mk_attention_mfma_wide(head_dim);
      if (code >= 8 && ((exists >> (code / 8 - 1)) & 1) && (half || (long long)max_q_len * group >= 128)) {
        staged = code;
      }
    }
    if (staged >= 8) rows = 32;
  }
  if (staged < 0) {
    // prompts: plenty of rows per sequence, enough workgroups of 64 of them; 16 rows a
    // wavefront measured faster than 32 there
    const bool yes = !split_forced && tile_rows <= 0 && (long long)max_q_len * group >= 64 &&
                     (total_rows / 64) * n_kv >= kAttentionStagedWorkgroups &&
                     t.mk_attention_mfma_staged(head_dim, 16) != 0;
    staged = yes ? -1 : 0;
    if (yes) rows = 16;
  }
  plan.rows = rows;
  plan.tile_rows = staged >= 8 && staged % 8 ? rows * 2 : (staged ? rows * 4 : rows);
  plan.num_tiles = count_tiles(counts, group, plan.tile_rows);
  if (staged == -1) {
    // A workgroup's chain of key blocks is cut into 2 or 4 chains side by side while that
    // leaves the chip short of wavefronts and every chain a few blocks (measured at 2,048
    // tokens, 14 heads of 64: 45, 35, 32 us with 1, 2, 4 groups; at 4,096: 95, 106, 91; at
    // 8,192: 264, 349, 284;
    // 28 heads of 128 at 2,048: 100, 91 with 1, 2; at 8,192: 878, 1055).
    staged = t.mk_attention_mfma_staged(head_dim, 16);
    while (staged > 1 && ((long long)plan.num_tiles * n_kv * 4 * staged > kAttentionStagedMaxWaves ||
                          blocks < 4 * staged)) {
      staged /= 2;
    }
  }
  plan.staged = staged;
  if (staged >= 8) return plan;
  const long long waves = std::max<long long>(1, (long long)plan.num_tiles * n_kv);
  if (!staged && waves < kAttentionTargetWaves) {
    // decoding, and short prompt portions over a long prefix (16 tokens over 2,032: 47 us as
    // one chain of key blocks per wavefront, 23 split): every tile's own range of keys in
    // equal parts
    const int by_blocks = std::max(1, blocks / kAttentionMinBlocksPerSplit);
    const int by_waves = (int)((kAttentionTargetWaves + waves - 1) / waves);
    plan.splits = std::max(1, std::min({by_blocks, by_waves, kAttentionMaxSplits}));
    // in fours, a workgroup's wavefronts take consecutive parts of one tile and add them up
    // through LDS before they write
    if (plan.splits >= 4) plan.splits = plan.splits / 4 * 4;
  }
  if (split_forced) {
    plan.splits = splits_in;
    plan.split_blocks = split_blocks_in;
  }
  // Decoding (every sequence brings one token, whose heads are one tile): no tile list, the
  // parts of the keys every splits-th block (the kernel then knows where a part starts before
  // it knows the sequence's length).
  if (!staged && !split_forced && tile_rows <= 0 && rows == 16 && max_q_len == 1 && window == 0 &&
      group <= 16 && total_rows == (long long)counts.size() * group) {
    plan.direct = true;
  }
  return plan;
}

std::string plan_defect(const AttentionPlan& plan, int head_dim, int page_size, int n_q, int n_kv) {
  if (!plan.mfma) return "";
  const KernelTable& t = need_mfma();
  const int width = n_q * head_dim;
  if (t.mk_attention_mfma_check(width, width, plan.num_tiles, page_size, n_q, n_kv, head_dim, 1.f, 0,
                                plan.rows, plan.staged, plan.splits, plan.split_blocks, 1) == 0) {
    return "";
  }
  return t.mfma_error();
}

}  // namespace mercury
