// The operation kinds the package's own parts lower themselves to, each a parameter block
// and a run function over the launch sequences of launch.h.  They are registered like any
// kind from outside would be (OpRegistry); the program walk knows none of them.
#pragma once

#include "launch.h"

namespace mercury {

// "embed": h = table[token_ids] * scale.
struct EmbedParams {
  const void* table = nullptr;
  int table_dtype = 0, vocab = 0;
  float scale = 1.f;
};

// "norm": x = rmsnorm(h + pending) * weight; with select_rows, of the step's wanted rows only
// (what an output head reads).
struct NormParams {
  const void* weight = nullptr;
  int weight_dtype = 0;
  float eps = 0.f;
  int select_rows = 0;
};

// "attention": q/k/v projection, position encoding, cache write, softmax attention over the
// cache, output projection into h (or left as partial sums).
struct AttentionParams {
  QkvArgs qkv;
  const void *w_o = nullptr, *b_o = nullptr;
  int b_o_dtype = 0;
  int group = 0;          // which of the step's block tables
  int window = 0;
  float scale = 0.f;
  float score_cap = 0.f;                    // > 0: the score is bounded to cap * tanh(. / cap)
  const float* distance_slopes = nullptr;   // [n_q]: slope * distance is subtracted from it
};

// "gated_mlp": h += (act(x Wg^T) * (x Wu^T)) Wd^T (or left as partial sums).
struct GatedMlpParams {
  const void *w_gate_up = nullptr, *w_down = nullptr;
  int inter = 0;
};

// "head": logits = x W^T (+ bias), optionally capped to cap * tanh(. / cap).
struct HeadParams {
  const void *weight = nullptr, *bias = nullptr;
  int bias_dtype = 0;
  float cap = 0.f;
};

void register_builtin_ops();

}  // namespace mercury
