// A model's step as data: the list of operations one step launches, built once from the
// model's parts, and the code that walks it, one call per step.
//
// Registers (all in a workspace the caller provides):
//   h        float32 [T, H]   the residual stream; persistent over the step
//   x        dtype   [T, H]   the last norm's output
//   pending  float32 [P, T, H] partial sums of the last projection that the next norm adds
//                             into h in the same pass (none when the projection added its
//                             output into h itself)
//   logits   float32 [R, V]
// An operation allocates its outputs and temporaries from one of two arenas, alternating, so
// that what the previous operation left is still there to read; `measure` walks the same code
// without launching and reports the sizes a step needs.
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "dispatch.h"

namespace mercury {

// How a position encoding transforms q and k: rotation by tabulated angles over the first
// `rotary_dim` dims of a head, pairing dim j with j + rotary_dim/2 ("half") or 2j with 2j+1
// ("interleaved"); rotary_dim 0 is no transformation.
struct PositionDesc {
  int rotary_dim = 0;
  const float* cos = nullptr;
  const float* sin = nullptr;
  int table_positions = 0;
  bool interleaved = false;
};

enum class OpKind { EMBED, NORM, ATTENTION, GATED_MLP, HEAD, HOST };

struct Op {
  OpKind kind = OpKind::HOST;
  // EMBED
  const void* table = nullptr;
  int table_dtype = 0, vocab = 0;
  // NORM, and the norm inside HEAD
  const void* norm_w = nullptr;
  int norm_w_dtype = 0;
  float eps = 0.f;
  // ATTENTION
  const void *w_qkv = nullptr, *b_qkv = nullptr, *w_o = nullptr, *b_o = nullptr;
  int b_qkv_dtype = 0, b_o_dtype = 0;
  int n_q = 0, n_kv = 0, head_dim = 0;
  PositionDesc pos;
  void *k_cache = nullptr, *v_cache = nullptr;
  int group = 0, page_size = 0, window = 0;
  float scale = 0.f;
  bool writes = true;
  // GATED_MLP
  const void *w_gate_up = nullptr, *w_down = nullptr;
  int inter = 0;
  // HEAD
  const void* head_w = nullptr;
  // HOST: the execution-list entry the caller runs itself
  int host_index = -1;
};

// The index arrays of a step on the device, and what the host knows of it.
struct StepView {
  int num_tokens = 0, num_seqs = 0, num_rows = 0;
  const int *token_ids = nullptr, *positions = nullptr, *token_seq = nullptr, *cu_q = nullptr,
            *kv_len = nullptr, *state_slots = nullptr, *logit_rows = nullptr;
  std::vector<const int*> tables;     // per cache group [S, width]
  std::vector<int> widths;
  std::vector<int> counts;            // tokens per sequence
  int max_q_len = 0, max_kv_len = 0;
  // attention tile lists by rows per tile (device), as the packer laid them out
  struct Tiles {
    int group = 0, tile_rows = 0, count = 0;
    const int *seq = nullptr, *row0 = nullptr;
  };
  std::vector<Tiles> tiles;
  const Tiles& tiles_for(int group, int tile_rows) const;
};

class Arena {
 public:
  void reset(char* base, size_t size, bool dry) {
    base_ = base;
    size_ = size;
    used_ = 0;
    dry_ = dry;
  }
  void rewind() { used_ = 0; }
  void* alloc(size_t bytes);
  size_t peak() const { return peak_; }
  bool dry() const { return dry_; }

 private:
  char* base_ = nullptr;
  size_t size_ = 0, used_ = 0, peak_ = 0;
  bool dry_ = true;
};

struct RunState {
  // in: where to start, and partial sums a caller-run layer left (pointer, slice count)
  int begin = 0;
  const float* pending = nullptr;
  int pending_count = 0;
  // out: the operation the walk stopped before (ops.size() when it ran to the end)
  int stopped_at = 0;
  float* h = nullptr;
  float* logits = nullptr;
};

struct WorkspaceNeed {
  size_t persistent = 0, arena = 0;
  size_t total() const { return persistent + 2 * arena; }
};

class Program {
 public:
  Program(int dtype, int hidden, int vocab) : dtype_(dtype), hidden_(hidden), vocab_(vocab) {}
  int dtype() const { return dtype_; }
  int hidden() const { return hidden_; }
  int vocab() const { return vocab_; }
  std::vector<Op>& ops() { return ops_; }
  const std::vector<Op>& ops() const { return ops_; }

  // The (heads-per-group, window, head size, page size ...) signatures of the program's
  // attention operations, each with the tile lists a step of these counts needs.
  struct TileNeed {
    int group, tile_rows;
  };
  std::vector<TileNeed> tile_needs(const std::vector<int>& counts, int max_q_len,
                                   int max_kv_len) const;

  WorkspaceNeed measure(const StepView& step) const;
  // Walk the operations from state.begin until the end or a HOST operation.  `workspace`
  // must hold measure(step).total() bytes.
  void run(const StepView& step, char* workspace, size_t workspace_bytes, void* stream,
           RunState& state) const;

 private:
  void walk(const StepView& step, char* workspace, size_t workspace_bytes, void* stream,
            RunState& state, bool dry, WorkspaceNeed* need) const;

  int dtype_, hidden_, vocab_;
  std::vector<Op> ops_;
};

}  // namespace mercury
