// A model's step as data: the list of operations one step launches, built once from the
// model's parts, and the code that walks it, one call per step.
//
// The walk knows nothing of what an operation computes.  An operation is a registered kind
// (op_abi.h: a name, a run function, optionally a function that says which row-tile lists a
// step must carry for it) and a block of parameter bytes; kinds are registered at run time,
// the package's own parts and anybody else's alike.  An entry may also be a *caller-run* step:
// the walk stops there, the caller does that work itself on the same registers, and the walk
// resumes behind it.
//
// Registers (op_abi.h) live in a workspace the caller provides: h and logits for the whole
// step; x and pending in the arena of the operation that produced them.  Operations allocate
// from one of two arenas in turn, so what the previous operation left is there to read and
// what the one before left is gone: x and pending are alive for exactly one operation, and
// the walk refuses (in a dry walk too, so at build time) a program in which an operation
// reads an x that is no longer there or would drop partial sums nobody added up.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <string>
#include <vector>

#include "errors.h"
#include "op_abi.h"

namespace mercury {

struct OpKind {
  std::string name;
  mk_op_run_fn run = nullptr;
  mk_op_tiles_fn tiles = nullptr;
  int flags = 0;
};

// name -> kind, for the process.  Registering a name again replaces the kind for programs
// built afterwards (programs hold their kinds by value).
class OpRegistry {
 public:
  static OpRegistry& instance();
  void add(const OpKind& kind);
  const OpKind& get(const std::string& name) const;
  bool has(const std::string& name) const { return kinds_.count(name) != 0; }
  std::vector<std::string> names() const;
  // Up to how many tokens a step of a model of this dtype and width keeps its residual
  // stream in fixed point (op_abi.h), 0 for never: set by whoever registers operations that
  // can (the rule depends on their kernels); null: never.
  int (*fixed_stream_tokens)(int dtype, int hidden) = nullptr;
  // >= 0: that many tokens whatever the rule says (0: never), for tests and for comparing.
  int fixed_stream_limit = -1;

 private:
  std::map<std::string, OpKind> kinds_;
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
  std::vector<mk_tile_list> tiles;    // as the packer laid them out

  // A step of this shape with no device arrays behind it, for dry walks.
  static StepView shape_only(const std::vector<int>& counts, int num_rows, int max_kv_len,
                             int num_groups);
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
  // in: where to start, and what a caller-run step left for the operation behind it
  int begin = 0;
  const void* x = nullptr;
  int x_rows = 0;
  const float* pending = nullptr;
  int pending_count = 0;
  // in, optional: a residual stream and room for logits of the caller's own (a single
  // operation run on tensors that exist already); the workspace is then all arena
  float* own_h = nullptr;
  float* own_logits = nullptr;
  bool own_stream = false;      // a dry walk for such a run (own_h is null there like every pointer)
  // out: the entry the walk stopped before (size() when it ran to the end), and the
  // registers as they stand there
  int stopped_at = 0;
  float* h = nullptr;
  float* logits = nullptr;      // null until an operation filled them
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

  // Append an operation of a registered kind; the parameter bytes are copied.
  void append(const std::string& kind, const void* params, size_t bytes);
  // Append a step the caller runs itself; `index` is the caller's own name for it, and
  // `gives_x` says whether it leaves an x for the operation behind it.
  void append_caller_step(int index, bool gives_x);

  size_t size() const { return entries_.size(); }
  // Whether a step of this many tokens runs on a residual stream in fixed point: every entry
  // an operation of a kind that can, and few enough tokens for the registry's rule.
  bool fixed_stream(int num_tokens) const;
  // The kind's name, or "host" for a caller-run step.
  std::string kind_of(size_t i) const;
  int caller_index(size_t i) const { return entries_.at(i).caller_index; }

  struct TileNeed {
    int group, tile_rows;
  };
  // The row-tile lists a step of this shape must carry for the program's operations.
  std::vector<TileNeed> tile_needs(const std::vector<int>& counts, int max_q_len,
                                   int max_kv_len) const;

  // Walk without launching: what a step of this shape needs of its workspace.  Throws when
  // the operations do not fit together.  given_x_rows > 0: the caller brings an x of that
  // many rows for the first operation (a program that is one operation of a model).
  // own_stream: for a run on a residual stream of the caller's own.
  WorkspaceNeed measure(const StepView& step, int given_x_rows = 0, bool own_stream = false) const;
  // Walk from state.begin until the end or a caller-run step.  `workspace` must hold
  // measure(step).total() bytes.
  void run(const StepView& step, char* workspace, size_t workspace_bytes, void* stream,
           RunState& state) const;

 private:
  struct Entry {
    OpKind kind;                 // run == nullptr: a caller-run step
    std::vector<char> params;    // 16-byte aligned copy (see append)
    size_t offset = 0;
    int caller_index = -1;
    bool gives_x = false;
  };
  void walk(const StepView& step, char* workspace, size_t workspace_bytes, void* stream,
            RunState& state, bool dry, WorkspaceNeed* need) const;

  int dtype_, hidden_, vocab_;
  std::vector<Entry> entries_;
};

}  // namespace mercury
