// The batch of one step, flattened: any number of sequences' next tokens (portions of
// prompts of any length beside single decoded tokens) as one int32 buffer that a single copy
// takes to the device (reference: the per-request tensors of mercury/runner.py:112-160, which
// run prompts and decoding as separate forwards).
//
// Layout, all int32: token ids [T], absolute positions [T], token -> sequence [T], prefix
// sums of the sequences' token counts [S+1], lengths once this step's tokens are written [S],
// state slots [S], wanted rows [R], one block table per cache group [S, W] (-1: none / given
// back), and the row-tile lists the program's operations asked for.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

#include "cache_manager.h"
#include "program.h"
#include "row_tiles.h"
#include "scheduler.h"

namespace mercury {

class BatchError : public std::invalid_argument {
 public:
  using std::invalid_argument::invalid_argument;
};

struct SeqInput {
  std::string key;
  const int32_t* tokens = nullptr;   // `count` token ids
  int count = 0;
  int start = 0;                     // tokens of the sequence earlier steps have run
  std::vector<int> want;             // indices into this step's tokens whose logits are wanted
};

struct PackedStep {
  int num_tokens = 0, num_seqs = 0, num_rows = 0;
  int max_q_len = 0, max_kv_len = 0;
  std::vector<int> counts, starts, firsts;    // per sequence
  std::vector<int> widths;                    // per group
  std::vector<int> fresh_slots;               // state slots of sequences that start at 0
  // offsets into the buffer, in ints
  size_t off_ids = 0, off_positions = 0, off_token_seq = 0, off_cu_q = 0, off_kv_len = 0,
         off_slots = 0, off_rows = 0;
  std::vector<size_t> off_tables;
  struct TileList {
    int group = 0, tile_rows = 0, count = 0;
    size_t off_seq = 0, off_row0 = 0;
  };
  std::vector<TileList> tiles;
  size_t total = 0;
  int32_t* host = nullptr;                    // the filled buffer (owned by the packer's ring)
  int ring_slot = -1;

  StepView view(const int32_t* device) const;
  // What must be equal for two steps to share device buffers and a captured graph.
  std::vector<int> layout() const;
};

class StepPacker {
 public:
  StepPacker(std::shared_ptr<CacheManager> manager, int vocab_size, int max_positions);
  ~StepPacker();
  StepPacker(const StepPacker&) = delete;
  StepPacker& operator=(const StepPacker&) = delete;

  // table_width < 0: as many columns as the longest sequence needs.  `program` may be null
  // (then no tile lists are laid out).  `check_ids` off when the ids are not the host's to know.
  // kv_bound > 0: the step is planned (how operations split long sequences) as if its longest sequence had
  // that many tokens, as a captured graph needs that later, longer steps will replay.
  PackedStep pack(const std::vector<SeqInput>& seqs, const Program* program, int table_width,
                  bool check_ids = true, int kv_bound = 0);
  PackedStep pack_plan(const Plan& plan, const Program* program, int table_width,
                       int kv_bound = 0);
  // Copy the packed buffer to `device` on `stream`; the buffer's place in the ring is free
  // again once the copy has run.
  void upload(const PackedStep& step, void* device, void* stream);
  void set_pinned(bool pinned) { pinned_ = pinned; }

 private:
  int32_t* acquire(size_t ints, int& slot);

  std::shared_ptr<CacheManager> manager_;
  int vocab_size_, max_positions_;
  bool pinned_ = true;
  struct Slot {
    int32_t* data = nullptr;
    size_t capacity = 0;
    void* event = nullptr;
    bool in_flight = false;
    bool pinned = false;
  };
  std::vector<Slot> ring_;
  int next_ = 0;
};

}  // namespace mercury
