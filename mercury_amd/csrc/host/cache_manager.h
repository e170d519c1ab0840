// The cache manager: block tables per sequence over one page pool per group of cache slots,
// and one slot of fixed-size state per sequence.
//
// Cache slots (one per writing entry of a model's execution list) with the same need (key and
// value heads and widths, element type, window) form a group.  A group has pages of its own
// and every sequence has one block table per group; all slots of a group use that table, each
// over its own key and value tensors.
//   * A group that keeps all keys takes the pages of a whole prompt at admission (reusable
//     prefix pages first, when prefix sharing is on) and one more page whenever the sequence
//     grows across a page edge.
//   * A group with a window takes pages step by step, for the tokens of the step, and gives
//     back every page whose last position the window has passed; the table keeps -1 there.
//   * Everything goes back to its pool when the sequence ends, is aborted or is preempted.
// Prefix sharing needs every group to keep all keys and no mixer to carry state of its own;
// otherwise a cached page does not describe all that a later sequence needs.
#pragma once

#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "page_pool.h"

namespace mercury {

struct GroupSpec {
  int kv_heads = 0, k_dim = 0, v_dim = 0;
  int dtype = -1;      // element type of keys and values; -1: the model's compute dtype
  int window = 0;      // 0: all earlier keys
  bool operator==(const GroupSpec& o) const {
    return kv_heads == o.kv_heads && k_dim == o.k_dim && v_dim == o.v_dim && dtype == o.dtype &&
           window == o.window;
  }
};

// A key that names no admitted sequence.
class UnknownSequence : public std::out_of_range {
 public:
  explicit UnknownSequence(const std::string& key)
      : std::out_of_range("'" + key + "' holds nothing in the cache") {}
};

class StateSlots {
 public:
  explicit StateSlots(int count);
  int count() const { return count_; }
  int available() const { return (int)free_.size(); }
  int take(const std::string& key);                 // -1 when none is free
  void give(const std::string& key);
  int slot_of(const std::string& key) const;
  void audit() const;

 private:
  int count_;
  std::vector<int> free_;
  std::unordered_map<std::string, int> owner_;
};

struct Sequence {
  std::vector<std::vector<int>> tables;   // per group: page ids, -1 = given back
  std::vector<int> first_live;            // per group: index of the first page still held
  int state_slot = -1;
  int cached_tokens = 0;
  int committed = 0;                      // full pages already offered to the prefix index
};

class CacheManager {
 public:
  struct Group {
    GroupSpec spec;
    std::vector<int> slots;
    std::unique_ptr<PagePool> pool;
  };

  // slots: (cache slot id, what it needs), in slot order.
  CacheManager(const std::vector<std::pair<int, GroupSpec>>& slots, int num_pages, int page_size,
               int max_sequences, bool has_state);

  int page_size() const { return page_size_; }
  bool prefix_sharing() const { return prefix_sharing_; }
  bool has_state() const { return has_state_; }
  int num_groups() const { return (int)groups_.size(); }
  const Group& group(int g) const { return groups_.at((size_t)g); }
  Group& group(int g) { return groups_.at((size_t)g); }
  int group_of_slot(int slot) const;
  StateSlots& state_slots() { return state_slots_; }
  PagePool* main_pool();            // the first all-keys group's pool (admission statistics)

  int available() const;            // pages the tightest group can still give
  int capacity_tokens() const;
  int cached_prefix_tokens(const std::vector<PageHash>& chain) const;
  int leaked_pages() const;
  bool holds(const std::string& key) const { return sequences_.count(key) != 0; }
  const Sequence& sequence(const std::string& key) const;
  size_t num_sequences() const { return sequences_.size(); }
  std::vector<std::string> keys() const;

  // Take a state slot and, in every all-keys group, the pages of a prompt of `num_tokens`.
  // Returns the number of leading tokens whose keys are already cached, or -1 (nothing
  // changed) when it does not fit.
  int admit(const std::string& key, const std::vector<PageHash>& chain, int num_tokens);
  // Make sure every group holds the pages for computing positions [start, new_len).  False,
  // with nothing changed, when a pool has no page left.
  bool grow(const std::string& key, int start, int new_len);
  // Give back the pages of window groups that no later query can see, now that positions
  // below `num_computed` are computed.  Returns how many pages went back.
  int trim(const std::string& key, int num_computed);
  // Offer the sequence's pages [committed, full_pages) to the prefix index under their chain
  // hashes (reference: mercury/engine.py:232-241).
  void commit(const std::string& key, const std::vector<PageHash>& chain, int full_pages);
  // Everything the sequence holds goes back: the pages of every group and its state slot.
  void release(const std::string& key);
  // No page lost, held twice without a shared hash, or freed twice; state slots whole.
  void audit() const;

 private:
  static int first_needed(const GroupSpec& spec, int next_position) {
    return spec.window == 0 ? 0 : std::max(0, next_position - spec.window + 1);
  }
  Sequence& mutable_sequence(const std::string& key);

  int page_size_;
  bool has_state_, prefix_sharing_;
  std::vector<Group> groups_;
  std::unordered_map<int, int> group_of_slot_;
  StateSlots state_slots_;
  std::unordered_map<std::string, Sequence> sequences_;
};

}  // namespace mercury
