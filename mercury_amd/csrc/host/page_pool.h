// A pool of fixed-size cache pages with an index of reusable prefix pages.
//
// Every page is in exactly one of three states (reference: mercury/allocator.py:7-16):
//   free   nobody holds it and no hash names it; it waits in the free queue
//   held   at least one sequence's block table names it
//   idle   nobody holds it but a hash still names it: reusable as a prefix page, and the
//          first to be recycled, least recently released first, when the free queue is empty
// The three states are two intrusive doubly-linked lists threaded through one array of page
// records (held pages are on neither), so every transition is O(1), and one hash table from
// page hash to page.  A page id addresses the same page in the keys and the values of every
// cache slot of the pool's group.  Pages are not cleared when they change hands: the kernels
// never read past a sequence's own length.
#pragma once

#include <cstdint>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "hashing.h"

namespace mercury {

class PoolError : public std::logic_error {
 public:
  using std::logic_error::logic_error;
};

class PagePool {
 public:
  struct Stats {
    int64_t hit_tokens = 0, query_tokens = 0, evictions = 0, prefills = 0, allocation_failures = 0;
  };

  PagePool(int num_pages, int page_size);

  int num_pages() const { return (int)pages_.size(); }
  int page_size() const { return page_size_; }
  int num_free() const { return free_.count; }
  int num_idle() const { return idle_.count; }
  int available() const { return free_.count + idle_.count; }
  int num_indexed() const { return (int)index_.size(); }
  int holders(int page) const { return pages_[page].holders; }
  bool hashed(int page) const { return pages_[page].hashed; }
  const PageHash& hash_of(int page) const { return pages_[page].hash; }
  int page_for(const PageHash& h) const;          // -1 when no page carries the hash
  std::vector<int> free_order() const { return order(free_); }
  std::vector<int> idle_order() const { return order(idle_); }   // next to be recycled first
  const Stats& stats() const { return stats_; }
  void reset_stats() { stats_ = Stats(); }
  double hit_rate() const {
    return stats_.query_tokens ? (double)stats_.hit_tokens / (double)stats_.query_tokens : 0.0;
  }

  // The pages that hold the longest indexed prefix of the chain.
  std::vector<int> match(const std::vector<PageHash>& chain) const;
  // How many leading pages a prompt of `num_tokens` would reuse: the match, cut so that at
  // least one token is left to compute (a prompt that is wholly cached would yield no
  // logits, reference: mercury/allocator.py:64-73) and to `cap` pages when cap >= 0.
  int reusable(const std::vector<PageHash>& chain, int num_tokens, int cap = -1) const;
  // Pages for a whole prompt: the reusable prefix pages (held once more) followed by fresh
  // ones.  False, with nothing changed but the failure count, when the pool cannot give them.
  bool reserve(const std::vector<PageHash>& chain, int num_tokens, int cap,
               std::vector<int>& pages_out, int& reused_tokens);
  // One fresh page held once, or -1.
  int take();
  // Make a full page findable under its hash; the first page to carry a hash keeps it, a
  // later page with the same content stays private (reference: mercury/allocator.py:104-108).
  void publish(int page, const PageHash& h);
  // Give pages back, the last first, so that a sequence's private tail is recycled before
  // the prefix that others may share (reference: mercury/allocator.py:110-121).
  void give_back(const int* pages, int count);
  // Every page in exactly one state, the lists and the index consistent.  O(pages).
  void audit() const;

 private:
  enum Where : uint8_t { HELD = 0, FREE = 1, IDLE = 2 };
  struct Page {
    int holders = 0;
    int prev = -1, next = -1;
    Where where = FREE;
    bool hashed = false;
    PageHash hash;
  };
  struct List {
    int head = -1, tail = -1, count = 0;
  };

  void push_back(List& list, Where where, int page);
  void unlink(List& list, int page);
  std::vector<int> order(const List& list) const;
  int recycle();      // the next page to hand out: free queue first, then the oldest idle page

  int page_size_;
  std::vector<Page> pages_;
  List free_, idle_;
  std::unordered_map<PageHash, int, PageHashHasher> index_;
  Stats stats_;
};

}  // namespace mercury
