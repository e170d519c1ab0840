#include "cache_manager.h"

#include <algorithm>

namespace mercury {

StateSlots::StateSlots(int count) : count_(count) {
  for (int s = count - 1; s >= 0; --s) free_.push_back(s);
}

int StateSlots::take(const std::string& key) {
  if (owner_.count(key)) throw PoolError("'" + key + "' already owns a state slot");
  if (free_.empty()) return -1;
  const int slot = free_.back();
  free_.pop_back();
  owner_[key] = slot;
  return slot;
}

void StateSlots::give(const std::string& key) {
  auto it = owner_.find(key);
  if (it == owner_.end()) throw PoolError("'" + key + "' owns no state slot");
  free_.push_back(it->second);
  owner_.erase(it);
}

int StateSlots::slot_of(const std::string& key) const {
  auto it = owner_.find(key);
  if (it == owner_.end()) throw PoolError("'" + key + "' owns no state slot");
  return it->second;
}

void StateSlots::audit() const {
  std::vector<uint8_t> seen((size_t)count_, 0);
  auto mark = [&](int slot) {
    if (slot < 0 || slot >= count_ || seen[slot]) {
      throw PoolError("a state slot is owned twice or both owned and free");
    }
    seen[slot] = 1;
  };
  for (const auto& kv : owner_) mark(kv.second);
  for (int slot : free_) mark(slot);
  if ((int)(owner_.size() + free_.size()) != count_) throw PoolError("a state slot was lost");
}

CacheManager::CacheManager(const std::vector<std::pair<int, GroupSpec>>& slots, int num_pages,
                           int page_size, int max_sequences, bool has_state)
    : page_size_(page_size), has_state_(has_state), state_slots_(max_sequences) {
  if (page_size <= 0 || (page_size & (page_size - 1))) {
    throw std::invalid_argument("page_size must be a positive power of two");
  }
  auto ordered = slots;
  std::sort(ordered.begin(), ordered.end(),
            [](const auto& a, const auto& b) { return a.first < b.first; });
  for (const auto& entry : ordered) {
    int found = -1;
    for (int g = 0; g < (int)groups_.size(); ++g) {
      if (groups_[g].spec == entry.second) found = g;
    }
    if (found < 0) {
      found = (int)groups_.size();
      Group group;
      group.spec = entry.second;
      group.pool = std::make_unique<PagePool>(num_pages, page_size);
      groups_.push_back(std::move(group));
    }
    groups_[found].slots.push_back(entry.first);
    group_of_slot_[entry.first] = found;
  }
  prefix_sharing_ = !has_state;
  for (const Group& g : groups_) prefix_sharing_ = prefix_sharing_ && g.spec.window == 0;
}

int CacheManager::group_of_slot(int slot) const {
  auto it = group_of_slot_.find(slot);
  if (it == group_of_slot_.end()) throw std::out_of_range("no cache slot " + std::to_string(slot));
  return it->second;
}

PagePool* CacheManager::main_pool() {
  for (Group& g : groups_) {
    if (g.spec.window == 0) return g.pool.get();
  }
  return groups_.empty() ? nullptr : groups_[0].pool.get();
}

int CacheManager::available() const {
  if (groups_.empty()) return 0;
  int least = groups_[0].pool->available();
  for (const Group& g : groups_) least = std::min(least, g.pool->available());
  return least;
}

int CacheManager::capacity_tokens() const {
  if (groups_.empty()) return 0;
  int least = groups_[0].pool->num_pages();
  for (const Group& g : groups_) least = std::min(least, g.pool->num_pages());
  return least * page_size_;
}

int CacheManager::cached_prefix_tokens(const std::vector<PageHash>& chain) const {
  if (!prefix_sharing_ || groups_.empty()) return 0;
  size_t least = chain.size();
  for (const Group& g : groups_) least = std::min(least, g.pool->match(chain).size());
  return (int)least * page_size_;
}

int CacheManager::leaked_pages() const {
  int total = 0;
  for (const Group& g : groups_) total += g.pool->num_pages() - g.pool->available();
  return total;
}

const Sequence& CacheManager::sequence(const std::string& key) const {
  auto it = sequences_.find(key);
  if (it == sequences_.end()) throw UnknownSequence(key);
  return it->second;
}

Sequence& CacheManager::mutable_sequence(const std::string& key) {
  auto it = sequences_.find(key);
  if (it == sequences_.end()) throw UnknownSequence(key);
  return it->second;
}

std::vector<std::string> CacheManager::keys() const {
  std::vector<std::string> out;
  for (const auto& kv : sequences_) out.push_back(kv.first);
  return out;
}

int CacheManager::admit(const std::string& key, const std::vector<PageHash>& chain_in,
                        int num_tokens) {
  if (sequences_.count(key)) throw PoolError("'" + key + "' is already admitted");
  if (state_slots_.available() == 0) return -1;
  static const std::vector<PageHash> none;
  const std::vector<PageHash>& chain = prefix_sharing_ ? chain_in : none;
  // All all-keys groups reuse the same number of prefix pages: what the least of them holds.
  int reuse = -1;
  for (const Group& g : groups_) {
    if (g.spec.window != 0) continue;
    const int here = g.pool->reusable(chain, num_tokens);
    reuse = reuse < 0 ? here : std::min(reuse, here);
  }
  Sequence seq;
  seq.tables.resize(groups_.size());
  seq.first_live.assign(groups_.size(), 0);
  std::vector<int> done;
  for (int g = 0; g < (int)groups_.size(); ++g) {
    if (groups_[g].spec.window != 0) continue;
    int cached = 0;
    if (!groups_[g].pool->reserve(chain, num_tokens, reuse, seq.tables[g], cached)) {
      for (int d : done) {
        groups_[d].pool->give_back(seq.tables[d].data(), (int)seq.tables[d].size());
      }
      return -1;
    }
    seq.cached_tokens = cached;
    done.push_back(g);
  }
  seq.state_slot = state_slots_.take(key);
  seq.committed = seq.cached_tokens / page_size_;
  const int cached = seq.cached_tokens;
  sequences_.emplace(key, std::move(seq));
  return cached;
}

bool CacheManager::grow(const std::string& key, int start, int new_len) {
  Sequence& seq = mutable_sequence(key);
  const int want = (new_len + page_size_ - 1) / page_size_;
  std::vector<std::pair<int, int>> added;      // (group, page)
  struct Skipped { int group, old_size, old_first; };
  std::vector<Skipped> skipped;
  bool ok = true;
  for (int g = 0; g < (int)groups_.size() && ok; ++g) {
    std::vector<int>& table = seq.tables[g];
    const GroupSpec& spec = groups_[g].spec;
    if (spec.window != 0 && (int)table.size() < want) {
      // Pages wholly before the window of the first new query are never read.
      const int skip_to = std::min(first_needed(spec, start) / page_size_, want);
      skipped.push_back({g, (int)table.size(), seq.first_live[g]});
      while ((int)table.size() < skip_to) table.push_back(-1);
      seq.first_live[g] = std::max(seq.first_live[g], std::min(skip_to, (int)table.size()));
    }
    while ((int)table.size() < want) {
      const int page = groups_[g].pool->take();
      if (page < 0) {
        ok = false;
        break;
      }
      table.push_back(page);
      added.emplace_back(g, page);
    }
  }
  if (ok) return true;
  for (auto it = added.rbegin(); it != added.rend(); ++it) {
    seq.tables[it->first].pop_back();
    groups_[it->first].pool->give_back(&it->second, 1);
  }
  for (auto it = skipped.rbegin(); it != skipped.rend(); ++it) {
    seq.tables[it->group].resize((size_t)it->old_size);
    seq.first_live[it->group] = it->old_first;
  }
  return false;
}

int CacheManager::trim(const std::string& key, int num_computed) {
  Sequence& seq = mutable_sequence(key);
  int freed = 0;
  for (int g = 0; g < (int)groups_.size(); ++g) {
    const GroupSpec& spec = groups_[g].spec;
    if (spec.window == 0) continue;
    std::vector<int>& table = seq.tables[g];
    const int keep_from = std::min(first_needed(spec, num_computed) / page_size_, (int)table.size());
    for (int index = seq.first_live[g]; index < keep_from; ++index) {
      if (table[index] >= 0) {
        groups_[g].pool->give_back(&table[index], 1);
        table[index] = -1;
        ++freed;
      }
    }
    seq.first_live[g] = std::max(seq.first_live[g], keep_from);
  }
  return freed;
}

void CacheManager::commit(const std::string& key, const std::vector<PageHash>& chain,
                          int full_pages) {
  Sequence& seq = mutable_sequence(key);
  if (!prefix_sharing_ || full_pages <= seq.committed) return;
  for (int g = 0; g < (int)groups_.size(); ++g) {
    const std::vector<int>& table = seq.tables[g];
    const int stop = std::min({full_pages, (int)table.size(), (int)chain.size()});
    for (int index = seq.committed; index < stop; ++index) {
      groups_[g].pool->publish(table[index], chain[index]);
    }
  }
  seq.committed = full_pages;
}

void CacheManager::release(const std::string& key) {
  auto it = sequences_.find(key);
  if (it == sequences_.end()) throw UnknownSequence(key);
  for (int g = 0; g < (int)groups_.size(); ++g) {
    std::vector<int> live;
    for (int page : it->second.tables[g]) {
      if (page >= 0) live.push_back(page);
    }
    groups_[g].pool->give_back(live.data(), (int)live.size());
  }
  sequences_.erase(it);
  state_slots_.give(key);
}

void CacheManager::audit() const {
  for (int g = 0; g < (int)groups_.size(); ++g) {
    const PagePool& pool = *groups_[g].pool;
    pool.audit();
    std::vector<int> in_tables((size_t)pool.num_pages(), 0);
    for (const auto& kv : sequences_) {
      for (int page : kv.second.tables[g]) {
        if (page >= 0) ++in_tables[page];
      }
    }
    for (int p = 0; p < pool.num_pages(); ++p) {
      if (in_tables[p] != pool.holders(p)) {
        throw PoolError("group " + std::to_string(g) + ": page " + std::to_string(p) + " is in " +
                        std::to_string(in_tables[p]) + " tables but has " +
                        std::to_string(pool.holders(p)) + " holders");
      }
      if (in_tables[p] > 1 && !pool.hashed(p)) {
        throw PoolError("group " + std::to_string(g) + ": unhashed page " + std::to_string(p) +
                        " is shared");
      }
    }
  }
  state_slots_.audit();
  for (const auto& kv : sequences_) {
    if (state_slots_.slot_of(kv.first) != kv.second.state_slot) {
      throw PoolError("'" + kv.first + "' and the slot pool disagree about its state slot");
    }
  }
}

}  // namespace mercury
