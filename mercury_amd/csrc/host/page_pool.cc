#include "page_pool.h"

#include <algorithm>

namespace mercury {

PagePool::PagePool(int num_pages, int page_size) : page_size_(page_size) {
  if (num_pages <= 0) throw std::invalid_argument("num_pages must be positive");
  if (page_size <= 0) throw std::invalid_argument("page_size must be positive");
  pages_.resize((size_t)num_pages);
  for (int p = 0; p < num_pages; ++p) push_back(free_, FREE, p);
}

void PagePool::push_back(List& list, Where where, int page) {
  Page& r = pages_[page];
  r.where = where;
  r.prev = list.tail;
  r.next = -1;
  if (list.tail >= 0) pages_[list.tail].next = page; else list.head = page;
  list.tail = page;
  ++list.count;
}

void PagePool::unlink(List& list, int page) {
  Page& r = pages_[page];
  if (r.prev >= 0) pages_[r.prev].next = r.next; else list.head = r.next;
  if (r.next >= 0) pages_[r.next].prev = r.prev; else list.tail = r.prev;
  r.prev = r.next = -1;
  r.where = HELD;
  --list.count;
}

std::vector<int> PagePool::order(const List& list) const {
  std::vector<int> out;
  out.reserve((size_t)list.count);
  for (int p = list.head; p >= 0; p = pages_[p].next) out.push_back(p);
  return out;
}

int PagePool::page_for(const PageHash& h) const {
  auto it = index_.find(h);
  return it == index_.end() ? -1 : it->second;
}

std::vector<int> PagePool::match(const std::vector<PageHash>& chain) const {
  std::vector<int> out;
  for (const PageHash& h : chain) {
    const int page = page_for(h);
    if (page < 0) break;
    out.push_back(page);
  }
  return out;
}

int PagePool::reusable(const std::vector<PageHash>& chain, int num_tokens, int cap) const {
  int limit = (num_tokens - 1) / page_size_;
  if (cap >= 0) limit = std::min(limit, cap);
  int n = 0;
  while (n < limit && n < (int)chain.size() && page_for(chain[n]) >= 0) ++n;
  return n;
}

int PagePool::recycle() {
  if (free_.head >= 0) {
    const int page = free_.head;
    unlink(free_, page);
    return page;
  }
  const int page = idle_.head;
  unlink(idle_, page);
  Page& r = pages_[page];
  index_.erase(r.hash);
  r.hashed = false;
  r.hash = PageHash();
  ++stats_.evictions;
  return page;
}

bool PagePool::reserve(const std::vector<PageHash>& chain, int num_tokens, int cap,
                       std::vector<int>& pages_out, int& reused_tokens) {
  const int reuse = reusable(chain, num_tokens, cap);
  const int total = (num_tokens + page_size_ - 1) / page_size_;
  const int fresh = total - reuse;
  // Reused pages that are idle now stop being available once they are held.
  int pinned = 0;
  for (int i = 0; i < reuse; ++i) pinned += pages_[page_for(chain[i])].holders == 0;
  if (fresh > available() - pinned) {
    ++stats_.allocation_failures;
    return false;
  }
  pages_out.clear();
  pages_out.reserve((size_t)total);
  for (int i = 0; i < reuse; ++i) {
    const int page = page_for(chain[i]);
    Page& r = pages_[page];
    if (r.holders == 0) unlink(idle_, page);
    ++r.holders;
    pages_out.push_back(page);
  }
  for (int i = 0; i < fresh; ++i) {
    const int page = recycle();
    pages_[page].holders = 1;
    pages_out.push_back(page);
  }
  reused_tokens = reuse * page_size_;
  stats_.hit_tokens += reused_tokens;
  stats_.query_tokens += num_tokens;
  ++stats_.prefills;
  return true;
}

int PagePool::take() {
  if (available() == 0) return -1;
  const int page = recycle();
  pages_[page].holders = 1;
  return page;
}

void PagePool::publish(int page, const PageHash& h) {
  Page& r = pages_.at((size_t)page);
  if (r.hashed || index_.count(h)) return;
  r.hashed = true;
  r.hash = h;
  index_.emplace(h, page);
}

void PagePool::give_back(const int* pages, int count) {
  for (int i = count - 1; i >= 0; --i) {
    const int page = pages[i];
    if (page < 0 || page >= num_pages()) throw PoolError("page " + std::to_string(page) + " does not exist");
    Page& r = pages_[page];
    if (r.holders <= 0) {
      throw PoolError("page " + std::to_string(page) + " is given back but nobody holds it");
    }
    if (--r.holders == 0) push_back(r.hashed ? idle_ : free_, r.hashed ? IDLE : FREE, page);
  }
}

void PagePool::audit() const {
  std::vector<uint8_t> seen((size_t)num_pages(), 0);
  auto walk = [&](const List& list, Where where, const char* name) {
    int count = 0, prev = -1;
    for (int p = list.head; p >= 0; p = pages_[p].next) {
      if (seen[p]) throw PoolError(std::string("page ") + std::to_string(p) + " is queued twice");
      seen[p] = 1;
      if (pages_[p].where != where || pages_[p].prev != prev) {
        throw PoolError(std::string("the ") + name + " queue is broken at page " + std::to_string(p));
      }
      prev = p;
      if (++count > num_pages()) throw PoolError(std::string("the ") + name + " queue has a cycle");
    }
    if (count != list.count || prev != list.tail) {
      throw PoolError(std::string("the ") + name + " queue's count or tail is wrong");
    }
  };
  walk(free_, FREE, "free");
  walk(idle_, IDLE, "idle");
  int hashed = 0;
  for (int p = 0; p < num_pages(); ++p) {
    const Page& r = pages_[p];
    if (r.holders < 0) throw PoolError("page " + std::to_string(p) + " has a negative holder count");
    if (r.where == FREE && (r.holders || r.hashed)) {
      throw PoolError("free page " + std::to_string(p) + " is held or hashed");
    }
    if (r.where == IDLE && (r.holders || !r.hashed)) {
      throw PoolError("idle page " + std::to_string(p) + " is held or has no hash");
    }
    if (r.where == HELD && r.holders == 0) {
      throw PoolError("page " + std::to_string(p) + " has no holder but is in no queue");
    }
    if (r.where == HELD && seen[p]) throw PoolError("held page " + std::to_string(p) + " is queued");
    if (r.hashed) {
      ++hashed;
      if (page_for(r.hash) != p) throw PoolError("page " + std::to_string(p) + "'s hash maps elsewhere");
    }
  }
  if (hashed != num_indexed()) throw PoolError("the hash index names pages that carry no hash");
}

}  // namespace mercury
