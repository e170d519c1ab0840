// Chain hashes of full pages of tokens: the keys under which the page pool finds a prefix
// that an earlier request left in the cache.
//
// h_i = H(h_{i-1}, tokens of page i), h_{-1} = 0, over full pages only, so one hash names the
// whole prefix that ends with its page (reference: mercury/hashing.py:19-46, whose default is
// Python's per-process hash and whose strong mode is SHA-256 cut to 128 bits).  The fast mode
// here is a 64-bit multiply-xorshift chain, the same in every process and run; the strong mode
// is SHA-256 over (parent as 16 bytes, tokens as 8-byte integers, all little-endian), of which
// the first 128 bits are kept.
#pragma once

#include <cstddef>
#include <cstdint>
#include <functional>
#include <vector>

namespace mercury {

struct PageHash {
  uint64_t lo = 0, hi = 0;
  bool operator==(const PageHash& o) const { return lo == o.lo && hi == o.hi; }
  bool operator!=(const PageHash& o) const { return !(*this == o); }
};

struct PageHashHasher {
  size_t operator()(const PageHash& h) const { return (size_t)(h.lo ^ (h.hi * 0x9E3779B97F4A7C15ull)); }
};

class PageHasher {
 public:
  PageHasher(int page_size, bool strong) : page_size_(page_size), strong_(strong) {}
  int page_size() const { return page_size_; }
  bool strong() const { return strong_; }

  PageHash page(const PageHash& parent, const int32_t* tokens, int count) const;
  // Grows `chain` to cover every full page of tokens[0, count); returns the pages added.
  int extend(std::vector<PageHash>& chain, const int32_t* tokens, size_t count) const;
  std::vector<PageHash> chain(const int32_t* tokens, size_t count) const {
    std::vector<PageHash> out;
    extend(out, tokens, count);
    return out;
  }

 private:
  int page_size_;
  bool strong_;
};

// SHA-256 of a byte string (FIPS 180-4); 32 bytes out.
void sha256(const uint8_t* data, size_t size, uint8_t out[32]);

}  // namespace mercury
