#include "hashing.h"

#include <cmath>
#include <cstring>

namespace mercury {

namespace {

inline uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

inline uint32_t rotr(uint32_t x, int n) { return (x >> n) | (x << (32 - n)); }

// The round constants are the first 32 bits of the fractional parts of the cube roots of the
// first 64 primes, the initial state those of the square roots of the first 8: computed once
// rather than typed in.
struct Sha256Tables {
  uint32_t k[64];
  uint32_t h0[8];
  Sha256Tables() {
    int found = 0;
    for (int n = 2; found < 64; ++n) {
      bool prime = true;
      for (int d = 2; d * d <= n; ++d) {
        if (n % d == 0) {
          prime = false;
          break;
        }
      }
      if (!prime) continue;
      const long double c = cbrtl((long double)n);
      k[found] = (uint32_t)((c - floorl(c)) * 4294967296.0L);
      if (found < 8) {
        const long double s = sqrtl((long double)n);
        h0[found] = (uint32_t)((s - floorl(s)) * 4294967296.0L);
      }
      ++found;
    }
  }
};

const Sha256Tables& tables() {
  static const Sha256Tables t;
  return t;
}

void sha256_block(uint32_t state[8], const uint8_t block[64]) {
  const uint32_t* k = tables().k;
  uint32_t w[64];
  for (int i = 0; i < 16; ++i) {
    w[i] = ((uint32_t)block[4 * i] << 24) | ((uint32_t)block[4 * i + 1] << 16) |
           ((uint32_t)block[4 * i + 2] << 8) | (uint32_t)block[4 * i + 3];
  }
  for (int i = 16; i < 64; ++i) {
    const uint32_t s0 = rotr(w[i - 15], 7) ^ rotr(w[i - 15], 18) ^ (w[i - 15] >> 3);
    const uint32_t s1 = rotr(w[i - 2], 17) ^ rotr(w[i - 2], 19) ^ (w[i - 2] >> 10);
    w[i] = w[i - 16] + s0 + w[i - 7] + s1;
  }
  uint32_t a = state[0], b = state[1], c = state[2], d = state[3];
  uint32_t e = state[4], f = state[5], g = state[6], h = state[7];
  for (int i = 0; i < 64; ++i) {
    const uint32_t s1 = rotr(e, 6) ^ rotr(e, 11) ^ rotr(e, 25);
    const uint32_t ch = (e & f) ^ (~e & g);
    const uint32_t t1 = h + s1 + ch + k[i] + w[i];
    const uint32_t s0 = rotr(a, 2) ^ rotr(a, 13) ^ rotr(a, 22);
    const uint32_t maj = (a & b) ^ (a & c) ^ (b & c);
    const uint32_t t2 = s0 + maj;
    h = g; g = f; f = e; e = d + t1;
    d = c; c = b; b = a; a = t1 + t2;
  }
  state[0] += a; state[1] += b; state[2] += c; state[3] += d;
  state[4] += e; state[5] += f; state[6] += g; state[7] += h;
}

}  // namespace

void sha256(const uint8_t* data, size_t size, uint8_t out[32]) {
  uint32_t state[8];
  std::memcpy(state, tables().h0, sizeof(state));
  size_t done = 0;
  for (; done + 64 <= size; done += 64) sha256_block(state, data + done);
  uint8_t tail[128] = {0};
  const size_t rest = size - done;
  std::memcpy(tail, data + done, rest);
  tail[rest] = 0x80;
  const size_t padded = rest + 9 <= 64 ? 64 : 128;
  const uint64_t bits = (uint64_t)size * 8;
  for (int i = 0; i < 8; ++i) tail[padded - 1 - i] = (uint8_t)(bits >> (8 * i));
  sha256_block(state, tail);
  if (padded == 128) sha256_block(state, tail + 64);
  for (int i = 0; i < 8; ++i) {
    out[4 * i] = (uint8_t)(state[i] >> 24);
    out[4 * i + 1] = (uint8_t)(state[i] >> 16);
    out[4 * i + 2] = (uint8_t)(state[i] >> 8);
    out[4 * i + 3] = (uint8_t)state[i];
  }
}

PageHash PageHasher::page(const PageHash& parent, const int32_t* tokens, int count) const {
  PageHash out;
  if (!strong_) {
    uint64_t h = mix64(parent.lo ^ 0x6D65726375727921ull);
    for (int i = 0; i < count; ++i) {
      h = mix64(h ^ ((uint64_t)(uint32_t)tokens[i] + ((uint64_t)(i + 1) << 32)));
    }
    out.lo = h ? h : 1;   // 0 is the chain's start
    return out;
  }
  std::vector<uint8_t> payload(16 + 8 * (size_t)count);
  for (int i = 0; i < 8; ++i) {
    payload[i] = (uint8_t)(parent.lo >> (8 * i));
    payload[8 + i] = (uint8_t)(parent.hi >> (8 * i));
  }
  for (int t = 0; t < count; ++t) {
    const int64_t v = tokens[t];
    for (int i = 0; i < 8; ++i) payload[16 + 8 * t + i] = (uint8_t)((uint64_t)v >> (8 * i));
  }
  uint8_t digest[32];
  sha256(payload.data(), payload.size(), digest);
  for (int i = 0; i < 8; ++i) {
    out.lo |= (uint64_t)digest[i] << (8 * i);
    out.hi |= (uint64_t)digest[8 + i] << (8 * i);
  }
  return out;
}

int PageHasher::extend(std::vector<PageHash>& chain, const int32_t* tokens, size_t count) const {
  const size_t full = count / (size_t)page_size_;
  PageHash parent = chain.empty() ? PageHash{} : chain.back();
  int added = 0;
  for (size_t index = chain.size(); index < full; ++index) {
    parent = page(parent, tokens + index * (size_t)page_size_, page_size_);
    chain.push_back(parent);
    ++added;
  }
  return added;
}

}  // namespace mercury
