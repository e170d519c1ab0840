// Random weights drawn on the host: the same values, bit for bit, that the device fill
// kernel computes for (key, index) (see random_normal.h).
#include "fill.h"

#include <algorithm>
#include <stdexcept>
#include <thread>
#include <vector>

#include "../random_normal.h"

namespace mercury {

void fill_normal(void* out, int dtype, int64_t count, uint64_t key, float mean, float std) {
  if (dtype != 0 && dtype != 1) throw std::invalid_argument("fill_normal: dtype code 0 or 1");
  auto work = [&](int64_t begin, int64_t end) {
    if (dtype == 1) {
      uint16_t* p = static_cast<uint16_t*>(out);
      for (int64_t i = begin; i < end; ++i) {
        p[i] = mk_round_bf16(mk_normal_scaled(key, (uint64_t)i, mean, std));
      }
    } else {
      float* p = static_cast<float*>(out);
      for (int64_t i = begin; i < end; ++i) p[i] = mk_normal_scaled(key, (uint64_t)i, mean, std);
    }
  };
  const int64_t per_thread = 1 << 20;
  const int workers = (int)std::min<int64_t>(std::max(1u, std::thread::hardware_concurrency()),
                                              (count + per_thread - 1) / per_thread);
  if (workers <= 1) {
    work(0, count);
    return;
  }
  std::vector<std::thread> threads;
  const int64_t share = (count + workers - 1) / workers;
  for (int t = 0; t < workers; ++t) {
    const int64_t begin = t * share, end = std::min(count, begin + share);
    if (begin < end) threads.emplace_back(work, begin, end);
  }
  for (auto& t : threads) t.join();
}

}  // namespace mercury
