#pragma once

#include <cstdint>

namespace mercury {

// out[i] = mean + std * normal(key, i) for i < count, float32 (dtype 0) or rounded to
// bfloat16 (dtype 1).
void fill_normal(void* out, int dtype, int64_t count, uint64_t key, float mean, float std);

}  // namespace mercury
