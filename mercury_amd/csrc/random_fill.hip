// Random weights drawn on the device: element i of a tensor is mean + std * normal(key, i),
// the same float32 value the host core computes for (key, i), rounded to the storage dtype.
#include "common.h"
#include "mercury_kernels.h"
#include "random_normal.h"

template <typename T>
__global__ void fill_normal_kernel(T* __restrict__ out, long long n, unsigned long long key,
                                   float mean, float std) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const float v = mk_normal_scaled(key, (uint64_t)i, mean, std);
    if constexpr (sizeof(T) == 2) {
      out[i] = mk_round_bf16(v);
    } else {
      out[i] = v;
    }
  }
}

extern "C" int mk_fill_normal(void* out, int dtype, long long n, unsigned long long key,
                              float mean, float std, hipStream_t stream) {
  MK_REQUIRE(out != nullptr || n == 0, "fill_normal: null output");
  MK_REQUIRE(n >= 0, "fill_normal: negative count");
  MK_REQUIRE(dtype == MK_F32 || dtype == MK_BF16, "fill_normal: dtype code %d", dtype);
  if (n == 0) return 0;
  const int threads = 256;
  long long blocks = (n + threads - 1) / threads;
  if (blocks > 256 * 32) blocks = 256 * 32;
  if (dtype == MK_BF16) {
    fill_normal_kernel<bf16_t><<<(int)blocks, threads, 0, stream>>>((bf16_t*)out, n, key, mean, std);
  } else {
    fill_normal_kernel<float><<<(int)blocks, threads, 0, stream>>>((float*)out, n, key, mean, std);
  }
  MK_LAUNCH_CHECK("fill_normal");
  return 0;
}
