// Shared declarations for the gfx950 kernel library: element types, conversions, reductions
// and the host-side error channel.  Every exported function returns 0 on success and a
// non-zero code after recording a message that mk_last_error() returns.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define MK_WAVE 64

enum MkDtype { MK_F32 = 0, MK_BF16 = 1 };

typedef uint16_t bf16_t;

// ---------------------------------------------------------------------------------- errors

void mk_set_error(const char* fmt, ...);

#define MK_REQUIRE(cond, ...)      \
  do {                             \
    if (!(cond)) {                 \
      mk_set_error(__VA_ARGS__);   \
      return 1;                    \
    }                              \
  } while (0)

#define MK_LAUNCH_CHECK(name)                                             \
  do {                                                                    \
    hipError_t e_ = hipGetLastError();                                    \
    if (e_ != hipSuccess) {                                               \
      mk_set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
      return 2;                                                           \
    }                                                                     \
  } while (0)

// ------------------------------------------------------------------------------ conversions

__device__ __forceinline__ float bf16_to_f32(bf16_t x) {
  return __uint_as_float(((uint32_t)x) << 16);
}

// Round to nearest, ties to even; NaN stays NaN (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  const __bf16 b = (__bf16)f;
  return __builtin_bit_cast(bf16_t, b);
}

// Two floats rounded to bfloat16 in one 32-bit word, `a` in the low half.
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
  bf16x2_t v;
  v[0] = (__bf16)a;
  v[1] = (__bf16)b;
  return __builtin_bit_cast(uint32_t, v);
}

template <typename T>
struct Elem;

template <>
struct Elem<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};

template <>
struct Elem<bf16_t> {
  static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ void store(bf16_t* p, float v) { *p = f32_to_bf16(v); }
  static __device__ __forceinline__ float round(float v) { return bf16_to_f32(f32_to_bf16(v)); }
};

// ------------------------------------------------------- the residual stream in fixed point
//
// In steps of a few tokens the residual stream is kept as 64-bit integers in units of 2^-32
// (range +-2^31, finer than float32 from 2^-8 up): projections add their results into it with
// integer atomics, whose sum does not depend on the order they arrive in, so that partial
// results over slices of K need neither a buffer nor a kernel that adds them up, and a value
// is the same whichever workgroup finished first.
typedef long long fixed_t;

__device__ __forceinline__ fixed_t to_fixed(float y) {
  return __float2ll_rn(fminf(fmaxf(y, -1.0e9f), 1.0e9f) * 4294967296.f);
}

__device__ __forceinline__ float from_fixed(fixed_t a) {
  return __ll2float_rn(a) * 2.3283064365386963e-10f;
}

__device__ __forceinline__ void add_fixed(fixed_t* p, float y) {
  atomicAdd((unsigned long long*)p, (unsigned long long)to_fixed(y));
}

// ------------------------------------------------------------------------------- reductions

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = MK_WAVE / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, MK_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = MK_WAVE / 2; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, MK_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds at least 16 floats.  Every thread
// gets the result.  The order of additions is fixed by the thread layout alone.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (MK_WAVE - 1);
  const int wave = threadIdx.x / MK_WAVE;
  const int waves = (blockDim.x + MK_WAVE - 1) / MK_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < waves; ++w) total += scratch[w];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (MK_WAVE - 1);
  const int wave = threadIdx.x / MK_WAVE;
  const int waves = (blockDim.x + MK_WAVE - 1) / MK_WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int w = 1; w < waves; ++w) total = fmaxf(total, scratch[w]);
  return total;
}

static inline int mk_is_pow2(int x) { return x > 0 && (x & (x - 1)) == 0; }
static inline int mk_log2(int x) {
  int s = 0;
  while ((1 << s) < x) ++s;
  return s;
}
