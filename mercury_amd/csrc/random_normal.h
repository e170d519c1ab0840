// Random weights that are the same numbers on the host and on the GPU.
//
// Element i of a tensor is a function of (key, i) alone: a counter-based bit mixer gives 48
// bits, a Box-Muller transform turns them into a normal deviate.  The logarithm, the cosine
// and the root are written out here with float32 additions, multiplications and divisions
// only (each correctly rounded, none contracted into a fused multiply-add), and the IEEE root,
// so that g++ on the host and hipcc on the device compute bit-identical values; libm and the
// device's math library would not agree.  The result is rounded to bfloat16 with the same
// integer code on both sides.  This file is included by the kernel library (device fill) and
// by the host core (host fill, what a written model folder holds).
#pragma once

#include <math.h>
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define MK_HOST_DEVICE __host__ __device__
#else
#define MK_HOST_DEVICE
#endif

// A 64-bit finaliser of the multiply-xorshift kind; `z` counts, the result is white.
MK_HOST_DEVICE static inline uint64_t mk_mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

MK_HOST_DEVICE static inline float mk_bits_to_float(uint32_t u) {
  float f;
  memcpy(&f, &u, sizeof(f));
  return f;
}

MK_HOST_DEVICE static inline uint32_t mk_float_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, sizeof(u));
  return u;
}

// Round to nearest even; the inputs here are finite.
MK_HOST_DEVICE static inline uint16_t mk_round_bf16(float f) {
  uint32_t u = mk_float_to_bits(f);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// ln(u) for u = (a + 1) / 2^24, a < 2^24: exponent and mantissa taken apart, the mantissa m
// brought into [1/sqrt 2, sqrt 2), ln m = 2 atanh((m - 1) / (m + 1)) by its series.
MK_HOST_DEVICE static inline float mk_ln_unit(uint32_t a) {
#if defined(__clang__)
#pragma clang fp contract(off)
#endif
  const float u = (float)(a + 1u) * 5.9604644775390625e-08f;   // exact: 24 bits times 2^-24
  const uint32_t bits = mk_float_to_bits(u);
  int e = (int)(bits >> 23) - 127;
  float m = mk_bits_to_float((bits & 0x007FFFFFu) | 0x3F800000u);
  if (m > 1.41421356f) {
    m = m * 0.5f;
    e += 1;
  }
  const float s = (m - 1.0f) / (m + 1.0f);
  const float z = s * s;
  float p = 0.111111111f;            // 1/9
  p = p * z + 0.142857143f;          // 1/7
  p = p * z + 0.2f;
  p = p * z + 0.333333333f;
  p = p * z + 1.0f;
  const float ln_m = (2.0f * s) * p;
  return (float)e * 0.693147181f + ln_m;
}

// cos(2 pi b / 2^24) for b < 2^24: the quadrant from the top two bits, the rest folded into
// [0, pi/4] where short Taylor polynomials of sine and cosine are exact to float32.
MK_HOST_DEVICE static inline float mk_cos_turn(uint32_t b) {
#if defined(__clang__)
#pragma clang fp contract(off)
#endif
  const uint32_t quadrant = b >> 22;
  float x = (float)(b & 0x3FFFFFu) * 2.384185791015625e-07f;    // fraction of the quadrant
  bool swap = false;
  if (x > 0.5f) {
    x = 1.0f - x;
    swap = true;
  }
  const float t = x * 1.57079633f;
  const float t2 = t * t;
  float sn = 2.75573192e-06f;        // 1/9!
  sn = sn * t2 - 1.98412698e-04f;    // 1/7!
  sn = sn * t2 + 8.33333333e-03f;    // 1/5!
  sn = sn * t2 - 1.66666667e-01f;    // 1/3!
  sn = sn * t2 + 1.0f;
  sn = sn * t;
  float cs = -2.75573192e-07f;       // 1/10!
  cs = cs * t2 + 2.48015873e-05f;    // 1/8!
  cs = cs * t2 - 1.38888889e-03f;    // 1/6!
  cs = cs * t2 + 4.16666667e-02f;    // 1/4!
  cs = cs * t2 - 0.5f;
  cs = cs * t2 + 1.0f;
  const float c = swap ? sn : cs;    // cos of the angle within the quadrant
  const float s = swap ? cs : sn;
  switch (quadrant) {
    case 0: return c;
    case 1: return -s;
    case 2: return -c;
    default: return s;
  }
}

// The standard normal deviate of element `index` of the stream `key`.
MK_HOST_DEVICE static inline float mk_normal(uint64_t key, uint64_t index) {
#if defined(__clang__)
#pragma clang fp contract(off)
#endif
  const uint64_t bits = mk_mix64(key ^ mk_mix64(index));
  const uint32_t a = (uint32_t)(bits >> 40);
  const uint32_t b = (uint32_t)(bits >> 8) & 0xFFFFFFu;
  const float radius = sqrtf(-2.0f * mk_ln_unit(a));
  return radius * mk_cos_turn(b);
}

// mean + std * normal, as float32.
MK_HOST_DEVICE static inline float mk_normal_scaled(uint64_t key, uint64_t index, float mean,
                                                    float std) {
#if defined(__clang__)
#pragma clang fp contract(off)
#endif
  return mean + std * mk_normal(key, index);
}
