// Sampling over float32 logits [rows, V]: argmax, and temperature / nucleus sampling by
// inverse CDF from one uniform number per row.
//
// Rule (reference: mercury/sampling.py:17-35): a row with temperature <= 0 takes the argmax
// of its raw logits (lowest index among equals).  Otherwise p = softmax(logits /
// max(temperature, 1e-5)) in float32; with top_p < 1 the tokens are kept whose preceding
// probability mass, in descending order of probability, does not exceed top_p (so the token
// that crosses top_p stays); the kept probabilities are renormalised and one token is drawn.
// The reference draws with a generator shared by the whole batch; here the caller passes a
// uniform number u in [0, 1) per row and the token is the first, in index order, whose
// inclusive cumulative kept mass exceeds u * total.  Equal probabilities at the nucleus
// edge are kept together.
#include "common.h"
#include "mercury_kernels.h"

#define SP_THREADS 1024

struct MaxIdx {
  float v;
  int i;
};

__device__ __forceinline__ MaxIdx better(MaxIdx a, MaxIdx b) {
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__device__ MaxIdx block_argmax(const float* row, int vocab, MaxIdx* scratch) {
  MaxIdx best = {-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float v = row[i];
    // NaN never wins; an all-NaN row resolves to index 0 below.
    if (v > best.v || (v == best.v && i < best.i)) best = {v, i};
  }
#pragma unroll
  for (int m = MK_WAVE / 2; m > 0; m >>= 1) {
    MaxIdx o = {__shfl_xor(best.v, m, MK_WAVE), __shfl_xor(best.i, m, MK_WAVE)};
    best = better(best, o);
  }
  const int lane = threadIdx.x & (MK_WAVE - 1), wave = threadIdx.x / MK_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = best;
  __syncthreads();
  MaxIdx total = scratch[0];
  for (int w = 1; w < (int)(blockDim.x / MK_WAVE); ++w) total = better(total, scratch[w]);
  if (total.i == 0x7fffffff) total.i = 0;
  return total;
}

__global__ __launch_bounds__(SP_THREADS) void argmax_kernel(const float* __restrict__ logits,
                                                            int vocab, long long row_stride,
                                                            int* __restrict__ out) {
  __shared__ MaxIdx scratch[SP_THREADS / MK_WAVE];
  const MaxIdx best = block_argmax(logits + (size_t)blockIdx.x * row_stride, vocab, scratch);
  if (threadIdx.x == 0) out[blockIdx.x] = best.i;
}

// Two stages for few rows of a large vocabulary: ARGMAX_PARTS workgroups per row each take a
// stretch of the row, then one wavefront per row picks among their results (lowest index
// among equals, as in the single-stage kernel).
#define ARGMAX_PARTS 64

__global__ __launch_bounds__(256) void argmax_part_kernel(const float* __restrict__ logits,
                                                          int vocab, long long row_stride,
                                                          MaxIdx* __restrict__ parts) {
  __shared__ MaxIdx scratch[256 / MK_WAVE];
  const int row = blockIdx.y, part = blockIdx.x;
  const int per = (vocab + ARGMAX_PARTS - 1) / ARGMAX_PARTS;
  const int begin = min(vocab, part * per), count = min(vocab, begin + per) - begin;
  MaxIdx best = block_argmax(logits + (size_t)row * row_stride + begin, count, scratch);
  best.i = count > 0 ? best.i + begin : 0x7fffffff;
  if (count <= 0) best.v = -INFINITY;
  if (threadIdx.x == 0) parts[row * ARGMAX_PARTS + part] = best;
}

__global__ __launch_bounds__(MK_WAVE) void argmax_pick_kernel(const MaxIdx* __restrict__ parts,
                                                              int* __restrict__ out) {
  MaxIdx best = parts[blockIdx.x * ARGMAX_PARTS + threadIdx.x];
#pragma unroll
  for (int m = MK_WAVE / 2; m > 0; m >>= 1) {
    MaxIdx o = {__shfl_xor(best.v, m, MK_WAVE), __shfl_xor(best.i, m, MK_WAVE)};
    best = better(best, o);
  }
  if (threadIdx.x == 0) out[blockIdx.x] = best.i == 0x7fffffff ? 0 : best.i;
}

extern "C" int mk_argmax(const float* logits, int rows, int vocab, long long row_stride,
                         int* out, void* parts, hipStream_t stream) {
  MK_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab, "argmax: bad sizes");
  if (rows == 0) return 0;
  if (parts != nullptr && rows <= 256 && vocab >= 16384) {
    static_assert(ARGMAX_PARTS == MK_WAVE, "the pick kernel reads one part per lane");
    argmax_part_kernel<<<dim3(ARGMAX_PARTS, rows), 256, 0, stream>>>(logits, vocab, row_stride,
                                                                      (MaxIdx*)parts);
    argmax_pick_kernel<<<rows, MK_WAVE, 0, stream>>>((const MaxIdx*)parts, out);
  } else {
    argmax_kernel<<<rows, SP_THREADS, 0, stream>>>(logits, vocab, row_stride, out);
  }
  MK_LAUNCH_CHECK("argmax");
  return 0;
}

// Mass of the probabilities strictly above the threshold.
__device__ float mass_above(const float* probs, int vocab, float threshold, float* scratch) {
  float s = 0.f;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float p = probs[i];
    if (p > threshold) s += p;
  }
  return block_sum(s, scratch);
}

__global__ __launch_bounds__(SP_THREADS) void sample_kernel(
    const float* __restrict__ logits, int vocab, long long row_stride,
    const float* __restrict__ temperatures, const float* __restrict__ top_ps,
    const float* __restrict__ uniforms, float* __restrict__ probs_all, int* __restrict__ out) {
  __shared__ MaxIdx mi_scratch[SP_THREADS / MK_WAVE];
  __shared__ float scratch[SP_THREADS / MK_WAVE];
  __shared__ float chunk_sum[SP_THREADS];
  __shared__ int chosen;
  const int r = blockIdx.x;
  const float* row = logits + (size_t)r * row_stride;
  float* probs = probs_all + (size_t)r * vocab;
  const float temperature = temperatures[r];

  const MaxIdx best = block_argmax(row, vocab, mi_scratch);
  if (temperature <= 0.f) {
    if (threadIdx.x == 0) out[r] = best.i;
    return;
  }
  const float inv_t = 1.f / fmaxf(temperature, 1e-5f);

  // softmax of the scaled logits; the maximum of the scaled row is at the argmax.
  const float top = best.v * inv_t;
  float z = 0.f;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float e = expf(row[i] * inv_t - top);
    probs[i] = e;
    z += e;
  }
  z = block_sum(z, scratch);
  const float inv_z = 1.f / z;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) probs[i] *= inv_z;
  __syncthreads();

  // The smallest kept probability: the least v with mass_above(v) <= top_p, found by
  // bisection over the bit patterns of non-negative floats (monotone in value).
  float keep_from = 0.f;
  const float top_p = top_ps[r];
  if (top_p < 1.f) {
    unsigned lo = 0u, hi = __float_as_uint(inv_z);  // exp(0) / z is the largest probability
    while (lo < hi) {
      const unsigned mid = lo + (hi - lo) / 2u;
      if (mass_above(probs, vocab, __uint_as_float(mid), scratch) <= top_p)
        hi = mid;
      else
        lo = mid + 1u;
    }
    keep_from = __uint_as_float(lo);
  }

  // Inverse CDF in index order: each thread owns one contiguous chunk.
  const int per = (vocab + blockDim.x - 1) / blockDim.x;
  const int begin = min(vocab, (int)threadIdx.x * per), end = min(vocab, begin + per);
  float mine = 0.f;
  for (int i = begin; i < end; ++i) {
    const float p = probs[i];
    if (p >= keep_from) mine += p;
  }
  chunk_sum[threadIdx.x] = mine;
  if (threadIdx.x == 0) chosen = -1;
  __syncthreads();
  if (threadIdx.x == 0) {
    float total = 0.f;
    for (int c = 0; c < (int)blockDim.x; ++c) total += chunk_sum[c];
    const float target = uniforms[r] * total;
    float running = 0.f;
    int c = 0;
    for (; c < (int)blockDim.x; ++c) {
      if (running + chunk_sum[c] > target) break;
      running += chunk_sum[c];
    }
    if (c == (int)blockDim.x) {
      // u * total rounded up to the total: take the last kept token.
      for (c = blockDim.x - 1; c > 0 && chunk_sum[c] == 0.f; --c) {}
      running = -1.f;
    }
    const int cb = min(vocab, c * per), ce = min(vocab, cb + per);
    int pick = -1, last_kept = -1;
    for (int i = cb; i < ce; ++i) {
      const float p = probs[i];
      if (p < keep_from) continue;
      last_kept = i;
      if (running >= 0.f) {
        running += p;
        if (running > target) {
          pick = i;
          break;
        }
      }
    }
    chosen = pick >= 0 ? pick : (last_kept >= 0 ? last_kept : best.i);
  }
  __syncthreads();
  if (threadIdx.x == 0) out[r] = chosen;
}

extern "C" int mk_sample(const float* logits, int rows, int vocab, long long row_stride,
                         const float* temperatures, const float* top_ps, const float* uniforms,
                         float* probs_scratch, int* out, hipStream_t stream) {
  MK_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab, "sample: bad sizes");
  MK_REQUIRE(probs_scratch != nullptr, "sample: needs a [rows, V] float32 scratch buffer");
  if (rows == 0) return 0;
  sample_kernel<<<rows, SP_THREADS, 0, stream>>>(logits, vocab, row_stride, temperatures, top_ps,
                                                 uniforms, probs_scratch, out);
  MK_LAUNCH_CHECK("sample");
  return 0;
}
