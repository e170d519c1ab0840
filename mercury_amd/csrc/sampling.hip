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
// edge are kept together.  Every pass over a row's vocabulary is shared out over 64
// workgroups.
#include <atomic>

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

// ------------------------------------------------------ argmax for callers that cannot allocate
//
// The two-stage search above needs rows * 64 partial results between its kernels.  Here they
// live in a device array of the library's own instead of a buffer the caller brings, so that
// a caller under graph capture, or one that may not allocate at all, has a variant that
// allocates nothing.  The array's name is a host-side stand-in in host code: its device
// address is asked for once per device (with that device current) and kept; only that address
// is ever handed to a kernel.  Nothing in the array has to start at zero: each call's first
// kernel writes every part that its second kernel reads.  Every call on a GPU uses that GPU's
// one array, so two calls that overlap on one GPU (different streams) race.  The first call
// on a device asks the runtime for the address, which is a query a stream capture should not
// contain: a caller that captures calls mk_argmax_static_init() (or mk_argmax_static itself)
// once on that device beforehand.
#define ARGMAX_STATIC_MAX_ROWS 256
static __device__ __align__(256) unsigned char
    argmax_static_scratch[ARGMAX_STATIC_MAX_ROWS * ARGMAX_PARTS * sizeof(MaxIdx)];

#define ARGMAX_STATIC_MAX_DEVICES 64
// One address per device, each written once.  Threads that ask at the same time for a device
// nobody has asked for yet all get the same answer from the runtime and store the same
// value; the slots are atomic so that this is no data race.
static std::atomic<void*> g_argmax_scratch_of_device[ARGMAX_STATIC_MAX_DEVICES];

// The array's address on the current device, asked of the runtime at the first call per
// device.  0 on success.
static int argmax_static_scratch_address(void** out) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  MK_REQUIRE(e == hipSuccess, "argmax_static: hipGetDevice: %s", hipGetErrorString(e));
  MK_REQUIRE(device >= 0 && device < ARGMAX_STATIC_MAX_DEVICES, "argmax_static: device %d", device);
  void* scratch = g_argmax_scratch_of_device[device].load(std::memory_order_acquire);
  if (scratch == nullptr) {
    e = hipGetSymbolAddress(&scratch, HIP_SYMBOL(argmax_static_scratch));
    MK_REQUIRE(e == hipSuccess && scratch != nullptr, "argmax_static: hipGetSymbolAddress: %s",
               hipGetErrorString(e));
    g_argmax_scratch_of_device[device].store(scratch, std::memory_order_release);
  }
  *out = scratch;
  return 0;
}

extern "C" int mk_argmax_static_max_rows(void) { return ARGMAX_STATIC_MAX_ROWS; }

extern "C" int mk_argmax_static_init(void) {
  void* scratch = nullptr;
  return argmax_static_scratch_address(&scratch);
}

extern "C" int mk_argmax_static(const float* logits, int rows, int vocab, long long row_stride,
                                int* out, hipStream_t stream) {
  MK_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab, "argmax_static: bad sizes");
  MK_REQUIRE(rows <= ARGMAX_STATIC_MAX_ROWS,
             "argmax_static: %d rows; the library's own scratch holds at most %d (use mk_argmax "
             "with a buffer of the caller's)", rows, ARGMAX_STATIC_MAX_ROWS);
  if (rows == 0) return 0;
  void* scratch = nullptr;
  if (int code = argmax_static_scratch_address(&scratch)) return code;
  if (vocab >= 16384) {
    argmax_part_kernel<<<dim3(ARGMAX_PARTS, rows), 256, 0, stream>>>(logits, vocab, row_stride,
                                                                      (MaxIdx*)scratch);
    argmax_pick_kernel<<<rows, MK_WAVE, 0, stream>>>((const MaxIdx*)scratch, out);
  } else {
    argmax_kernel<<<rows, SP_THREADS, 0, stream>>>(logits, vocab, row_stride, out);
  }
  MK_LAUNCH_CHECK("argmax_static");
  return 0;
}

// ------------------------------------------------------------- sampling without a nucleus
//
// When no row restricts the nucleus (top_p >= 1) the draw needs no threshold search, and the
// vocabulary is shared out: SAMPLE_PARTS workgroups per row each take a stretch of it and
// report its maximum (with the index, for greedy rows) and the sum of exp(x / t - maximum);
// one workgroup per row then rescales the sums to the row's maximum, finds by their running
// total (in part order) the stretch in which u * total is crossed, and walks that stretch
// alone.  The order of every addition is fixed by the layout, not by timing.
#define SAMPLE_PARTS 64

struct SamplePart {
  float best_v;  // largest raw logit of the stretch
  int best_i;
  float m;       // largest scaled logit (x / t)
  float z;       // sum of exp(x / t - m)
};

__global__ __launch_bounds__(256) void sample_parts_kernel(const float* __restrict__ logits,
                                                           int vocab, long long row_stride,
                                                           const float* __restrict__ temperatures,
                                                           SamplePart* __restrict__ parts) {
  __shared__ MaxIdx mi_scratch[256 / MK_WAVE];
  __shared__ float scratch[16];
  const int row = blockIdx.y, part = blockIdx.x;
  const int per = (vocab + SAMPLE_PARTS - 1) / SAMPLE_PARTS;
  const int begin = min(vocab, part * per), count = min(vocab, begin + per) - begin;
  const float* x = logits + (size_t)row * row_stride + begin;
  MaxIdx best = block_argmax(x, count, mi_scratch);
  SamplePart out;
  out.best_v = count > 0 ? best.v : -INFINITY;
  out.best_i = count > 0 ? best.i + begin : 0x7fffffff;
  const float t = temperatures[row];
  out.m = -INFINITY;
  out.z = 0.f;
  if (t > 0.f && count > 0) {
    const float inv_t = 1.f / fmaxf(t, 1e-5f);
    out.m = best.v * inv_t;
    float z = 0.f;
    for (int i = threadIdx.x; i < count; i += blockDim.x) z += expf(x[i] * inv_t - out.m);
    out.z = block_sum(z, scratch);
  }
  if (threadIdx.x == 0) parts[row * SAMPLE_PARTS + part] = out;
}

// The value a token weighs in a row's draw, and whether the nucleus keeps it: kept are the
// tokens whose weight's bit pattern is at least `keep_from` (weights are positive floats, so
// their patterns order as they do).
__device__ __forceinline__ float draw_weight(float x, float inv_t, float m, unsigned keep_from) {
  const float e = expf(x * inv_t - m);
  return __float_as_uint(e) >= keep_from ? e : 0.f;
}

__global__ __launch_bounds__(256) void sample_pick_kernel(const float* __restrict__ logits,
                                                          int vocab, long long row_stride,
                                                          const float* __restrict__ temperatures,
                                                          const float* __restrict__ uniforms,
                                                          const SamplePart* __restrict__ parts,
                                                          const unsigned* __restrict__ keep,
                                                          int* __restrict__ out) {
  static_assert(SAMPLE_PARTS == MK_WAVE, "one part per lane of the first wavefront");
  __shared__ float running[SAMPLE_PARTS + 1];   // mass before each part, at the row's maximum
  __shared__ float chunk_sum[256];
  __shared__ int where[2];                      // the part that holds the draw; greedy answer
  __shared__ float row_max;
  const int row = blockIdx.x, tid = threadIdx.x;
  const float t = temperatures[row];
  if (tid < MK_WAVE) {
    const SamplePart mine = parts[row * SAMPLE_PARTS + tid];
    MaxIdx best = {mine.best_v, mine.best_i};
    float m = mine.m;
#pragma unroll
    for (int k = MK_WAVE / 2; k > 0; k >>= 1) {
      MaxIdx o = {__shfl_xor(best.v, k, MK_WAVE), __shfl_xor(best.i, k, MK_WAVE)};
      best = better(best, o);
      m = fmaxf(m, __shfl_xor(m, k, MK_WAVE));
    }
    // inclusive running total of the rescaled sums, in part order
    float mass = mine.z > 0.f ? mine.z * expf(mine.m - m) : 0.f;
    float incl = mass;
#pragma unroll
    for (int k = 1; k < MK_WAVE; k <<= 1) {
      const float up = __shfl_up(incl, k, MK_WAVE);
      if (tid >= k) incl += up;
    }
    running[tid + 1] = incl;
    if (tid == 0) {
      running[0] = 0.f;
      where[1] = best.i == 0x7fffffff ? 0 : best.i;
      row_max = m;
    }
  }
  __syncthreads();
  if (t <= 0.f) {
    if (tid == 0) out[row] = where[1];
    return;
  }
  const float total = running[SAMPLE_PARTS];
  const float target = uniforms[row] * total;
  if (tid == 0) {
    // the first part whose running total passes the target; if u * total rounded up to the
    // total, the last part that holds any mass
    int c = 0;
    while (c < SAMPLE_PARTS && !(running[c + 1] > target)) ++c;
    if (c == SAMPLE_PARTS)
      for (c = SAMPLE_PARTS - 1; c > 0 && running[c + 1] == running[c]; --c) {}
    where[0] = c;
  }
  __syncthreads();
  const int c = where[0];
  const int per = (vocab + SAMPLE_PARTS - 1) / SAMPLE_PARTS;
  const int begin = min(vocab, c * per), count = min(vocab, begin + per) - begin;
  const float* x = logits + (size_t)row * row_stride + begin;
  const float inv_t = 1.f / fmaxf(t, 1e-5f), m = row_max;
  const unsigned keep_from = keep ? keep[row] : 0u;
  // every thread a contiguous chunk of the stretch, then the chunks in order
  const int each = (count + 255) / 256;
  const int lo = min(count, tid * each), hi = min(count, lo + each);
  float mine = 0.f;
  for (int i = lo; i < hi; ++i) mine += draw_weight(x[i], inv_t, m, keep_from);
  chunk_sum[tid] = mine;
  __syncthreads();
  if (tid == 0) {
    float before = running[c];
    int k = 0;
    for (; k < 256; ++k) {
      if (before + chunk_sum[k] > target) break;
      before += chunk_sum[k];
    }
    // the token that crosses the target, or, where rounding lets none cross (u * total
    // rounded up to the total; the two sums of a chunk differing), the last kept one
    if (k == 256) k = 255;
    int pick = -1, last_kept = -1;
    for (; k >= 0 && pick < 0 && last_kept < 0; --k) {
      const int klo = min(count, k * each), khi = min(count, klo + each);
      for (int i = klo; i < khi; ++i) {
        const float e = draw_weight(x[i], inv_t, m, keep_from);
        if (e <= 0.f) continue;
        last_kept = begin + i;
        before += e;
        if (before > target) {
          pick = begin + i;
          break;
        }
      }
      before = INFINITY;                      // earlier chunks only lend their last kept token
    }
    if (pick < 0) pick = last_kept >= 0 ? last_kept : where[1];
    out[row] = max(0, min(vocab - 1, pick));
  }
}

// ------------------------------------------------------------------- the nucleus, found
//
// A token is kept iff the mass of the tokens weightier than it is at most top_p of the row's
// (so the token that crosses top_p stays, and tokens of equal weight stay or go together).
// With weights e = exp(x / t - max) in (0, 1], whose float bit patterns order as the values
// do, that is: kept are the patterns >= the least pattern b with mass(patterns > b) <=
// top_p * total.  The search takes three histograms of the mass by pattern: over the upper 11
// bits, then, inside the bin found, over the next 11, then over the last 10.  Every
// workgroup gathers its stretch's histogram in LDS and adds the bins it touched to the
// row's; mass is added up as 40-bit fixed point integers, so no sum depends on the order of
// the atomic additions.
#define NUCLEUS_LEVELS 3
__device__ __host__ constexpr int nucleus_shift(int level) { return level == 0 ? 21 : (level == 1 ? 10 : 0); }
__device__ __host__ constexpr int nucleus_bins(int level) { return level == 0 ? 512 : (level == 1 ? 2048 : 1024); }
#define NUCLEUS_ROW_BINS (512 + 2048 + 1024)

struct NucleusRow {
  unsigned long long above;  // mass of the patterns above the prefix's range
  unsigned long long limit;  // top_p of the total
  unsigned prefix;           // the threshold's upper bits found so far, in place
  unsigned pad;
};

__device__ __forceinline__ unsigned long long fixed_mass(float e) {
  return (unsigned long long)((double)e * 1099511627776.0);   // 2^40
}

__global__ void zero_u64_kernel(unsigned long long* p, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x)
    p[i] = 0ull;
}

// The row's largest scaled logit, out of the parts' (every thread of the workgroup gets it).
__device__ float row_maximum(const SamplePart* parts, int row, float* shared) {
  if (threadIdx.x < MK_WAVE) {
    const float m = wave_max(parts[row * SAMPLE_PARTS + threadIdx.x].m);
    if (threadIdx.x == 0) *shared = m;
  }
  __syncthreads();
  return *shared;
}

// Mass by the LEVEL's bits of the pattern, of the tokens whose bits above them equal the
// prefix found so far.  hist: the row's bins of this level.
template <int LEVEL>
__global__ __launch_bounds__(256) void nucleus_histogram_kernel(
    const float* __restrict__ logits, int vocab, long long row_stride,
    const float* __restrict__ temperatures, const float* __restrict__ top_ps,
    const SamplePart* __restrict__ parts, const NucleusRow* __restrict__ rows,
    unsigned long long* __restrict__ hist) {
  constexpr int SHIFT = nucleus_shift(LEVEL), BINS = nucleus_bins(LEVEL);
  constexpr int ABOVE = LEVEL == 0 ? 32 : nucleus_shift(LEVEL - 1);   // bits from here up are the prefix
  __shared__ unsigned long long local[BINS];
  __shared__ float row_max;
  const int row = blockIdx.y, part = blockIdx.x;
  const float t = temperatures[row];
  if (t <= 0.f || top_ps[row] >= 1.f) return;     // greedy, or nothing to restrict
  for (int i = threadIdx.x; i < BINS; i += blockDim.x) local[i] = 0ull;
  const int per = (vocab + SAMPLE_PARTS - 1) / SAMPLE_PARTS;
  const int begin = min(vocab, part * per), count = min(vocab, begin + per) - begin;
  const float* x = logits + (size_t)row * row_stride + begin;
  const float inv_t = 1.f / fmaxf(t, 1e-5f), m = row_maximum(parts, row, &row_max);   // syncs
  const unsigned prefix = LEVEL == 0 ? 0u : rows[row].prefix;
  for (int i = threadIdx.x; i < count; i += blockDim.x) {
    const float e = expf(x[i] * inv_t - m);
    const unsigned b = __float_as_uint(e);
    if (LEVEL == 0 || (b >> ABOVE) == (prefix >> ABOVE))
      atomicAdd(&local[(b >> SHIFT) & (BINS - 1)], fixed_mass(e));
  }
  __syncthreads();
  unsigned long long* mine = hist + (size_t)row * BINS;
  for (int i = threadIdx.x; i < BINS; i += blockDim.x)
    if (local[i] != 0ull) atomicAdd(mine + i, local[i]);
}

// Walk a level's histogram from its top: the least bin with mass(bins above it) + what lies
// above the prefix's range <= limit.  One workgroup per row; thread k sums bins
// [k * EACH, (k + 1) * EACH), the first thread then walks the sums and the bins of one.
template <int LEVEL>
__global__ __launch_bounds__(256) void nucleus_pick_kernel(
    const float* __restrict__ temperatures, const float* __restrict__ top_ps,
    const unsigned long long* __restrict__ hist, NucleusRow* __restrict__ rows,
    unsigned* __restrict__ keep) {
  constexpr int BINS = nucleus_bins(LEVEL), EACH = BINS / 256, SHIFT = nucleus_shift(LEVEL);
  __shared__ unsigned long long chunk[256];
  const int row = blockIdx.x, tid = threadIdx.x;
  if (temperatures[row] <= 0.f || top_ps[row] >= 1.f) {
    if (LEVEL == NUCLEUS_LEVELS - 1 && tid == 0) keep[row] = 0u;   // everything is kept
    return;
  }
  const unsigned long long* bins = hist + (size_t)row * BINS;
  unsigned long long sum = 0ull;
  for (int i = 0; i < EACH; ++i) sum += bins[tid * EACH + i];
  chunk[tid] = sum;
  __syncthreads();
  if (tid != 0) return;
  unsigned long long above, limit;
  if (LEVEL == 0) {
    unsigned long long total = 0ull;
    for (int k = 0; k < 256; ++k) total += chunk[k];
    above = 0ull;
    limit = (unsigned long long)((double)top_ps[row] * (double)total);
  } else {
    above = rows[row].above;
    limit = rows[row].limit;
  }
  // `above` never passes the limit: the bin it belongs to is a valid threshold.  Down the
  // chunks while a whole chunk still fits, then down the bins of the chunk that does not.
  int k = 255;
  while (k > 0 && above + chunk[k] <= limit) above += chunk[k--];
  int i = EACH - 1;
  while (i > 0 && above + bins[k * EACH + i] <= limit) above += bins[k * EACH + i--];
  const unsigned found = (unsigned)(k * EACH + i);
  const unsigned prefix = (LEVEL == 0 ? 0u : rows[row].prefix) | (found << SHIFT);
  rows[row].above = above;
  rows[row].limit = limit;
  rows[row].prefix = prefix;
  if (LEVEL == NUCLEUS_LEVELS - 1) keep[row] = prefix;
}

// The parts again, for the draw, into a second array: the row's maximum for every part, and
// the kept mass only.
__global__ __launch_bounds__(256) void nucleus_parts_kernel(const float* __restrict__ logits,
                                                            int vocab, long long row_stride,
                                                            const float* __restrict__ temperatures,
                                                            const unsigned* __restrict__ keep,
                                                            const SamplePart* __restrict__ parts,
                                                            SamplePart* __restrict__ kept) {
  __shared__ float scratch[16];
  __shared__ float row_max;
  const int row = blockIdx.y, part = blockIdx.x;
  SamplePart out = parts[row * SAMPLE_PARTS + part];
  out.z = 0.f;
  const float t = temperatures[row];
  if (t > 0.f) {   // the same for every thread of the workgroup
    const float m = row_maximum(parts, row, &row_max);
    const int per = (vocab + SAMPLE_PARTS - 1) / SAMPLE_PARTS;
    const int begin = min(vocab, part * per), count = min(vocab, begin + per) - begin;
    const float* x = logits + (size_t)row * row_stride + begin;
    const float inv_t = 1.f / fmaxf(t, 1e-5f);
    const unsigned keep_from = keep[row];
    float z = 0.f;
    for (int i = threadIdx.x; i < count; i += blockDim.x) z += draw_weight(x[i], inv_t, m, keep_from);
    out.z = block_sum(z, scratch);
    out.m = m;
  }
  if (threadIdx.x == 0) kept[row * SAMPLE_PARTS + part] = out;
}

static size_t align_up(size_t n) { return (n + 255) / 256 * 256; }

// Bytes of scratch mk_sample needs for `rows` rows: the parts alone without a nucleus, else
// the parts twice, the rows' search records and thresholds, and the two histograms.
extern "C" long long mk_sample_scratch_bytes(int rows, int nucleus) {
  const size_t parts = align_up((size_t)rows * SAMPLE_PARTS * sizeof(SamplePart));
  if (!nucleus) return (long long)parts;
  return (long long)(2 * parts + align_up((size_t)rows * sizeof(NucleusRow)) +
                     align_up((size_t)rows * sizeof(unsigned)) +
                     (size_t)rows * NUCLEUS_ROW_BINS * 8);
}

extern "C" int mk_sample(const float* logits, int rows, int vocab, long long row_stride,
                         const float* temperatures, const float* top_ps, const float* uniforms,
                         void* scratch, int* out, hipStream_t stream) {
  MK_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab, "sample: bad sizes");
  if (rows == 0) return 0;
  MK_REQUIRE(scratch != nullptr && rows <= 65535,
             "sample: needs its scratch buffer (mk_sample_scratch_bytes) and at most 65535 rows");
  char* at = (char*)scratch;
  SamplePart* parts = (SamplePart*)at;
  const dim3 grid(SAMPLE_PARTS, rows);
  sample_parts_kernel<<<grid, 256, 0, stream>>>(logits, vocab, row_stride, temperatures, parts);
  if (top_ps == nullptr) {   // no row restricts the nucleus
    sample_pick_kernel<<<rows, 256, 0, stream>>>(logits, vocab, row_stride, temperatures, uniforms,
                                                 parts, nullptr, out);
    MK_LAUNCH_CHECK("sample");
    return 0;
  }
  const size_t parts_bytes = align_up((size_t)rows * SAMPLE_PARTS * sizeof(SamplePart));
  at += parts_bytes;
  SamplePart* kept = (SamplePart*)at;
  at += parts_bytes;
  NucleusRow* search = (NucleusRow*)at;
  at += align_up((size_t)rows * sizeof(NucleusRow));
  unsigned* keep = (unsigned*)at;
  at += align_up((size_t)rows * sizeof(unsigned));
  unsigned long long* hist0 = (unsigned long long*)at;
  unsigned long long* hist1 = hist0 + (size_t)rows * nucleus_bins(0);
  unsigned long long* hist2 = hist1 + (size_t)rows * nucleus_bins(1);
  const size_t bins = (size_t)rows * NUCLEUS_ROW_BINS;
  zero_u64_kernel<<<(int)((bins + 1023) / 1024 < 1024 ? (bins + 1023) / 1024 : 1024), 256, 0,
                    stream>>>(hist0, bins);
  nucleus_histogram_kernel<0><<<grid, 256, 0, stream>>>(logits, vocab, row_stride, temperatures,
                                                         top_ps, parts, search, hist0);
  nucleus_pick_kernel<0><<<rows, 256, 0, stream>>>(temperatures, top_ps, hist0, search, keep);
  nucleus_histogram_kernel<1><<<grid, 256, 0, stream>>>(logits, vocab, row_stride, temperatures,
                                                         top_ps, parts, search, hist1);
  nucleus_pick_kernel<1><<<rows, 256, 0, stream>>>(temperatures, top_ps, hist1, search, keep);
  nucleus_histogram_kernel<2><<<grid, 256, 0, stream>>>(logits, vocab, row_stride, temperatures,
                                                         top_ps, parts, search, hist2);
  nucleus_pick_kernel<2><<<rows, 256, 0, stream>>>(temperatures, top_ps, hist2, search, keep);
  nucleus_parts_kernel<<<grid, 256, 0, stream>>>(logits, vocab, row_stride, temperatures, keep,
                                                 parts, kept);
  sample_pick_kernel<<<rows, 256, 0, stream>>>(logits, vocab, row_stride, temperatures, uniforms,
                                               kept, keep, out);
  MK_LAUNCH_CHECK("sample");
  return 0;
}
