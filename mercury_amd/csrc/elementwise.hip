// Row-wise and element-wise kernels: embedding gather, RMSNorm (with the residual sum folded
// in), SiLU-gating, rotary position encoding fused with the write into the paged cache.
// Arithmetic is float32 throughout; the element type only decides storage.
#include "common.h"
#include "mercury_kernels.h"

// ------------------------------------------------------------------------------- embedding

template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                             float* __restrict__ out, int hidden, int vocab, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  // Ids are validated on the host; the clamp only keeps a bad id from reading outside.
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* row = table + (size_t)id * hidden;
  float* dst = out + (size_t)t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = Elem<T>::load(row + i) * scale;
}

// bfloat16 rows of a multiple of 8 elements: 16 bytes in, 32 bytes out per thread and turn.
__global__ void embed_bf16x8_kernel(const int* __restrict__ ids, const bf16_t* __restrict__ table,
                                    float* __restrict__ out, int hidden, int vocab, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const uint4* row = (const uint4*)(table + (size_t)id * hidden);
  float4* dst = (float4*)(out + (size_t)t * hidden);
  for (int i = threadIdx.x; i < hidden / 8; i += blockDim.x) {
    const uint4 u = row[i];
    dst[2 * i] = make_float4(__uint_as_float(u.x << 16) * scale,
                             __uint_as_float(u.x & 0xffff0000u) * scale,
                             __uint_as_float(u.y << 16) * scale,
                             __uint_as_float(u.y & 0xffff0000u) * scale);
    dst[2 * i + 1] = make_float4(__uint_as_float(u.z << 16) * scale,
                                 __uint_as_float(u.z & 0xffff0000u) * scale,
                                 __uint_as_float(u.w << 16) * scale,
                                 __uint_as_float(u.w & 0xffff0000u) * scale);
  }
}

extern "C" int mk_embed(const int* ids, const void* table, int dtype, float* out, int tokens,
                        int hidden, int vocab, float scale, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && hidden > 0 && vocab > 0, "embed: bad sizes T=%d H=%d V=%d", tokens,
             hidden, vocab);
  if (tokens == 0) return 0;
  if (dtype == MK_BF16 && hidden % 8 == 0) {
    const int chunks = hidden / 8;
    embed_bf16x8_kernel<<<tokens, chunks >= 256 ? 256 : (chunks + 63) / 64 * 64, 0, stream>>>(
        ids, (const bf16_t*)table, out, hidden, vocab, scale);
    MK_LAUNCH_CHECK("embed");
    return 0;
  }
  const int threads = hidden >= 256 ? 256 : 64;
  if (dtype == MK_F32)
    embed_kernel<float><<<tokens, threads, 0, stream>>>(ids, (const float*)table, out, hidden,
                                                        vocab, scale);
  else if (dtype == MK_BF16)
    embed_kernel<bf16_t><<<tokens, threads, 0, stream>>>(ids, (const bf16_t*)table, out, hidden,
                                                         vocab, scale);
  else
    MK_REQUIRE(false, "embed: unknown dtype %d", dtype);
  MK_LAUNCH_CHECK("embed");
  return 0;
}

// The same into the fixed-point residual stream of a step of few tokens.
template <typename T>
__global__ void embed_fixed_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                   fixed_t* __restrict__ out, int hidden, int vocab, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* row = table + (size_t)id * hidden;
  fixed_t* dst = out + (size_t)t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_fixed(Elem<T>::load(row + i) * scale);
}

extern "C" int mk_embed_fixed(const int* ids, const void* table, int dtype, long long* out,
                              int tokens, int hidden, int vocab, float scale, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && hidden > 0 && vocab > 0, "embed: bad sizes T=%d H=%d V=%d", tokens,
             hidden, vocab);
  MK_REQUIRE(dtype == MK_F32 || dtype == MK_BF16, "embed: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  const int threads = hidden >= 1024 ? 1024 : (hidden + 63) / 64 * 64;
  if (dtype == MK_F32)
    embed_fixed_kernel<float><<<tokens, threads, 0, stream>>>(ids, (const float*)table,
                                                              (fixed_t*)out, hidden, vocab, scale);
  else
    embed_fixed_kernel<bf16_t><<<tokens, threads, 0, stream>>>(ids, (const bf16_t*)table,
                                                               (fixed_t*)out, hidden, vocab, scale);
  MK_LAUNCH_CHECK("embed_fixed");
  return 0;
}

// ------------------------------------------------------------------------------- logit cap

// x <- cap * tanh(x / cap), in place: a smooth bound on the logits' size.  tanh from one
// exponential: tanh(z) = 1 - 2 / (exp(2 z) + 1), exact at both ends (exp overflows to inf,
// the quotient goes to 0).
__global__ void logit_cap_kernel(float* __restrict__ x, long long n, float cap) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float z = x[i] / cap;
  x[i] = cap * (1.f - 2.f / (__expf(2.f * z) + 1.f));
}

extern "C" int mk_logit_cap(float* logits, long long count, float cap, hipStream_t stream) {
  MK_REQUIRE(count >= 0 && cap > 0.f, "logit_cap: bad arguments n=%lld cap=%g", count, (double)cap);
  if (count == 0) return 0;
  const long long blocks = (count + 255) / 256;
  MK_REQUIRE(blocks < (1ll << 31), "logit_cap: %lld elements are too many for one launch", count);
  logit_cap_kernel<<<(unsigned)blocks, 256, 0, stream>>>(logits, count, cap);
  MK_LAUNCH_CHECK("logit_cap");
  return 0;
}

// ----------------------------------------------------------- per-request state of fixed size

// State rows live in slots [num_slots, width] (float32); a sequence's slot is
// slots[token_seq[t]].  Store: every token at absolute position `at_position` writes its row of
// x into its sequence's slot.  Load: every token reads its sequence's row.
template <typename T>
__global__ void state_store_kernel(const T* __restrict__ x, float* __restrict__ state,
                                   const int* __restrict__ slots, const int* __restrict__ token_seq,
                                   const int* __restrict__ positions, int at_position, int width) {
  const int t = blockIdx.x;
  if (positions[t] != at_position) return;
  float* dst = state + (size_t)slots[token_seq[t]] * width;
  const T* src = x + (size_t)t * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = Elem<T>::load(src + i);
}

template <typename T>
__global__ void state_load_kernel(const float* __restrict__ state, const int* __restrict__ slots,
                                  const int* __restrict__ token_seq, T* __restrict__ out, int width) {
  const int t = blockIdx.x;
  const float* src = state + (size_t)slots[token_seq[t]] * width;
  T* dst = out + (size_t)t * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) Elem<T>::store(dst + i, src[i]);
}

extern "C" int mk_state_store(const void* x, int dtype, float* state, const int* slots,
                              const int* token_seq, const int* positions, int at_position,
                              int tokens, int width, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && width > 0 && at_position >= 0, "state_store: bad sizes");
  MK_REQUIRE(dtype == MK_F32 || dtype == MK_BF16, "state_store: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  const int threads = width >= 256 ? 256 : 64;
  if (dtype == MK_F32)
    state_store_kernel<float><<<tokens, threads, 0, stream>>>((const float*)x, state, slots,
                                                              token_seq, positions, at_position, width);
  else
    state_store_kernel<bf16_t><<<tokens, threads, 0, stream>>>((const bf16_t*)x, state, slots,
                                                               token_seq, positions, at_position, width);
  MK_LAUNCH_CHECK("state_store");
  return 0;
}

extern "C" int mk_state_load(const float* state, const int* slots, const int* token_seq, void* out,
                             int dtype, int tokens, int width, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && width > 0, "state_load: bad sizes");
  MK_REQUIRE(dtype == MK_F32 || dtype == MK_BF16, "state_load: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  const int threads = width >= 256 ? 256 : 64;
  if (dtype == MK_F32)
    state_load_kernel<float><<<tokens, threads, 0, stream>>>(state, slots, token_seq, (float*)out, width);
  else
    state_load_kernel<bf16_t><<<tokens, threads, 0, stream>>>(state, slots, token_seq, (bf16_t*)out, width);
  MK_LAUNCH_CHECK("state_load");
  return 0;
}

// --------------------------------------------------------------------------------- RMSNorm

// Sum of p[0], p[stride], ..., p[(n-1) stride], four loads in flight at a time; the order of
// the additions is fixed: ((p0 + p1) + (p2 + p3)) per group, groups in ascending order.
__device__ __forceinline__ float sum_partials(const float* __restrict__ p, int n, size_t stride) {
  float total = 0.f;
  int k = 0;
  for (; k + 4 <= n; k += 4) {
    const float a = p[(size_t)k * stride], b = p[(size_t)(k + 1) * stride];
    const float c = p[(size_t)(k + 2) * stride], d = p[(size_t)(k + 3) * stride];
    total += (a + b) + (c + d);
  }
  for (; k < n; ++k) total += p[(size_t)k * stride];
  return total;
}

// One block per output row.  h is the float32 residual stream.  When `partials` is given,
// the P partial sums of the preceding projection are first added into h (in the order
// 0..P-1) and written back, so the residual sum and the norm are one pass.
// out = round(round(x * rsqrt(mean(x^2) + eps)) * w): the normalised value is rounded to the
// storage type before the weight multiplies it, as the unfused reference path does
// (reference: mercury/model/qwen2.py:27-31).
template <typename TO, typename TW>
__global__ void rmsnorm_kernel(float* __restrict__ h, const float* __restrict__ partials,
                               int num_partials, size_t partial_stride,
                               const TW* __restrict__ weight, float eps,
                               const int* __restrict__ rows, TO* __restrict__ out, int hidden) {
  __shared__ float scratch[16];
  const int out_row = blockIdx.x;
  const int in_row = rows ? rows[out_row] : out_row;
  float* x = h + (size_t)in_row * hidden;
  float sq = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = x[i];
    if (num_partials > 0) {
      v += sum_partials(partials + (size_t)in_row * hidden + i, num_partials, partial_stride);
      x[i] = v;
    }
    sq += v * v;
  }
  const float total = block_sum(sq, scratch);
  const float rstd = rsqrtf(total / (float)hidden + eps);
  TO* dst = out + (size_t)out_row * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float n = Elem<TO>::round(x[i] * rstd);
    Elem<TO>::store(dst + i, n * Elem<TW>::load(weight + i));
  }
}

// The same with 16-byte accesses and the row kept in registers between the two passes: thread
// t holds chunks t, t + threads, ... (CH of them at most) of four values each, and asks for
// its weights before it waits for the sum of squares.  Needs H % 4 == 0.
template <int N>
struct WeightChunk;
template <>
struct WeightChunk<0> {  // float32
  static __device__ __forceinline__ float4 load(const void* w, int chunk) {
    return ((const float4*)w)[chunk];
  }
};
template <>
struct WeightChunk<1> {  // bfloat16
  static __device__ __forceinline__ float4 load(const void* w, int chunk) {
    const uint2 u = ((const uint2*)w)[chunk];
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                       __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
  }
};

template <typename TO, int WBF16, int CH>
__global__ void rmsnorm_vec_kernel(float* __restrict__ h, const float* __restrict__ partials,
                                   int num_partials, size_t partial_stride,
                                   const void* __restrict__ weight, float eps,
                                   const int* __restrict__ rows, TO* __restrict__ out,
                                   int hidden) {
  __shared__ float scratch[16];
  const int out_row = blockIdx.x;
  const int in_row = rows ? rows[out_row] : out_row;
  const int chunks = hidden >> 2;
  float4* x4 = (float4*)(h + (size_t)in_row * hidden);
  float4 v[CH], w[CH];
  float sq = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int idx = threadIdx.x + c * blockDim.x;
    v[c] = make_float4(0.f, 0.f, 0.f, 0.f);
    w[c] = v[c];
    if (idx < chunks) {
      v[c] = x4[idx];
      w[c] = WeightChunk<WBF16>::load(weight, idx);
    }
  }
  if (num_partials > 0) {
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int idx = threadIdx.x + c * blockDim.x;
      if (idx >= chunks) continue;
      const float4* p4 = (const float4*)(partials + (size_t)in_row * hidden) + idx;
      const size_t stride4 = partial_stride >> 2;
      // Up to sixteen slices' loads are in flight at once (a decode step's norm is a chain of
      // round trips to the L2 and little else); the additions keep their order: groups of
      // four as (a + b) + (c + d), group after group, then what is left one by one.
      float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
      for (int k0 = 0; k0 < num_partials; k0 += 16) {
        float4 part[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          part[j] = k0 + j < num_partials ? p4[(size_t)(k0 + j) * stride4]
                                          : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int j = 0; j < 16; j += 4) {
          if (k0 + j + 4 <= num_partials) {
            t.x += (part[j].x + part[j + 1].x) + (part[j + 2].x + part[j + 3].x);
            t.y += (part[j].y + part[j + 1].y) + (part[j + 2].y + part[j + 3].y);
            t.z += (part[j].z + part[j + 1].z) + (part[j + 2].z + part[j + 3].z);
            t.w += (part[j].w + part[j + 1].w) + (part[j + 2].w + part[j + 3].w);
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              if (k0 + j + i < num_partials) {
                t.x += part[j + i].x;
                t.y += part[j + i].y;
                t.z += part[j + i].z;
                t.w += part[j + i].w;
              }
            }
          }
        }
      }
      v[c] = make_float4(v[c].x + t.x, v[c].y + t.y, v[c].z + t.z, v[c].w + t.w);
      x4[idx] = v[c];
    }
  }
#pragma unroll
  for (int c = 0; c < CH; ++c)
    sq += (v[c].x * v[c].x + v[c].y * v[c].y) + (v[c].z * v[c].z + v[c].w * v[c].w);
  const float total = block_sum(sq, scratch);
  const float rstd = rsqrtf(total / (float)hidden + eps);
  TO* dst = out + (size_t)out_row * hidden;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int idx = threadIdx.x + c * blockDim.x;
    if (idx >= chunks) continue;
    const float a = Elem<TO>::round(v[c].x * rstd) * w[c].x, b = Elem<TO>::round(v[c].y * rstd) * w[c].y;
    const float cc = Elem<TO>::round(v[c].z * rstd) * w[c].z, d = Elem<TO>::round(v[c].w * rstd) * w[c].w;
    if constexpr (sizeof(TO) == 2) {
      *(uint2*)(dst + 4 * idx) = make_uint2(pack_bf16x2(a, b), pack_bf16x2(cc, d));
    } else {
      *(float4*)(dst + 4 * idx) = make_float4(a, b, cc, d);
    }
  }
}

template <typename TO>
static int launch_rmsnorm(float* h, const float* partials, int num_partials,
                          size_t partial_stride, const void* weight, int weight_dtype, float eps,
                          const int* rows, TO* out, int out_rows, int hidden,
                          hipStream_t stream) {
  // Few rows (decoding): as many threads per row as it has chunks of four, so that every
  // thread waits for one group of loads only; many rows: 256 threads each.
  if (hidden % 4 == 0 && (num_partials == 0 || partial_stride % 4 == 0)) {
    const int chunks = hidden / 4;
    int threads = out_rows <= 256 ? (chunks + 63) / 64 * 64 : 256;
    while (threads < 1024 && chunks > 4 * threads) threads *= 2;   // wide rows: at most 4 chunks a thread
    if (threads > 1024) threads = 1024;
    const int ch = (chunks + threads - 1) / threads;
#define RMS_VEC(CH)                                                                            \
  do {                                                                                         \
    if (weight_dtype == MK_F32)                                                                \
      rmsnorm_vec_kernel<TO, 0, CH><<<out_rows, threads, 0, stream>>>(                         \
          h, partials, num_partials, partial_stride, weight, eps, rows, out, hidden);          \
    else                                                                                       \
      rmsnorm_vec_kernel<TO, 1, CH><<<out_rows, threads, 0, stream>>>(                         \
          h, partials, num_partials, partial_stride, weight, eps, rows, out, hidden);          \
    return 0;                                                                                  \
  } while (0)
    if (ch == 1) RMS_VEC(1);
    if (ch == 2) RMS_VEC(2);
    if (ch <= 4) RMS_VEC(4);
    if (ch <= 8) RMS_VEC(8);
#undef RMS_VEC
  }
  int threads = hidden >= 512 ? 256 : (hidden >= 256 ? 128 : 64);
  if (out_rows <= 64 && num_partials > 0) threads = hidden >= 1024 ? 1024 : (hidden + 63) / 64 * 64;
  if (weight_dtype == MK_F32)
    rmsnorm_kernel<TO, float><<<out_rows, threads, 0, stream>>>(
        h, partials, num_partials, partial_stride, (const float*)weight, eps, rows, out, hidden);
  else
    rmsnorm_kernel<TO, bf16_t><<<out_rows, threads, 0, stream>>>(
        h, partials, num_partials, partial_stride, (const bf16_t*)weight, eps, rows, out, hidden);
  return 0;
}

// RMSNorm of rows of the fixed-point residual stream: one block per output row, the row's
// values two a thread and turn, the formula and the roundings of rmsnorm_kernel.
template <typename TO>
__global__ void rmsnorm_fixed_kernel(const fixed_t* __restrict__ h64, const void* __restrict__ weight,
                                     int weight_bf16, float eps, const int* __restrict__ rows,
                                     TO* __restrict__ out, int hidden) {
  __shared__ float scratch[16];
  const int out_row = blockIdx.x;
  const int in_row = rows ? rows[out_row] : out_row;
  const fixed_t* x = h64 + (size_t)in_row * hidden;
  float sq = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = from_fixed(x[i]);
    sq += v * v;
  }
  const float total = block_sum(sq, scratch);
  const float rstd = rsqrtf(total / (float)hidden + eps);
  TO* dst = out + (size_t)out_row * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float n = Elem<TO>::round(from_fixed(x[i]) * rstd);
    const float w = weight_bf16 ? bf16_to_f32(((const bf16_t*)weight)[i]) : ((const float*)weight)[i];
    Elem<TO>::store(dst + i, n * w);
  }
}

extern "C" int mk_rmsnorm_fixed(const long long* h64, const void* weight, int weight_dtype,
                                float eps, const int* rows, void* out, int out_dtype, int out_rows,
                                int hidden, hipStream_t stream) {
  MK_REQUIRE(out_rows >= 0 && hidden > 0, "rmsnorm: bad sizes rows=%d H=%d", out_rows, hidden);
  MK_REQUIRE(weight_dtype == MK_F32 || weight_dtype == MK_BF16, "rmsnorm: weight dtype %d",
             weight_dtype);
  MK_REQUIRE(out_dtype == MK_F32 || out_dtype == MK_BF16, "rmsnorm: unknown out dtype %d", out_dtype);
  if (out_rows == 0) return 0;
  const int threads = hidden >= 1024 ? 1024 : (hidden + 63) / 64 * 64;
  if (out_dtype == MK_F32)
    rmsnorm_fixed_kernel<float><<<out_rows, threads, 0, stream>>>(
        (const fixed_t*)h64, weight, weight_dtype == MK_BF16, eps, rows, (float*)out, hidden);
  else
    rmsnorm_fixed_kernel<bf16_t><<<out_rows, threads, 0, stream>>>(
        (const fixed_t*)h64, weight, weight_dtype == MK_BF16, eps, rows, (bf16_t*)out, hidden);
  MK_LAUNCH_CHECK("rmsnorm_fixed");
  return 0;
}

// h64[i] += the sum of `count` float32 partial sums p[k * stride + i] (k in ascending order,
// as sum_partials adds them), for i < n: what a projection that left partial sums owes the
// fixed-point residual stream.
__global__ void fixed_add_kernel(fixed_t* __restrict__ h64, const float* __restrict__ partials,
                                 int count, size_t stride, long long n) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  h64[i] += to_fixed(sum_partials(partials + i, count, stride));
}

extern "C" int mk_fixed_add(long long* h64, const float* partials, int count, long long stride,
                            long long n, hipStream_t stream) {
  MK_REQUIRE(count >= 1 && partials && h64 && n >= 0 && stride >= n, "fixed_add: bad arguments");
  if (n == 0) return 0;
  const long long blocks = (n + 255) / 256;
  MK_REQUIRE(blocks < (1ll << 31), "fixed_add: %lld elements are too many for one launch", n);
  fixed_add_kernel<<<(unsigned)blocks, 256, 0, stream>>>((fixed_t*)h64, partials, count,
                                                         (size_t)stride, n);
  MK_LAUNCH_CHECK("fixed_add");
  return 0;
}

extern "C" int mk_rmsnorm(float* h, const float* partials, int num_partials,
                          long long partial_stride, const void* weight, int weight_dtype,
                          float eps, const int* rows, void* out, int out_dtype, int out_rows,
                          int hidden, hipStream_t stream) {
  MK_REQUIRE(out_rows >= 0 && hidden > 0, "rmsnorm: bad sizes rows=%d H=%d", out_rows, hidden);
  MK_REQUIRE(num_partials >= 0 && (num_partials == 0 || partials != nullptr),
             "rmsnorm: %d partial sums but no buffer", num_partials);
  MK_REQUIRE(weight_dtype == MK_F32 || weight_dtype == MK_BF16, "rmsnorm: weight dtype %d",
             weight_dtype);
  if (out_rows == 0) return 0;
  if (out_dtype == MK_F32)
    launch_rmsnorm<float>(h, partials, num_partials, (size_t)partial_stride, weight,
                          weight_dtype, eps, rows, (float*)out, out_rows, hidden, stream);
  else if (out_dtype == MK_BF16)
    launch_rmsnorm<bf16_t>(h, partials, num_partials, (size_t)partial_stride, weight,
                           weight_dtype, eps, rows, (bf16_t*)out, out_rows, hidden, stream);
  else
    MK_REQUIRE(false, "rmsnorm: unknown out dtype %d", out_dtype);
  MK_LAUNCH_CHECK("rmsnorm");
  return 0;
}

// ------------------------------------------------------------------------------ SiLU gating

// gate_up is [T, 2*I]: columns [0, I) hold the gate, [I, 2I) the up projection.
// out = round(round(silu(g)) * u) (reference: mercury/model/qwen2.py:42).
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out,
                                int inter, size_t total) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / inter;
    const int i = (int)(idx - t * inter);
    const T* row = gate_up + t * 2 * (size_t)inter;
    const float g = Elem<T>::load(row + i);
    const float u = Elem<T>::load(row + inter + i);
    const float s = Elem<T>::round(g / (1.f + expf(-g)));
    Elem<T>::store(out + idx, s * u);
  }
}

extern "C" int mk_silu_mul(const void* gate_up, void* out, int dtype, int tokens, int inter,
                           hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && inter > 0, "silu_mul: bad sizes T=%d I=%d", tokens, inter);
  if (tokens == 0) return 0;
  const size_t total = (size_t)tokens * inter;
  const int threads = 256;
  size_t blocks = (total + threads - 1) / threads;
  if (blocks > 65536) blocks = 65536;
  if (dtype == MK_F32)
    silu_mul_kernel<float><<<(int)blocks, threads, 0, stream>>>((const float*)gate_up,
                                                               (float*)out, inter, total);
  else if (dtype == MK_BF16)
    silu_mul_kernel<bf16_t><<<(int)blocks, threads, 0, stream>>>((const bf16_t*)gate_up,
                                                                (bf16_t*)out, inter, total);
  else
    MK_REQUIRE(false, "silu_mul: unknown dtype %d", dtype);
  MK_LAUNCH_CHECK("silu_mul");
  return 0;
}

// ------------------------------------------------------- rotary encoding + paged cache write

// qkv is [T, row_stride] with q heads first, then k heads, then v heads, each of width d.
// The first `rot` dims of every q and k head are rotated in the half-split layout: dims j
// and j + rot/2 form a pair turned by the angle of (position, j):
//   y[j]         = x[j] * cos - x[j + rot/2] * sin
//   y[j + rot/2] = x[j + rot/2] * cos + x[j] * sin
// (reference: mercury/model/rope.py:6-17).  cos/sin are float32 tables [positions, rot/2].
// q is rotated in place; rotated k and raw v go to the token's slot of the paged cache, keys
// as [pages, n_kv, page_size, d] and values transposed within the page as
// [pages, n_kv, d, page_size], the page taken from the sequence's block table
// (reference: mercury/runner.py:32-34, mercury/model/attention.py:35-45).
template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, int row_stride,
                                     const float* __restrict__ cos_table,
                                     const float* __restrict__ sin_table,
                                     const int* __restrict__ positions,
                                     const int* __restrict__ token_seq,
                                     const int* __restrict__ block_table, int table_stride,
                                     T* __restrict__ k_cache, T* __restrict__ v_cache,
                                     int page_shift, int n_q, int n_kv, int d, int rot,
                                     int interleaved, int write_kv) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = rot / 2;
  const float* cs = cos_table + (size_t)pos * half;
  const float* sn = sin_table + (size_t)pos * half;
  T* row = qkv + (size_t)t * row_stride;

  // q heads: pairwise, in place.  Pair j is dims (j, j + half), or (2j, 2j + 1) when the
  // layout is interleaved.
  for (int idx = threadIdx.x; idx < n_q * half; idx += blockDim.x) {
    const int head = idx / half, j = idx - head * half;
    T* x = row + head * d;
    const int ia = interleaved ? 2 * j : j, ib = interleaved ? 2 * j + 1 : j + half;
    const float a = Elem<T>::load(x + ia), b = Elem<T>::load(x + ib);
    const float c = cs[j], s = sn[j];
    Elem<T>::store(x + ia, a * c - b * s);
    Elem<T>::store(x + ib, b * c + a * s);
  }
  if (!write_kv) return;

  const int page_size = 1 << page_shift;
  const int seq = token_seq[t];
  const int page = block_table[(size_t)seq * table_stride + (pos >> page_shift)];
  if (page < 0) return;  // the host never schedules a write into a page that was given back
  const int off = pos & (page_size - 1);
  const T* k_src = row + n_q * d;
  const T* v_src = k_src + n_kv * d;
  for (int idx = threadIdx.x; idx < n_kv * d; idx += blockDim.x) {
    const int head = idx / d, j = idx - head * d;
    const size_t dst = (((size_t)page * n_kv + head) * page_size + off) * d + j;
    const T* x = k_src + head * d;
    float y;
    if (interleaved && j < rot) {
      const int pair = j >> 1;
      y = (j & 1) ? Elem<T>::load(x + j) * cs[pair] + Elem<T>::load(x + j - 1) * sn[pair]
                  : Elem<T>::load(x + j) * cs[pair] - Elem<T>::load(x + j + 1) * sn[pair];
    } else if (j < half) {
      y = Elem<T>::load(x + j) * cs[j] - Elem<T>::load(x + j + half) * sn[j];
    } else if (j < rot) {
      y = Elem<T>::load(x + j) * cs[j - half] + Elem<T>::load(x + j - half) * sn[j - half];
    } else {
      y = Elem<T>::load(x + j);
    }
    Elem<T>::store(k_cache + dst, y);
    v_cache[(((size_t)page * n_kv + head) * d + j) * page_size + off] = v_src[head * d + j];
  }
}

extern "C" int mk_rope_kv_write(void* qkv, int dtype, int row_stride, const float* cos_table,
                                const float* sin_table, int table_positions,
                                const int* positions, const int* token_seq,
                                const int* block_table, int table_stride, void* k_cache,
                                void* v_cache, int page_size, int n_q, int n_kv, int d, int rot,
                                int interleaved, int write_kv, int tokens, hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && n_q > 0 && n_kv >= 0 && d > 0, "rope: bad sizes");
  MK_REQUIRE(rot >= 0 && rot <= d && rot % 2 == 0, "rope: rotary width %d not in [0, %d] / even",
             rot, d);
  MK_REQUIRE(mk_is_pow2(page_size), "rope: page size %d is not a power of two", page_size);
  MK_REQUIRE(row_stride >= (n_q + (write_kv ? 2 * n_kv : 0)) * d,
             "rope: row stride %d too small for %d+2*%d heads of %d", row_stride, n_q, n_kv, d);
  MK_REQUIRE(rot == 0 || table_positions > 0, "rope: empty angle table");
  if (tokens == 0) return 0;
  const int threads = 128;
  if (dtype == MK_F32)
    rope_kv_write_kernel<float><<<tokens, threads, 0, stream>>>(
        (float*)qkv, row_stride, cos_table, sin_table, positions, token_seq, block_table,
        table_stride, (float*)k_cache, (float*)v_cache, mk_log2(page_size), n_q, n_kv, d, rot,
        interleaved, write_kv);
  else if (dtype == MK_BF16)
    rope_kv_write_kernel<bf16_t><<<tokens, threads, 0, stream>>>(
        (bf16_t*)qkv, row_stride, cos_table, sin_table, positions, token_seq, block_table,
        table_stride, (bf16_t*)k_cache, (bf16_t*)v_cache, mk_log2(page_size), n_q, n_kv, d, rot,
        interleaved, write_kv);
  else
    MK_REQUIRE(false, "rope: unknown dtype %d", dtype);
  MK_LAUNCH_CHECK("rope_kv_write");
  return 0;
}

// ------------------------------------------ consumers of split-K partial sums (decode path)

// The q/k/v projection arrives as float32 slices [p, T, (n_q + 2 n_kv) d]; this adds them up,
// adds the bias, rotates q and k, writes q [T, n_q d] and the cache.  Sums and rotation are
// float32; q, k and v are rounded to the storage type first, as a stored projection would be.
// Workgroup (t, y) takes heads [y * heads_per_group, ...) of token t (a rotation pairs dims
// of one head), so that a few tokens still occupy the chip.
template <typename T, typename TB>
__global__ void qkv_finish_kernel(const float* __restrict__ partials, int num_partials,
                                  size_t partial_stride, const TB* __restrict__ bias,
                                  T* __restrict__ q_out, const float* __restrict__ cos_table,
                                  const float* __restrict__ sin_table,
                                  const int* __restrict__ positions,
                                  const int* __restrict__ token_seq,
                                  const int* __restrict__ block_table, int table_stride,
                                  T* __restrict__ k_cache, T* __restrict__ v_cache,
                                  int page_shift, int n_q, int n_kv, int d, int rot,
                                  int write_kv, int heads_per_group) {
  extern __shared__ float vals[];  // the group's heads of the token: summed, biased, rounded
  const int t = blockIdx.x;
  const int heads = n_q + (write_kv ? 2 * n_kv : 0);
  const int head0 = blockIdx.y * heads_per_group;
  const int count = (min(heads, head0 + heads_per_group) - head0) * d;  // values of this group
  if (count <= 0) return;
  const int pos = positions[t];
  const int half = rot / 2;
  const float* cs = cos_table + (size_t)pos * half;
  const float* sn = sin_table + (size_t)pos * half;
  const int width = (n_q + 2 * n_kv) * d;
  const int col0 = head0 * d;
  const float* row = partials + (size_t)t * width + col0;
  // Where the token's keys and values go, and by what this thread's first value turns: asked
  // for now, beside the partial sums, and not in a chain of trips to memory behind them.
  int page = -1, off = 0;
  const int page_size = 1 << page_shift;
  if (write_kv) {
    page = block_table[(size_t)token_seq[t] * table_stride + (pos >> page_shift)];
    off = pos & (page_size - 1);
  }
  float first_c = 1.f, first_s = 0.f;
  if (rot > 0) {
    const int j = min((int)threadIdx.x, count - 1) % d;
    const int jj = min(j < half ? j : j - half, half - 1);
    first_c = cs[jj];
    first_s = sn[jj];
  }
  if ((d & 3) == 0 && (partial_stride & 3) == 0 &&
      (bias == nullptr || (uintptr_t)bias % 16 == 0)) {
    for (int i = threadIdx.x * 4; i < count; i += blockDim.x * 4) {
      float o[4] = {0.f, 0.f, 0.f, 0.f};
      if (bias) {
        if constexpr (sizeof(TB) == 2) {
          const ushort4 b = *(const ushort4*)(bias + col0 + i);
          o[0] = bf16_to_f32(b.x), o[1] = bf16_to_f32(b.y), o[2] = bf16_to_f32(b.z), o[3] = bf16_to_f32(b.w);
        } else {
          const float4 b = *(const float4*)(bias + col0 + i);
          o[0] = b.x, o[1] = b.y, o[2] = b.z, o[3] = b.w;
        }
      }
      // Up to sixteen slices' loads in flight at once (at clamped places: a load under a
      // condition is a branch the next load waits behind); the additions in the order of
      // sum_partials: fours as (a + b) + (c + d), then what is left one by one.
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      for (int k0 = 0; k0 < num_partials; k0 += 16) {
        float4 part[16];
#pragma unroll
        for (int j = 0; j < 16; ++j)
          part[j] = *(const float4*)(row + i + (size_t)min(k0 + j, num_partials - 1) * partial_stride);
#pragma unroll
        for (int j = 0; j < 16; j += 4) {
          if (k0 + j + 4 <= num_partials) {
            v.x += (part[j].x + part[j + 1].x) + (part[j + 2].x + part[j + 3].x);
            v.y += (part[j].y + part[j + 1].y) + (part[j + 2].y + part[j + 3].y);
            v.z += (part[j].z + part[j + 1].z) + (part[j + 2].z + part[j + 3].z);
            v.w += (part[j].w + part[j + 1].w) + (part[j + 2].w + part[j + 3].w);
          } else {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              if (k0 + j + u < num_partials) {
                v.x += part[j + u].x, v.y += part[j + u].y, v.z += part[j + u].z, v.w += part[j + u].w;
              }
            }
          }
        }
      }
      vals[i] = Elem<T>::round(v.x + o[0]);
      vals[i + 1] = Elem<T>::round(v.y + o[1]);
      vals[i + 2] = Elem<T>::round(v.z + o[2]);
      vals[i + 3] = Elem<T>::round(v.w + o[3]);
    }
  } else {
    for (int i = threadIdx.x; i < count; i += blockDim.x) {
      float v = sum_partials(row + i, num_partials, partial_stride);
      if (bias) v += Elem<TB>::load(bias + col0 + i);
      vals[i] = Elem<T>::round(v);
    }
  }
  __syncthreads();

  auto rotated = [&](int base, int j, bool first) {
    if (j >= rot) return vals[base + j];
    const int jj = j < half ? j : j - half;
    const float c = first ? first_c : cs[jj], sine = first ? first_s : sn[jj];
    if (j < half) return vals[base + j] * c - vals[base + j + half] * sine;
    return vals[base + j] * c + vals[base + j - half] * sine;
  };
  for (int i = threadIdx.x; i < count; i += blockDim.x) {
    const int local = i / d, j = i - local * d, head = head0 + local;
    if (head < n_q) {
      Elem<T>::store(q_out + ((size_t)t * n_q + head) * d + j, rotated(local * d, j, i == (int)threadIdx.x));
    } else if (page >= 0) {
      if (head < n_q + n_kv) {
        const int kh = head - n_q;
        Elem<T>::store(k_cache + (((size_t)page * n_kv + kh) * page_size + off) * d + j,
                       rotated(local * d, j, i == (int)threadIdx.x));
      } else {
        const int vh = head - n_q - n_kv;
        Elem<T>::store(v_cache + (((size_t)page * n_kv + vh) * d + j) * page_size + off, vals[i]);
      }
    }
  }
}

extern "C" int mk_qkv_finish(const float* partials, int num_partials, long long partial_stride,
                             const void* bias, int bias_dtype, void* q_out, int dtype,
                             const float* cos_table, const float* sin_table, int table_positions,
                             const int* positions, const int* token_seq, const int* block_table,
                             int table_stride, void* k_cache, void* v_cache, int page_size,
                             int n_q, int n_kv, int d, int rot, int write_kv, int tokens,
                             hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && n_q > 0 && n_kv >= 0 && d > 0 && num_partials >= 1,
             "qkv_finish: bad sizes");
  MK_REQUIRE(rot >= 0 && rot <= d && rot % 2 == 0, "qkv_finish: rotary width %d", rot);
  MK_REQUIRE(mk_is_pow2(page_size), "qkv_finish: page size %d is not a power of two", page_size);
  MK_REQUIRE(rot == 0 || table_positions > 0, "qkv_finish: empty angle table");
  MK_REQUIRE(dtype == MK_BF16 || dtype == MK_F32, "qkv_finish: unknown dtype %d", dtype);
  if (tokens == 0) return 0;
  const int shift = mk_log2(page_size);
  // about two workgroups of 256 threads per compute unit, whole heads each
  const int heads = n_q + (write_kv ? 2 * n_kv : 0);
  int groups = (512 + tokens - 1) / tokens;
  groups = groups < 1 ? 1 : (groups > heads ? heads : groups);
  const int heads_per_group = (heads + groups - 1) / groups;
  groups = (heads + heads_per_group - 1) / heads_per_group;
  const size_t lds_bytes = (size_t)heads_per_group * d * sizeof(float);
  const int threads = 256;
  MK_REQUIRE(lds_bytes <= 64 * 1024, "qkv_finish: %d heads of %d values exceed LDS",
             heads_per_group, d);
  MK_REQUIRE(groups <= 65535, "qkv_finish: %d head groups", groups);
#define QKV_LAUNCH(T, TB)                                                                      \
  qkv_finish_kernel<T, TB><<<dim3(tokens, groups), threads, lds_bytes, stream>>>(              \
      partials, num_partials, (size_t)partial_stride, (const TB*)bias, (T*)q_out, cos_table,   \
      sin_table, positions, token_seq, block_table, table_stride, (T*)k_cache, (T*)v_cache,    \
      shift, n_q, n_kv, d, rot, write_kv, heads_per_group)
  if (dtype == MK_BF16) {
    if (bias && bias_dtype == MK_BF16) QKV_LAUNCH(bf16_t, bf16_t);
    else QKV_LAUNCH(bf16_t, float);
  } else {
    if (bias && bias_dtype == MK_BF16) QKV_LAUNCH(float, bf16_t);
    else QKV_LAUNCH(float, float);
  }
#undef QKV_LAUNCH
  MK_LAUNCH_CHECK("qkv_finish");
  return 0;
}
