// Causal grouped-query attention over the paged cache, one wavefront per (token, head).
//
// This kernel serves the true 32-bit path and every head size the matrix-core kernels do not
// cover.  It makes no distinction between a prompt portion and a decoded token: a query at
// absolute position p of its sequence reads the keys [first, p] of that sequence from the
// cache, first being 0 or p - window + 1.  Keys lie as [page, kv head, slot, dim], values
// transposed within the page as [page, kv head, dim, slot].  Keys are walked in ascending
// chunks of 64 from `first`, so the order of every sum depends on the query's own position
// only, not on how the sequence was cut into steps or on what else is in the batch.
//
// Scores, softmax and the weighted sum are float32 (reference formulas:
// mercury/model/attention.py:9-32 and :87-101, scale = head_dim^-0.5 passed by the caller).
// Two modifications of the score the reference does not have, for mixers that want them:
// score_cap > 0 bounds it to cap * tanh(score / cap), and distance_slopes [n_q] subtracts
// slope[head] * (query position - key position), a position encoding that lives in the score.
#include "common.h"
#include "mercury_kernels.h"

#define AG_MAX_D 256

template <typename T>
__global__ __launch_bounds__(64) void attention_generic_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ token_seq,
    const int* __restrict__ block_table, int table_stride, int page_shift, int n_q, int n_kv,
    int d, float scale, int window, float score_cap, const float* __restrict__ distance_slopes) {
  __shared__ float qs[AG_MAX_D];
  __shared__ float probs[MK_WAVE];
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int kvh = head / (n_q / n_kv);
  const int pos = positions[t];
  const int* table = block_table + (size_t)token_seq[t] * table_stride;
  const int page_size = 1 << page_shift, page_mask = page_size - 1;
  const int first = window > 0 ? max(0, pos - window + 1) : 0;
  const float slope = distance_slopes ? distance_slopes[head] : 0.f;

  for (int i = lane; i < d; i += MK_WAVE)
    qs[i] = Elem<T>::load(q + (size_t)t * q_stride + head * d + i);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[AG_MAX_D / MK_WAVE];
#pragma unroll
  for (int c = 0; c < AG_MAX_D / MK_WAVE; ++c) acc[c] = 0.f;

  for (int j0 = first; j0 <= pos; j0 += MK_WAVE) {
    const int j = j0 + lane;
    float score = -INFINITY;
    if (j <= pos) {
      const int page = table[j >> page_shift];
      const T* krow =
          k_cache + (((size_t)page * n_kv + kvh) * page_size + (j & page_mask)) * d;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot = fmaf(qs[i], Elem<T>::load(krow + i), dot);
      score = dot * scale;
      // a smooth bound on the score, then a penalty that grows with the distance: both leave
      // the order of the sums alone
      if (score_cap > 0.f) score = score_cap * tanhf(score / score_cap);
      score -= slope * (float)(pos - j);
    }
    const float m_new = fmaxf(m, wave_max(score));
    const float p = j <= pos ? expf(score - m_new) : 0.f;
    const float corr = expf(m - m_new);  // 0 on the first chunk, where m is -inf
    l = l * corr + wave_sum(p);
#pragma unroll
    for (int c = 0; c < AG_MAX_D / MK_WAVE; ++c) acc[c] *= corr;
    __syncthreads();
    probs[lane] = p;
    __syncthreads();
    const int count = min(MK_WAVE, pos - j0 + 1);
    for (int jj = 0; jj < count; ++jj) {
      const int key = j0 + jj;
      const int page = table[key >> page_shift];
      // values are stored transposed within a page: [page, kv head, dim, slot]
      const T* vcol =
          v_cache + ((size_t)page * n_kv + kvh) * page_size * d + (key & page_mask);
      const float pj = probs[jj];
#pragma unroll
      for (int c = 0; c < AG_MAX_D / MK_WAVE; ++c) {
        const int dim = lane + c * MK_WAVE;
        if (dim < d)
          acc[c] = fmaf(pj, Elem<T>::load(vcol + (size_t)dim * page_size), acc[c]);
      }
    }
    m = m_new;
  }

  const float inv = 1.f / l;
#pragma unroll
  for (int c = 0; c < AG_MAX_D / MK_WAVE; ++c) {
    const int dim = lane + c * MK_WAVE;
    if (dim < d) Elem<T>::store(out + (size_t)t * out_stride + head * d + dim, acc[c] * inv);
  }
}

extern "C" int mk_attention_generic(const void* q, int q_stride, void* out, int out_stride,
                                    const void* k_cache, const void* v_cache, int dtype,
                                    const int* positions, const int* token_seq,
                                    const int* block_table, int table_stride, int page_size,
                                    int n_q, int n_kv, int d, float scale, int window,
                                    float score_cap, const float* distance_slopes, int tokens,
                                    hipStream_t stream) {
  MK_REQUIRE(tokens >= 0 && n_q > 0 && n_kv > 0 && d > 0, "attention: bad sizes");
  MK_REQUIRE(n_q % n_kv == 0, "attention: %d query heads are not a multiple of %d kv heads",
             n_q, n_kv);
  MK_REQUIRE(d <= AG_MAX_D, "attention: head size %d exceeds the supported maximum %d", d,
             AG_MAX_D);
  MK_REQUIRE(mk_is_pow2(page_size), "attention: page size %d is not a power of two", page_size);
  MK_REQUIRE(n_q <= 65535, "attention: too many heads (%d)", n_q);
  MK_REQUIRE(window >= 0, "attention: negative window");
  MK_REQUIRE(score_cap >= 0.f, "attention: negative score cap");
  if (tokens == 0) return 0;
  dim3 grid(tokens, n_q);
  if (dtype == MK_F32)
    attention_generic_kernel<float><<<grid, MK_WAVE, 0, stream>>>(
        (const float*)q, q_stride, (float*)out, out_stride, (const float*)k_cache,
        (const float*)v_cache, positions, token_seq, block_table, table_stride,
        mk_log2(page_size), n_q, n_kv, d, scale, window, score_cap, distance_slopes);
  else if (dtype == MK_BF16)
    attention_generic_kernel<bf16_t><<<grid, MK_WAVE, 0, stream>>>(
        (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_cache,
        (const bf16_t*)v_cache, positions, token_seq, block_table, table_stride,
        mk_log2(page_size), n_q, n_kv, d, scale, window, score_cap, distance_slopes);
  else
    MK_REQUIRE(false, "attention: unknown dtype %d", dtype);
  MK_LAUNCH_CHECK("attention_generic");
  return 0;
}
