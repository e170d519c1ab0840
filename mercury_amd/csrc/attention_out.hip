// Decoding: the merge of the attention's key splits folded into the output projection.
//
// When the keys of a decoded token are split over workgroups, the attention kernel leaves, per
// (token, key/value head, part, row), a running maximum, a sum of weights and a weighted sum
// of values.  Merging them is a kernel of its own with next to nothing to do, followed by a
// projection with little more; here one kernel does both.  A workgroup owns 64 or 128 rows of
// the output matrix W [N, n_q D] and HP query heads (a slice of K): it first asks for its
// weights, then merges its heads' parts for all M tokens into LDS (bfloat16, what the
// attention would have written), multiplies, and writes a float32 partial sum
// out[slice, M, N] that the next norm adds up in slice order, or adds its result into the
// fixed-point residual stream.  Every workgroup of a slice repeats the slice's merge (the
// parts come out of the L2); the host chooses this kernel where that repetition is small
// beside the weights.
#include "common.h"
#include "mercury_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

union OutFrag {
  bf16x8 v;
  uint4 u;
};

struct AttnOutParams {
  const float* part_o;   // [token, kv head, part, 16, D]
  const float* part_ml;  // [token, kv head, part, 16, 2]: base-2 running maximum, sum of weights
  const bf16_t* w;       // [N, n_q * D]
  float* out;            // [n_q / HP, M, N], or null and
  fixed_t* fixed_out;    // [M, N]: the fixed-point residual stream the result is added into
  int M, N, n_kv, group, parts;
};

#define OUT_MAX_WEIGHTS 2048   // (token, head) pairs of a slice x parts a workgroup weighs

// D: head size; HP: query heads per slice; MT: 16-token tiles; NW: 16-row tiles of W per wavefront.
template <int D, int HP, int MT, int NW>
__global__ __launch_bounds__(256) void attn_out_kernel(AttnOutParams p) {
  constexpr int KW = HP * D;            // the slice's width in k
  constexpr int STRIDE = KW + 8;        // row stride in LDS: 16 bytes of padding against bank conflicts
  constexpr int KSTEPS = KW / 32;
  __shared__ __align__(16) bf16_t merged[16 * MT * STRIDE];
  __shared__ float weight[OUT_MAX_WEIGHTS];   // [pair][part]: first the maxima, then the weights
  __shared__ float mass[OUT_MAX_WEIGHTS];     // [pair][part]: the parts' sums of weights
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g4 = lane >> 4;
  const int K = p.n_kv * p.group * D;
  const int slice = blockIdx.y, head0 = slice * HP;
  const int n0 = (blockIdx.x * 4 + wave) * (16 * NW);
  const int S = p.parts, pairs = p.M * HP;

  // The weights first: they come from HBM and depend on nothing.
  OutFrag a[NW][KSTEPS];
#pragma unroll
  for (int t = 0; t < NW; ++t) {
    const bf16_t* row = p.w + (size_t)min(n0 + t * 16 + r, p.N - 1) * K + head0 * D + g4 * 8;
#pragma unroll
    for (int k = 0; k < KSTEPS; ++k) a[t][k].u = *(const uint4*)(row + k * 32);
  }

  // Where (token, head hh of the slice)'s parts begin, in rows of 16-row tiles.
  auto base_of = [&](int pair) {
    const int tok = pair / HP, head = head0 + pair % HP;
    const int kvh = head / p.group, j = head - kvh * p.group;
    return (((size_t)tok * p.n_kv + kvh) * S) * 16 + j;
  };

  // The parts' weighted values are asked for now as well, where a thread's share of them fits
  // its registers (sixteen loads of four floats): they depend on nothing either, and asked
  // for after the weights are known (below) they would be a second chain of trips to memory
  // behind the first.  A thread's items are (pair, four dims) number threadIdx.x + 256 it.
  constexpr int QUADS = D / 4;
  constexpr int ITEMS = (16 * MT * HP * QUADS + 255) / 256;   // items per thread
  constexpr int HELD = 16 / ITEMS;                            // parts per item a thread can hold
  // (From 17 tokens on: with fewer the merge hides behind the weights' way from HBM either
  // way, 1.010 against 1.013 ms a step of 8 tokens of the 0.5B shapes; 64 tokens: 1.634
  // against 1.662.)
  const bool ahead = MT >= 2 && ITEMS <= 4 && S <= HELD;
  float4 held[MT >= 2 && ITEMS <= 4 ? ITEMS : 1][MT >= 2 && ITEMS <= 4 ? HELD : 1];
  if constexpr (MT >= 2 && ITEMS <= 4) {
    if (ahead) {
#pragma unroll
      for (int it = 0; it < ITEMS; ++it) {
        const int i = threadIdx.x + 256 * it;
        const int pair = i / QUADS, quad = i - pair * QUADS;
        const bool real = i < 16 * MT * HP * QUADS && pair / HP < p.M;
        const float4* src = (const float4*)(p.part_o + base_of(real ? pair : 0) * D + quad * 4);
#pragma unroll
        for (int s2 = 0; s2 < HELD; ++s2) {
          held[it][s2] = real && s2 < S ? src[(size_t)s2 * (16 * D / 4)] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
      }
    }
  }

  // Merge, step 1: every part's maximum and sum, all loads at once.
  for (int i = threadIdx.x; i < pairs * S; i += 256) {
    const int pair = i / S, part = i - pair * S;
    const float2 ml = *(const float2*)(p.part_ml + (base_of(pair) + (size_t)part * 16) * 2);
    weight[i] = ml.x;
    mass[i] = ml.y;
  }
  __syncthreads();
  // Step 2: a thread per pair turns the maxima into weights: w = 2^(m - max) / total, in part
  // order.
  for (int pair = threadIdx.x; pair < pairs; pair += 256) {
    float* w = weight + pair * S;
    const float* l = mass + pair * S;
    float mx = -INFINITY;
    for (int s2 = 0; s2 < S; ++s2) mx = fmaxf(mx, w[s2]);
    float total = 0.f;
    for (int s2 = 0; s2 < S; ++s2) {
      const float e = w[s2] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(w[s2] - mx);
      w[s2] = e;
      total += l[s2] * e;
    }
    const float inv = 1.f / total;
    for (int s2 = 0; s2 < S; ++s2) w[s2] *= inv;
  }
  __syncthreads();
  // Step 3: a thread per four dims of a pair adds the weighted parts up in part order (in
  // fours, then what is left one by one: the same sums whether the values were asked for
  // ahead or are only now, four parts' loads in flight at a time) and leaves bfloat16 in LDS
  // (what the attention would have written).
  bool done = false;
  if constexpr (MT >= 2 && ITEMS <= 4) {
    if (ahead) {
#pragma unroll
      for (int it = 0; it < ITEMS; ++it) {
        const int i = threadIdx.x + 256 * it;
        if (i >= 16 * MT * HP * QUADS) continue;
        const int pair = i / QUADS, quad = i - pair * QUADS;
        const int tok = pair / HP, hh = pair - tok * HP;
        uint2* dst = (uint2*)(merged + tok * STRIDE + hh * D + quad * 4);
        if (tok >= p.M) {
          *dst = make_uint2(0u, 0u);
          continue;
        }
        const float* w = weight + pair * S;
        float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int g = 0; g < HELD; g += 4) {       // (constant indices: the values are registers)
          if (g + 4 <= HELD && g + 4 <= S) {
            const float4 v0 = held[it][g], v1 = held[it][g + 1 < HELD ? g + 1 : 0];
            const float4 v2 = held[it][g + 2 < HELD ? g + 2 : 0], v3 = held[it][g + 3 < HELD ? g + 3 : 0];
            const float w0 = w[g], w1 = w[g + 1], w2 = w[g + 2], w3 = w[g + 3];
            o.x += (v0.x * w0 + v1.x * w1) + (v2.x * w2 + v3.x * w3);
            o.y += (v0.y * w0 + v1.y * w1) + (v2.y * w2 + v3.y * w3);
            o.z += (v0.z * w0 + v1.z * w1) + (v2.z * w2 + v3.z * w3);
            o.w += (v0.w * w0 + v1.w * w1) + (v2.w * w2 + v3.w * w3);
          } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              if (g + k < HELD && g + k < S) {
                const float4 v = held[it][g + k < HELD ? g + k : 0];
                const float ws = w[g + k];
                o.x += v.x * ws, o.y += v.y * ws, o.z += v.z * ws, o.w += v.w * ws;
              }
            }
          }
        }
        *dst = make_uint2(pack_bf16x2(o.x, o.y), pack_bf16x2(o.z, o.w));
      }
      done = true;
    }
  }
  if (!done) {
    for (int i = threadIdx.x; i < 16 * MT * HP * QUADS; i += 256) {
      const int pair = i / QUADS, quad = i - pair * QUADS;
      const int tok = pair / HP, hh = pair - tok * HP;
      uint2* dst = (uint2*)(merged + tok * STRIDE + hh * D + quad * 4);
      if (tok >= p.M) {
        *dst = make_uint2(0u, 0u);
        continue;
      }
      const float4* src = (const float4*)(p.part_o + base_of(pair) * D + quad * 4);
      const size_t step = (size_t)16 * D / 4;
      const float* w = weight + pair * S;
      float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
      int s2 = 0;
      for (; s2 + 4 <= S; s2 += 4) {
        const float4 v0 = src[(size_t)s2 * step], v1 = src[(size_t)(s2 + 1) * step];
        const float4 v2 = src[(size_t)(s2 + 2) * step], v3 = src[(size_t)(s2 + 3) * step];
        const float w0 = w[s2], w1 = w[s2 + 1], w2 = w[s2 + 2], w3 = w[s2 + 3];
        o.x += (v0.x * w0 + v1.x * w1) + (v2.x * w2 + v3.x * w3);
        o.y += (v0.y * w0 + v1.y * w1) + (v2.y * w2 + v3.y * w3);
        o.z += (v0.z * w0 + v1.z * w1) + (v2.z * w2 + v3.z * w3);
        o.w += (v0.w * w0 + v1.w * w1) + (v2.w * w2 + v3.w * w3);
      }
      for (; s2 < S; ++s2) {
        const float4 v = src[(size_t)s2 * step];
        const float ws = w[s2];
        o.x += v.x * ws, o.y += v.y * ws, o.z += v.z * ws, o.w += v.w * ws;
      }
      *dst = make_uint2(pack_bf16x2(o.x, o.y), pack_bf16x2(o.z, o.w));
    }
  }
  __syncthreads();

  f32x4 acc[NW][MT];
#pragma unroll
  for (int t = 0; t < NW; ++t)
#pragma unroll
    for (int tb = 0; tb < MT; ++tb) acc[t][tb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int k = 0; k < KSTEPS; ++k) {
#pragma unroll
    for (int tb = 0; tb < MT; ++tb) {
      OutFrag b;
      b.u = *(const uint4*)(merged + (tb * 16 + r) * STRIDE + k * 32 + g4 * 8);
#pragma unroll
      for (int t = 0; t < NW; ++t)
        acc[t][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][k].v, b.v, acc[t][tb], 0, 0, 0);
    }
  }
  // acc[t][tb][i] = y[token tb*16 + r][row n0 + t*16 + g4*4 + i of W]
#pragma unroll
  for (int tb = 0; tb < MT; ++tb) {
    const int m = tb * 16 + r;
    if (m >= p.M) continue;
    if (p.fixed_out) {
      fixed_t* sum = p.fixed_out + (size_t)m * p.N;
#pragma unroll
      for (int t = 0; t < NW; ++t) {
        const int n = n0 + t * 16 + g4 * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < p.N) add_fixed(sum + n + i, acc[t][tb][i]);
      }
      continue;
    }
    float* dst = p.out + ((size_t)slice * p.M + m) * p.N;
#pragma unroll
    for (int t = 0; t < NW; ++t) {
      const int n = n0 + t * 16 + g4 * 4;
      if (n + 3 < p.N && (p.N & 3) == 0) {
        *(float4*)(dst + n) = make_float4(acc[t][tb][0], acc[t][tb][1], acc[t][tb][2], acc[t][tb][3]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < p.N) dst[n + i] = acc[t][tb][i];
      }
    }
  }
}

// How many query heads go into one slice: as few as leave at most 16 slices (each slice is a
// partial sum [M, N] the next norm reads), in a count that divides the heads; 0 where this
// kernel does not take the sizes.  `atomic`: the slices are added into the fixed-point
// residual stream, M x N atomic additions each, all slices on the same places: from four
// tokens on, twice the heads a slice where that fits (14 heads of 64 into 896, 8 tokens:
// 0.960 against 0.970 ms a step; one token: no difference).
extern "C" int mk_attention_out_heads_per_slice(int n_q, int n_kv, int d, int M, int N, int atomic) {
  if ((d != 64 && d != 128) || M < 1 || M > 64 || n_q < 1 || n_kv < 1 || n_q % n_kv || N < 16) return 0;
  auto fits = [&](int hp) { return hp <= 4 && n_q % hp == 0 && n_q / hp <= 16 && hp * d <= 512; };
  for (int hp = 1; hp <= 4; hp *= 2) {
    if (!fits(hp)) continue;
    return atomic && M >= 4 && fits(2 * hp) ? 2 * hp : hp;
  }
  return 0;
}

// The most parts per (tile, kv head) mk_attention_out takes for M tokens and this many heads
// per slice: its workgroups keep a weight per (token, head of the slice, part) in LDS.
extern "C" int mk_attention_out_max_parts(int M, int heads_per_slice) {
  if (M < 1 || heads_per_slice < 1) return 0;
  const int most = OUT_MAX_WEIGHTS / (M * heads_per_slice);
  return most > 128 ? 128 : most;
}

template <int D, int HP, int NW>
static void launch_out(const AttnOutParams& p, int n_q, hipStream_t stream) {
  const dim3 grid((p.N + 64 * NW - 1) / (64 * NW), n_q / HP);
  if (p.M <= 16) attn_out_kernel<D, HP, 1, NW><<<grid, 256, 0, stream>>>(p);
  else if (p.M <= 32) attn_out_kernel<D, HP, 2, NW><<<grid, 256, 0, stream>>>(p);
  else attn_out_kernel<D, HP, 4, NW><<<grid, 256, 0, stream>>>(p);
}

extern "C" int mk_attention_out(const float* part_o, const float* part_ml, int parts,
                                const void* w_o, float* out, long long* fixed_out, int M, int N,
                                int n_q, int n_kv, int d, int heads_per_slice, int wide,
                                hipStream_t stream) {
  MK_REQUIRE(parts >= 2 && parts <= mk_attention_out_max_parts(M, heads_per_slice),
             "attention_out: %d parts (2 to %d for %d tokens and %d heads per slice)", parts,
             mk_attention_out_max_parts(M, heads_per_slice), M, heads_per_slice);
  MK_REQUIRE(heads_per_slice > 0 &&
                 heads_per_slice == mk_attention_out_heads_per_slice(n_q, n_kv, d, M, N,
                                                                     fixed_out != nullptr),
             "attention_out: sizes not taken (head size 64 or 128, at most 64 tokens), or another "
             "number of heads per slice than mk_attention_out_heads_per_slice gives");
  MK_REQUIRE(part_o && part_ml && w_o && (out != nullptr) != (fixed_out != nullptr),
             "attention_out: null argument, or not exactly one of the two outputs");
  MK_REQUIRE(((n_q * d) & 7) == 0, "attention_out: rows of W must be 16-byte aligned");
  AttnOutParams p;
  p.part_o = part_o;
  p.part_ml = part_ml;
  p.w = (const bf16_t*)w_o;
  p.out = out;
  p.fixed_out = (fixed_t*)fixed_out;
  p.M = M;
  p.N = N;
  p.n_kv = n_kv;
  p.group = n_q / n_kv;
  p.parts = parts;
#define MK_OUT(D_, HP_)                                                 \
  if (d == D_ && heads_per_slice == HP_) {                              \
    if (wide) launch_out<D_, HP_, 2>(p, n_q, stream);                   \
    else launch_out<D_, HP_, 1>(p, n_q, stream);                        \
  }
  MK_OUT(64, 1) MK_OUT(64, 2) MK_OUT(64, 4) MK_OUT(128, 1) MK_OUT(128, 2) MK_OUT(128, 4)
#undef MK_OUT
  MK_LAUNCH_CHECK("attention_out");
  return 0;
}
