// bfloat16 projections on the matrix cores: y[M,N] = x[M,K] W[N,K]^T, float32 accumulate.
//
// Two kernels:
//
//  * skinny (at most 16 rows of x; the q/k/v projection up to 64): the weights are read once,
//    straight from HBM into the A operand of v_mfma_f32_16x16x32_bf16 (16 rows of W by 32 k
//    per instruction); the few rows of x are the B operand and come out of the L2.  A
//    workgroup owns 16 or 32 rows of W, its wavefronts taking the k-steps in turn.  A
//    workgroup that keeps all of K finishes the job in its epilogue: adds into the float32
//    residual stream, gates (gate/up projection), or adds the bias, rotates and writes q and
//    the paged cache (q/k/v projection).  Otherwise K is split: every slice writes its own
//    float32 partial result [slice, M, N], and whichever kernel consumes the projection
//    (RMSNorm, rotary + cache write) adds the slices up in slice order, so results are
//    reproducible.  It is the kernel of choice for a handful of rows and matrices of modest
//    size; from 8 rows on, and for large matrices, the tiled kernel streams weights faster.
//
//  * tiled: tiles of y per workgroup (256 x 256 down to 64 x 64, whichever is estimated
//    fastest for the problem), K in stages through a ring of LDS buffers that global memory
//    is loaded into directly, several stages ahead of the products.  Epilogues: bfloat16
//    store with bias, float32 store, float32 accumulate into the residual stream, SiLU
//    gating, or float32 partial sums over slices of K.
//
// In both, lane l of a wavefront holds row (l % 16) and k-slots (l / 16) * 8 .. + 8 of an
// operand, so the four lanes of a row read 64 contiguous bytes per load instruction.
#include "common.h"
#include "mercury_kernels.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

union Frag {
  bf16x8 v;
  uint4 u;
};

__device__ __forceinline__ uint4 ld16(const bf16_t* p) { return *(const uint4*)p; }

// ------------------------------------------------------------------------------ skinny

#define SK_WAVES 4  // wavefronts of a workgroup where the grid has many; they share the rows
                    // and split the k-steps.  Kernels whose grid is one workgroup per compute
                    // unit or fewer (SK_ACC, SK_QKV) take 8, for more bytes in flight per unit.

// What a workgroup's rows of W are and what becomes of the result:
//   SK_PARTIAL  rows n0.. of W; out[(slice * M + m) * N + n] float32, one slice of K each.
//   SK_GATED    W is [gate rows | up rows] of N each; tile 0 is gate rows n0.., tile 1 the
//               matching up rows N + n0..; act[m][n] = silu(g) * u in bfloat16
//               (reference: mercury/model/qwen2.py:42).  All of K in the workgroup.
//   SK_ACC      rows n0.. of W; out[m][n] += y (+ bias) in float32: the residual stream takes
//               the projection directly.  All of K in the workgroup.
//   SK_QKV      W is [q heads | k heads | v heads] of d rows each; tile 0 is rows j*16.. of a
//               head's first half and tile 1 the same rows of its second half, so every lane
//               holds both members of a rotation pair: bias, rounding, rotation by the token's
//               position, q to `q_out`, k and v into the paged cache.  All of K.
//   SK_FIXED    rows n0.. of W, one slice of K each; y (+ bias, from slice 0) is added into
//               the fixed-point residual stream out[m][n] with integer atomics.
// NORMED (SK_GATED, SK_QKV, at most 16 rows): x is not read but made: the rows of the
// fixed-point residual stream `h64`, RMS-normalised and weighted as the norm kernel would
// have left them (reference: mercury/model/qwen2.py:27-31), each by one wavefront, into LDS.
enum { SK_PARTIAL = 0, SK_GATED = 1, SK_ACC = 2, SK_QKV = 3, SK_FIXED = 4 };

// Where the q/k/v projection's results go, and how they are rotated on the way.
struct QkvTarget {
  bf16_t* q_out;           // [M, n_q d]
  const float* cos_table;  // [positions, d / 2]
  const float* sin_table;
  const int* positions;    // [M]
  const int* token_seq;    // [M]
  const int* block_table;
  int table_stride;
  bf16_t* k_cache;         // [pages, n_kv, page, d]
  bf16_t* v_cache;         // [pages, n_kv, d, page]
  int page_shift, n_q, n_kv, d, rotate;
};

struct SkinnyArgs : QkvTarget {
  const bf16_t* x;  // [M, K]
  const bf16_t* w;
  void* out;
  int M, N, K, steps_per_slice;
  const void* bias;  // SK_ACC, SK_QKV, SK_FIXED: [N] or null
  int bias_bf16;
  // NORMED
  const fixed_t* h64;   // [M, K]
  const void* norm_w;   // [K]
  int norm_bf16;
  float norm_eps;
};

// The rows of x a NORMED workgroup makes for itself: [M][K + 8] bfloat16 (16 bytes of padding
// a row against bank conflicts).
extern __shared__ __align__(16) unsigned char skinny_rows[];

// g * sigmoid(g) for a result that is rounded to bfloat16 next: the hardware's exponential
// and reciprocal (an ulp or two of float32 each) in place of the library's, a dozen
// instructions less per element of an epilogue that has 80 of them a thread.
// (reference: mercury/model/qwen2.py:42)
__device__ __forceinline__ float silu_for_bf16(float g) {
  return g * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(g * -1.44269504088896340736f));
}

__device__ __forceinline__ float load_scalar(const void* p, int is_bf16, int i) {
  return is_bf16 ? bf16_to_f32(((const bf16_t*)p)[i]) : ((const float*)p)[i];
}

// Where token m's keys and values go: its position and the page that holds it (-1: none).
// Looked up once per token, before any store: the stores might alias the tables for all the
// compiler knows, and it would fetch them again after each.
struct QkvPlace {
  int pos, page;
};

__device__ __forceinline__ QkvPlace qkv_place(const QkvTarget& p, int m) {
  QkvPlace place;
  place.pos = p.positions[m];
  place.page = p.n_kv > 0 ? p.block_table[(size_t)p.token_seq[m] * p.table_stride +
                                          (place.pos >> p.page_shift)]
                          : -1;
  return place;
}

// The rotation of the 4 pairs (dims dd .. dd + 4 and their partners) of a token at the place's
// position: asked for apart from the store, so that a kernel can have the angles on their way
// while it still multiplies.  Heads of values, and models without rotation, turn by nothing.
struct QkvAngles {
  float4 c, s;
};

__device__ __forceinline__ QkvAngles qkv_angles(const QkvTarget& p, const QkvPlace& place, int head,
                                                int dd) {
  QkvAngles a;
  a.c = make_float4(1.f, 1.f, 1.f, 1.f);
  a.s = make_float4(0.f, 0.f, 0.f, 0.f);
  if (p.rotate && head < p.n_q + p.n_kv) {
    const int half = p.d / 2;
    a.c = *(const float4*)(p.cos_table + (size_t)place.pos * half + dd);
    a.s = *(const float4*)(p.sin_table + (size_t)place.pos * half + dd);
  }
  return a;
}

// Token m's values (bias added) at dims dd .. dd + 4 (`lo`) and dd + d/2 .. (`hi`) of head
// `head` of [q heads | k heads | v heads]: rounded to bfloat16 as a stored projection would
// be, q and k rotated by the token's position (the four lanes' dims are 4 rotation pairs), q
// written to q_out, k and v into the paged cache.
// Formulas: reference mercury/model/qwen2.py:57-64, mercury/model/rope.py:19-29.
__device__ __forceinline__ void qkv_store(const QkvTarget& p, const QkvPlace& place,
                                          const QkvAngles& angles, int m, int head, int dd,
                                          float* lo, float* hi) {
  const int d = p.d, half = d / 2;
  const int pos = place.pos;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    lo[i] = Elem<bf16_t>::round(lo[i]);
    hi[i] = Elem<bf16_t>::round(hi[i]);
  }
  const bool is_v = head >= p.n_q + p.n_kv;
  if (p.rotate && !is_v) {
    const float cs[4] = {angles.c.x, angles.c.y, angles.c.z, angles.c.w};
    const float sn[4] = {angles.s.x, angles.s.y, angles.s.z, angles.s.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float u = lo[i], v = hi[i];
      lo[i] = u * cs[i] - v * sn[i];
      hi[i] = v * cs[i] + u * sn[i];
    }
  }
  const ushort4 lo4 = make_ushort4(f32_to_bf16(lo[0]), f32_to_bf16(lo[1]), f32_to_bf16(lo[2]),
                                   f32_to_bf16(lo[3]));
  const ushort4 hi4 = make_ushort4(f32_to_bf16(hi[0]), f32_to_bf16(hi[1]), f32_to_bf16(hi[2]),
                                   f32_to_bf16(hi[3]));
  if (head < p.n_q) {
    bf16_t* dst = p.q_out + (size_t)m * p.n_q * d + head * d + dd;
    *(ushort4*)dst = lo4;
    *(ushort4*)(dst + half) = hi4;
    return;
  }
  const int page = place.page;
  if (page < 0) return;
  const int ps = 1 << p.page_shift, off = pos & (ps - 1);
  if (!is_v) {
    const int kh = head - p.n_q;
    bf16_t* dst = p.k_cache + (((size_t)page * p.n_kv + kh) * ps + off) * d + dd;
    *(ushort4*)dst = lo4;
    *(ushort4*)(dst + half) = hi4;
  } else {
    const int vh = head - p.n_q - p.n_kv;
    bf16_t* dst = p.v_cache + (((size_t)page * p.n_kv + vh) * d + dd) * ps + off;
    const bf16_t l[4] = {lo4.x, lo4.y, lo4.z, lo4.w}, h4[4] = {hi4.x, hi4.y, hi4.z, hi4.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      dst[(size_t)i * ps] = l[i];
      dst[(size_t)(half + i) * ps] = h4[i];
    }
  }
}

// One workgroup: NT tiles of 16 rows of W, its four wavefronts taking the slice's 128-wide
// k-steps in turn (wave w: steps w, w + 4, ...), the next step's loads in flight during the
// current step's products; the wavefronts' results are added through LDS in wave order.
// Product j of a step takes k = step*128 + j*32 + g4*8 .. + 8 from a lane, so that one load
// instruction reads 64 contiguous bytes of each of its 16 rows.
template <int MT, int NT, int EPI, int WAVES, int NORMED = 0, bool ONE_ROW = false>
__global__ __launch_bounds__(64 * WAVES) void gemm_skinny_kernel(SkinnyArgs p) {
  static_assert((EPI != SK_GATED && EPI != SK_QKV) || NT == 2, "paired tiles");
  static_assert(NORMED == 0 || MT == 1, "rows made in LDS: at most 16");
  static_assert(NORMED == 0 || NORMED == 8 || NORMED == 16, "a lane's pairs of a row: 8 or 16");
  __shared__ float red[WAVES - 1][NT * MT * 4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, g4 = lane >> 4;
  const int M = p.M, N = p.N, K = p.K;
  const int slice = blockIdx.y;
  const int step_begin = slice * p.steps_per_slice;
  const int step_end = min((K + 127) / 128, step_begin + p.steps_per_slice);

  // SK_QKV: the head and the 16-row stretch of its halves this workgroup owns.
  const int per_head = EPI == SK_QKV ? p.d / 32 : 1;
  const int head = EPI == SK_QKV ? blockIdx.x / per_head : 0;
  const int dd0 = EPI == SK_QKV ? (blockIdx.x - head * per_head) * 16 : 0;
  const int n0 = EPI == SK_QKV ? head * p.d + dd0 : blockIdx.x * (EPI == SK_GATED ? 16 : 16 * NT);

  const bf16_t* wrow[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    int row;
    if (EPI == SK_GATED) row = t * N + min(n0 + r, N - 1);
    else if (EPI == SK_QKV) row = n0 + t * (p.d / 2) + r;
    else row = min(n0 + t * 16 + r, N - 1);
    wrow[t] = p.w + (size_t)row * K;
  }
  const bf16_t* xrow[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) xrow[t] = NORMED ? nullptr : p.x + (size_t)min(t * 16 + r, M - 1) * K;
  const bf16_t* made = (const bf16_t*)skinny_rows;   // NORMED
  const int made_stride = K + 8, made_row = min(r, M - 1) * made_stride;

  // Eight wavefronts over rows of at most 1,024 (NORMED 8) take one k-step each: no buffers
  // for steps ahead, and with the registers they would take, two workgroups fit a compute
  // unit, so that the gated projection's 304 workgroups run in one round instead of two.
  // (ONE_ROW: at most one row a wavefront, M <= WAVES; the instantiation for more rows keeps
  // the buffers.)
  static_assert(!ONE_ROW || NORMED != 0, "rows made by the workgroup");
  constexpr int DEPTH = (NORMED == 8 && WAVES == 8 && ONE_ROW) ? 1 : (MT == 1 ? 3 : (MT == 2 ? 2 : 1));
  Frag a[DEPTH][NT][4], b[DEPTH][MT][4];
  auto load_w = [&](int buf, int step) {
    const int kk = step * 128 + g4 * 8;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool ok = kk + j * 32 < K;
#pragma unroll
      for (int t = 0; t < NT; ++t)
        a[buf][t][j].u = ok ? ld16(wrow[t] + kk + j * 32) : make_uint4(0, 0, 0, 0);
    }
  };
  auto load_x = [&](int buf, int step) {
    const int kk = step * 128 + g4 * 8;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool ok = kk + j * 32 < K;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        if constexpr (NORMED) {
          b[buf][t][j].u = ok ? *(const uint4*)(made + made_row + kk + j * 32) : make_uint4(0, 0, 0, 0);
        } else {
          b[buf][t][j].u = ok ? ld16(xrow[t] + kk + j * 32) : make_uint4(0, 0, 0, 0);
        }
      }
    }
  };

  // NORMED: the norm's weights at this lane's places and the wavefront's first row of the
  // residual stream are asked for before anything else, so that they are back (from the L2)
  // and worked on while the first weights of W are still on their way from HBM.  (Loads at
  // clamped places and values chosen afterwards: a load under a condition is a branch, and
  // the compiler waits for it before the next.)
  constexpr int HOLD = NORMED ? NORMED : 1;   // rows of up to 128 * HOLD values
  float g[HOLD][2];
  longlong2 v[HOLD];
  if constexpr (NORMED) {
    if (wave < M) {
      if (p.norm_bf16) {
#pragma unroll
        for (int i = 0; i < HOLD; ++i) {
          const uint32_t u = *(const uint32_t*)((const bf16_t*)p.norm_w + min(i * 128 + lane * 2, K - 2));
          g[i][0] = __uint_as_float(u << 16);
          g[i][1] = __uint_as_float(u & 0xffff0000u);
        }
      } else {
#pragma unroll
        for (int i = 0; i < HOLD; ++i) {
          const float2 u = *(const float2*)((const float*)p.norm_w + min(i * 128 + lane * 2, K - 2));
          g[i][0] = u.x;
          g[i][1] = u.y;
        }
      }
#pragma unroll
      for (int i = 0; i < HOLD; ++i)
        v[i] = *(const longlong2*)(p.h64 + (size_t)wave * K + min(i * 128 + lane * 2, K - 2));
    }
  }

  int step = step_begin + wave;
  if (step < step_end) load_w(0, step);

  // SK_QKV: where the tokens' keys and values go and by what their pairs turn is asked for
  // now, by the wavefront that will write them: three trips to memory, each waiting for the
  // one before, that would otherwise follow the products.
  constexpr bool EARLY_PLACE = EPI == SK_QKV && MT <= 2;
  QkvPlace place[MT];
  QkvAngles angles[MT];
  if constexpr (EARLY_PLACE) {
    if (wave == 0) {
#pragma unroll
      for (int tb = 0; tb < MT; ++tb) {
        place[tb] = qkv_place(p, min(tb * 16 + r, M - 1));
        angles[tb] = qkv_angles(p, place[tb], head, dd0 + g4 * 4);
      }
    }
  }

  // SK_QKV: the bias of this lane's eight columns as well, in two loads (asked for one by one
  // behind the products, each load waits for the one before it).
  float bias_lo[4] = {0.f, 0.f, 0.f, 0.f}, bias_hi[4] = {0.f, 0.f, 0.f, 0.f};
  if constexpr (EPI == SK_QKV) {
    if (p.bias && wave == 0) {
      const int at = n0 + g4 * 4, half = p.d / 2;
      if (p.bias_bf16) {
        const ushort4 l = *(const ushort4*)((const bf16_t*)p.bias + at);
        const ushort4 h = *(const ushort4*)((const bf16_t*)p.bias + at + half);
        bias_lo[0] = bf16_to_f32(l.x), bias_lo[1] = bf16_to_f32(l.y);
        bias_lo[2] = bf16_to_f32(l.z), bias_lo[3] = bf16_to_f32(l.w);
        bias_hi[0] = bf16_to_f32(h.x), bias_hi[1] = bf16_to_f32(h.y);
        bias_hi[2] = bf16_to_f32(h.z), bias_hi[3] = bf16_to_f32(h.w);
      } else {
        const float4 l = *(const float4*)((const float*)p.bias + at);
        const float4 h = *(const float4*)((const float*)p.bias + at + half);
        bias_lo[0] = l.x, bias_lo[1] = l.y, bias_lo[2] = l.z, bias_lo[3] = l.w;
        bias_hi[0] = h.x, bias_hi[1] = h.y, bias_hi[2] = h.z, bias_hi[3] = h.w;
      }
    }
  }

  // SK_ACC: the values the result is added to are asked for now, by the wavefront that will
  // write them, so that the epilogue does not wait for them.
  const bool vec_out = (N & 3) == 0;
  float4 old[NT][MT];
  if constexpr (EPI == SK_ACC) {
    if (wave == 0 && vec_out) {
#pragma unroll
      for (int ta = 0; ta < NT; ++ta)
#pragma unroll
        for (int tb = 0; tb < MT; ++tb) {
          const int m = tb * 16 + r, n = n0 + ta * 16 + g4 * 4;
          old[ta][tb] = (m < M && n + 3 < N) ? *(const float4*)((const float*)p.out + (size_t)m * N + n)
                                             : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
  }

  // NORMED: wavefront w makes rows w, w + WAVES, ...: a lane holds its two values of every
  // 128 of the row (at most 2,048 wide: eight or sixteen loads, all in flight at once; the norm's
  // weights at the same places are shared by every row of the wavefront), adds up their
  // squares, and leaves the normalised, weighted, rounded values in LDS.  The lane layout is
  // the same whichever wavefront takes the row, so a row's x does not depend on the batch.
  // The weights of W this wavefront multiplies first are on their way meanwhile.
  if constexpr (NORMED) {
#pragma unroll
    for (int d = 1; d < DEPTH - 1; ++d)
      if (step + d * WAVES < step_end) load_w(d, step + d * WAVES);
    bf16_t* rows_out = (bf16_t*)skinny_rows;
    for (int m = wave; m < M; m += ONE_ROW ? M : WAVES) {
      if (m != wave) {
#pragma unroll
        for (int i = 0; i < HOLD; ++i)
          v[i] = *(const longlong2*)(p.h64 + (size_t)m * K + min(i * 128 + lane * 2, K - 2));
      }
      float f[HOLD][2], ss = 0.f;
#pragma unroll
      for (int i = 0; i < HOLD; ++i) {
        const bool in = i * 128 + lane * 2 < K;
        f[i][0] = in ? from_fixed(v[i].x) : 0.f;
        f[i][1] = in ? from_fixed(v[i].y) : 0.f;
        ss += f[i][0] * f[i][0] + f[i][1] * f[i][1];
      }
      const float rstd = rsqrtf(wave_sum(ss) / (float)K + p.norm_eps);
#pragma unroll
      for (int i = 0; i < HOLD; ++i) {
        const int k0 = i * 128 + lane * 2;
        if (k0 < K) {
          *(uint32_t*)(rows_out + (size_t)m * made_stride + k0) =
              pack_bf16x2(Elem<bf16_t>::round(f[i][0] * rstd) * g[i][0],
                          Elem<bf16_t>::round(f[i][1] * rstd) * g[i][1]);
        }
      }
    }
    __syncthreads();
  }

  if (step < step_end) load_x(0, step);

  f32x4 acc[NT][MT];
#pragma unroll
  for (int ta = 0; ta < NT; ++ta)
#pragma unroll
    for (int tb = 0; tb < MT; ++tb) acc[ta][tb] = (f32x4){0.f, 0.f, 0.f, 0.f};

  auto products = [&](int buf) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int ta = 0; ta < NT; ++ta)
#pragma unroll
        for (int tb = 0; tb < MT; ++tb)
          acc[ta][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[buf][ta][j].v, b[buf][tb][j].v,
                                                                acc[ta][tb], 0, 0, 0);
  };
  // DEPTH k-steps per wavefront between a load's issue and its use: three for one tile of x
  // rows, two for two; with three or four tiles of x rows the extra buffers would cost
  // wavefronts per SIMD, and one step at a time is faster.
  if constexpr (DEPTH == 1) {
    for (; step < step_end; step += WAVES) {
      products(0);
      if (step + WAVES < step_end) {
        load_w(0, step + WAVES);
        load_x(0, step + WAVES);
      }
    }
  } else {
#pragma unroll
    for (int d = 1; d < DEPTH - 1; ++d) {
      if (step + d * WAVES < step_end) {
        if constexpr (!NORMED) load_w(d, step + d * WAVES);
        load_x(d, step + d * WAVES);
      }
    }
    for (; step < step_end; step += DEPTH * WAVES) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int now = step + d * WAVES, ahead = now + (DEPTH - 1) * WAVES;
        if (now < step_end) {
          if (ahead < step_end) {
            load_w((d + DEPTH - 1) % DEPTH, ahead);
            load_x((d + DEPTH - 1) % DEPTH, ahead);
          }
          products(d);
        }
      }
    }
  }

  if (wave > 0) {
#pragma unroll
    for (int ta = 0; ta < NT; ++ta)
#pragma unroll
      for (int tb = 0; tb < MT; ++tb)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave - 1][(ta * MT + tb) * 4 + i][lane] = acc[ta][tb][i];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int v = 0; v < WAVES - 1; ++v)
#pragma unroll
    for (int ta = 0; ta < NT; ++ta)
#pragma unroll
      for (int tb = 0; tb < MT; ++tb)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[ta][tb][i] += red[v][(ta * MT + tb) * 4 + i][lane];

  // acc[ta][tb][i] = y[m = tb*16 + r][row g4*4 + i of tile ta]
#pragma unroll
  for (int tb = 0; tb < MT; ++tb) {
    const int m = tb * 16 + r;
    if (m >= M) continue;
    if constexpr (EPI == SK_GATED) {
      bf16_t* dst = (bf16_t*)p.out + (size_t)m * N;
      const int n = n0 + g4 * 4;
      bf16_t o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float g = Elem<bf16_t>::round(acc[0][tb][i]), u = Elem<bf16_t>::round(acc[1][tb][i]);
        o[i] = f32_to_bf16(Elem<bf16_t>::round(silu_for_bf16(g)) * u);
      }
      if (n + 3 < N && (N & 3) == 0) {
        *(ushort4*)(dst + n) = make_ushort4(o[0], o[1], o[2], o[3]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < N) dst[n + i] = o[i];
      }
    } else if constexpr (EPI == SK_QKV) {
      // Both halves of 4 rotation pairs of one head: dims dd.. and dd + d/2..
      const int half = p.d / 2, dd = dd0 + g4 * 4;
      float lo[4], hi[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        lo[i] = acc[0][tb][i] + bias_lo[i];
        hi[i] = acc[1][tb][i] + bias_hi[i];
      }
      if constexpr (!EARLY_PLACE) {
        place[tb] = qkv_place(p, m);
        angles[tb] = qkv_angles(p, place[tb], head, dd);
      }
      qkv_store(p, place[tb], angles[tb], m, head, dd, lo, hi);
    } else if constexpr (EPI == SK_FIXED) {
      fixed_t* dst = (fixed_t*)p.out + (size_t)m * N;
#pragma unroll
      for (int ta = 0; ta < NT; ++ta) {
        const int n = n0 + ta * 16 + g4 * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (n + i >= N) continue;
          float y = acc[ta][tb][i];
          if (p.bias && slice == 0) y += load_scalar(p.bias, p.bias_bf16, n + i);
          add_fixed(dst + n + i, y);
        }
      }
    } else {
      float* dst = (float*)p.out + ((size_t)(EPI == SK_PARTIAL ? slice : 0) * M + m) * N;
#pragma unroll
      for (int ta = 0; ta < NT; ++ta) {
        const int n = n0 + ta * 16 + g4 * 4;
        float y[4] = {acc[ta][tb][0], acc[ta][tb][1], acc[ta][tb][2], acc[ta][tb][3]};
        if constexpr (EPI == SK_ACC) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (p.bias && n + i < N) y[i] += load_scalar(p.bias, p.bias_bf16, n + i);
        }
        if (n + 3 < N && vec_out) {
          float4* q = (float4*)(dst + n);
          if constexpr (EPI == SK_ACC) {
            const float4 o = old[ta][tb];
            *q = make_float4(o.x + y[0], o.y + y[1], o.z + y[2], o.w + y[3]);
          } else {
            *q = make_float4(y[0], y[1], y[2], y[3]);
          }
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < N) dst[n + i] = EPI == SK_ACC ? dst[n + i] + y[i] : y[i];
        }
      }
    }
  }
}

// What a skinny projection over `slices` slices of K costs, relative to one workgroup
// streaming 32 whole rows of W: the chip serves every compute unit about the same share of
// HBM bandwidth, so the time is that of the unit with the most bytes, workgroups being dealt
// out over the 256 units in turn; every further slice adds a little (partial results, x read
// again, a workgroup's start and finish).  Measured at 5120 x 27648, 8 rows: 71, 77, 57, 62, 65, 59, 60, 56 us for 1..8
// slices, which is this function's shape.
static double skinny_split_cost(int tiles, int slices, int M, int K) {
  const long groups = (long)tiles * slices;
  const double extra = 0.02 * (slices - 1) + 2.0 * slices * M / K;   // the second: partial results
  return (double)((groups + 255) / 256) / slices * (1.0 + extra);
}

// Slices of K for the plain skinny projection: the count with the least cost above, every
// wavefront of a workgroup with at least one k-step, and no more partial results than the
// weights are worth (slices * M * 4 bytes per output column against K * 2).
extern "C" int mk_linear_skinny_slices(int M, int N, int K) {
  const int tiles = (N + 31) / 32;
  const int steps = (K + 127) / 128;
  int limit = (steps + SK_WAVES - 1) / SK_WAVES;
  const int cap = K / (8 * (M > 0 ? M : 1));
  if (limit > cap) limit = cap;
  if (limit > 16) limit = 16;
  int best = 1;
  double best_cost = skinny_split_cost(tiles, 1, M, K);
  for (int slices = 2; slices <= limit; ++slices) {
    const int per = (steps + slices - 1) / slices;
    if ((steps + per - 1) / per != slices) continue;   // not a count the steps divide into
    const double cost = skinny_split_cost(tiles, slices, M, K);
    if (cost < best_cost - 1e-9) best = slices, best_cost = cost;
  }
  return best;
}

// Whether a projection added straight into the residual stream should keep all of K in one
// workgroup of 16 rows (no partial results): for at most 16 rows of x, when the matrix is so
// small that latency, not bandwidth, is what its kernel costs, or when 16-row workgroups
// spread over the compute units clearly more evenly than the best split does (they stream a
// little slower than 32-row workgroups over half of K: 32.7 against 29.6 us at
// 3584 x 18944).  With more rows of x every workgroup re-reads so much of x from the L2 that
// fewer, larger workgroups over slices of K are faster.
extern "C" int mk_linear_skinny_unsplit(int M, int N, int K) {
  if (M > 16) return 0;
  if ((double)N * K * 2.0 <= 4.0e6) return 1;
  const int tiles16 = (N + 15) / 16;
  const double whole = 0.5 * ((tiles16 + 255) / 256);
  const double split = skinny_split_cost((N + 31) / 32, mk_linear_skinny_slices(M, N, K), M, K);
  return whole < 0.9 * split;
}

template <int NT, int EPI, int NORMED = 0, int WAVES = 0, bool ONE_ROW = false>
static void launch_skinny(const SkinnyArgs& a, dim3 grid, hipStream_t stream, size_t lds = 0) {
  // 8 wavefronts where the grid is small; with 3 or 4 tiles of x rows they would not fit
  // the register file.  More than 16 rows of x only for the q/k/v projection: the others
  // take the tiled kernel there.
  constexpr int W = WAVES ? WAVES : ((EPI == SK_ACC || EPI == SK_QKV || NORMED) ? 8 : SK_WAVES);
  const int tiles = (a.M + 15) / 16;
  if (tiles == 1) {
    gemm_skinny_kernel<1, NT, EPI, W, NORMED, ONE_ROW><<<grid, 64 * W, lds, stream>>>(a);
  } else if constexpr (EPI == SK_QKV && !NORMED) {
    if (tiles == 2) gemm_skinny_kernel<2, NT, EPI, W><<<grid, 64 * W, 0, stream>>>(a);
    else if (tiles == 3) gemm_skinny_kernel<3, NT, EPI, SK_WAVES><<<grid, 64 * SK_WAVES, 0, stream>>>(a);
    else gemm_skinny_kernel<4, NT, EPI, SK_WAVES><<<grid, 64 * SK_WAVES, 0, stream>>>(a);
  }
}

static SkinnyArgs skinny_args(const void* x, const void* w, void* out, int M, int N, int K,
                              int steps_per_slice) {
  SkinnyArgs a = {};
  a.x = (const bf16_t*)x;
  a.w = (const bf16_t*)w;
  a.out = out;
  a.M = M;
  a.N = N;
  a.K = K;
  a.steps_per_slice = steps_per_slice;
  return a;
}

extern "C" int mk_linear_skinny(const void* x, const void* w, float* out, int M, int N, int K,
                                int slices, hipStream_t stream) {
  MK_REQUIRE(M >= 1 && M <= 16, "skinny projection: M=%d outside 1..16", M);
  MK_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "skinny projection: K=%d must be a multiple of 8", K);
  const int steps = (K + 127) / 128;
  MK_REQUIRE(slices >= 1 && slices <= steps, "skinny projection: %d slices for %d steps", slices,
             steps);
  const int per = (steps + slices - 1) / slices;
  MK_REQUIRE((per * (slices - 1)) < steps, "skinny projection: an empty slice");
  MK_REQUIRE(slices <= 65535, "skinny projection: too many slices");
  launch_skinny<2, SK_PARTIAL>(skinny_args(x, w, out, M, N, K, per),
                                      dim3((N + 31) / 32, slices), stream);
  MK_LAUNCH_CHECK("linear_skinny");
  return 0;
}

// h64[M, N] (the fixed-point residual stream) += x W^T (+ bias), 1 <= M <= 16, K in `slices`
// slices as mk_linear_skinny takes them: no partial results are left, and the sum does not
// depend on the order the slices finish in.
extern "C" int mk_linear_skinny_fixed(const void* x, const void* w, const void* bias,
                                      int bias_dtype, long long* h64, int M, int N, int K,
                                      int slices, hipStream_t stream) {
  MK_REQUIRE(M >= 1 && M <= 16, "skinny projection: M=%d outside 1..16", M);
  MK_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "skinny projection: K=%d must be a multiple of 8", K);
  MK_REQUIRE(bias_dtype == MK_F32 || bias_dtype == MK_BF16, "skinny projection: bias dtype");
  MK_REQUIRE(x && w && h64, "skinny projection: null argument");
  const int steps = (K + 127) / 128;
  MK_REQUIRE(slices >= 1 && slices <= steps && slices <= 65535,
             "skinny projection: %d slices for %d steps", slices, steps);
  const int per = (steps + slices - 1) / slices;
  MK_REQUIRE((per * (slices - 1)) < steps, "skinny projection: an empty slice");
  SkinnyArgs a = skinny_args(x, w, h64, M, N, K, per);
  a.bias = bias;
  a.bias_bf16 = bias_dtype == MK_BF16;
  launch_skinny<2, SK_FIXED>(a, dim3((N + 31) / 32, slices), stream);
  MK_LAUNCH_CHECK("linear_skinny_fixed");
  return 0;
}

// out[M, N] (float32) += x W^T (+ bias), 1 <= M <= 16, all of K in each workgroup.
extern "C" int mk_linear_skinny_acc(const void* x, const void* w, const void* bias,
                                    int bias_dtype, float* out, int M, int N, int K,
                                    hipStream_t stream) {
  MK_REQUIRE(M >= 1 && M <= 16, "skinny projection: M=%d outside 1..16", M);
  MK_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "skinny projection: K=%d must be a multiple of 8", K);
  MK_REQUIRE(bias_dtype == MK_F32 || bias_dtype == MK_BF16, "skinny projection: bias dtype");
  SkinnyArgs a = skinny_args(x, w, out, M, N, K, (K + 127) / 128);
  a.bias = bias;
  a.bias_bf16 = bias_dtype == MK_BF16;
  // 16 rows a workgroup until those alone are more workgroups than the chip holds at once
  if ((N + 15) / 16 <= 1024)
    launch_skinny<1, SK_ACC>(a, dim3((N + 15) / 16, 1), stream);
  else
    launch_skinny<2, SK_ACC>(a, dim3((N + 31) / 32, 1), stream);
  MK_LAUNCH_CHECK("linear_skinny_acc");
  return 0;
}

// act[M, I] = silu(x Wg^T) * (x Wu^T) for W = [Wg | Wu] stacked as [2 I, K], 1 <= M <= 16.
extern "C" int mk_gated_skinny(const void* x, const void* w, void* act, int M, int inter, int K,
                               hipStream_t stream) {
  MK_REQUIRE(M >= 1 && M <= 16, "gated projection: M=%d outside 1..16", M);
  MK_REQUIRE(inter > 0 && K > 0 && K % 8 == 0, "gated projection: K=%d must be a multiple of 8",
             K);
  launch_skinny<2, SK_GATED>(skinny_args(x, w, act, M, inter, K, (K + 127) / 128),
                             dim3((inter + 15) / 16, 1), stream);
  MK_LAUNCH_CHECK("gated_skinny");
  return 0;
}

// The widest row (K) the projections below take for M rows: the rows they make live in LDS.
extern "C" int mk_skinny_normed_max_k(int M) {
  if (M < 1 || M > 16) return 0;
  const int fits = ((48 * 1024) / (2 * M) - 8) / 8 * 8;
  return fits < 2048 ? fits : 2048;   // a lane holds its share of a row in registers
}

static int set_normed(SkinnyArgs& a, const long long* h64, const void* norm_w, int norm_dtype,
                      float eps) {
  MK_REQUIRE(h64 && norm_w, "normed projection: null argument");
  MK_REQUIRE((uintptr_t)h64 % 16 == 0 && (uintptr_t)norm_w % 8 == 0,
             "normed projection: the residual stream must be 16-byte aligned, the norm's weights 8");
  MK_REQUIRE(norm_dtype == MK_F32 || norm_dtype == MK_BF16, "normed projection: weight dtype");
  MK_REQUIRE(a.M >= 1 && a.M <= 16 && a.K <= mk_skinny_normed_max_k(a.M),
             "normed projection: %d rows of %d are more than its workgroups hold (K <= %d)", a.M,
             a.K, mk_skinny_normed_max_k(a.M));
  a.h64 = (const fixed_t*)h64;
  a.norm_w = norm_w;
  a.norm_bf16 = norm_dtype == MK_BF16;
  a.norm_eps = eps;
  return 0;
}

static size_t normed_lds(const SkinnyArgs& a) { return (size_t)a.M * (a.K + 8) * 2; }

// mk_gated_skinny on x = rmsnorm(h64) * norm_w, made by every workgroup for itself from the
// fixed-point residual stream h64 [M, K].
extern "C" int mk_gated_skinny_normed(const long long* h64, const void* norm_w, int norm_dtype,
                                      float eps, const void* w, void* act, int M, int inter, int K,
                                      hipStream_t stream) {
  MK_REQUIRE(inter > 0 && K > 0 && K % 8 == 0, "gated projection: K=%d must be a multiple of 8",
             K);
  MK_REQUIRE(w && act, "gated projection: null argument");
  SkinnyArgs a = skinny_args(nullptr, w, act, M, inter, K, (K + 127) / 128);
  if (set_normed(a, h64, norm_w, norm_dtype, eps)) return 1;
  const dim3 grid((inter + 15) / 16, 1);
  if (K <= 1024) {
    if (M <= 4) launch_skinny<2, SK_GATED, 8, 4>(a, grid, stream, normed_lds(a));
    else if (M <= 8) launch_skinny<2, SK_GATED, 8, 8, true>(a, grid, stream, normed_lds(a));
    else launch_skinny<2, SK_GATED, 8, 8>(a, grid, stream, normed_lds(a));
  } else {
    if (M <= 4) launch_skinny<2, SK_GATED, 16, 4>(a, grid, stream, normed_lds(a));
    else launch_skinny<2, SK_GATED, 16, 8>(a, grid, stream, normed_lds(a));
  }
  MK_LAUNCH_CHECK("gated_skinny_normed");
  return 0;
}

// The q/k/v projection of 1 <= M <= 64 tokens with everything that follows it: bias, rotation
// of q and k by the token's position (full head width, or none), q [M, n_q d] out, k and v
// into the paged cache (n_kv = 0: queries only).  W is [(n_q + 2 n_kv) d, K].
// Formulas: reference mercury/model/qwen2.py:57-64, mercury/model/rope.py:19-29.
static int qkv_skinny_any(const void* x, const long long* h64, const void* norm_w, int norm_dtype,
                          float eps, const void* w, const void* bias, int bias_dtype,
                          void* q_out, const float* cos_table, const float* sin_table,
                          int table_positions, const int* positions, const int* token_seq,
                          const int* block_table, int table_stride, void* k_cache,
                          void* v_cache, int page_size, int n_q, int n_kv, int d, int rotate,
                          int M, int K, hipStream_t stream) {
  MK_REQUIRE(M >= 1 && M <= 64, "qkv projection: M=%d outside 1..64", M);
  MK_REQUIRE(n_q > 0 && n_kv >= 0 && d > 0 && d % 32 == 0,
             "qkv projection: head size %d is not a multiple of 32", d);
  MK_REQUIRE(K > 0 && K % 8 == 0, "qkv projection: K=%d must be a multiple of 8", K);
  MK_REQUIRE(!rotate || (cos_table && sin_table && table_positions > 0),
             "qkv projection: rotation needs the angle tables");
  MK_REQUIRE(n_kv == 0 || (k_cache && v_cache && block_table && mk_is_pow2(page_size)),
             "qkv projection: the cache and a power-of-two page size are required");
  MK_REQUIRE(bias_dtype == MK_F32 || bias_dtype == MK_BF16, "qkv projection: bias dtype");
  MK_REQUIRE((uintptr_t)bias % 16 == 0, "qkv projection: the bias must be 16-byte aligned");
  const int N = (n_q + 2 * n_kv) * d;
  SkinnyArgs a = skinny_args(x, w, nullptr, M, N, K, (K + 127) / 128);
  a.bias = bias;
  a.bias_bf16 = bias_dtype == MK_BF16;
  a.q_out = (bf16_t*)q_out;
  a.cos_table = cos_table;
  a.sin_table = sin_table;
  a.positions = positions;
  a.token_seq = token_seq;
  a.block_table = block_table;
  a.table_stride = table_stride;
  a.k_cache = (bf16_t*)k_cache;
  a.v_cache = (bf16_t*)v_cache;
  a.page_shift = mk_log2(page_size > 0 ? page_size : 1);
  a.n_q = n_q;
  a.n_kv = n_kv;
  a.d = d;
  a.rotate = rotate;
  const dim3 grid((n_q + 2 * n_kv) * (d / 32), 1);
  if (h64) {
    if (set_normed(a, h64, norm_w, norm_dtype, eps)) return 1;
    if (K <= 1024 && M <= 8) launch_skinny<2, SK_QKV, 8, 8, true>(a, grid, stream, normed_lds(a));
    else if (K <= 1024) launch_skinny<2, SK_QKV, 8>(a, grid, stream, normed_lds(a));
    else launch_skinny<2, SK_QKV, 16>(a, grid, stream, normed_lds(a));
  } else {
    MK_REQUIRE(x, "qkv projection: null argument");
    launch_skinny<2, SK_QKV>(a, grid, stream);
  }
  MK_LAUNCH_CHECK("qkv_skinny");
  return 0;
}

extern "C" int mk_qkv_skinny(const void* x, const void* w, const void* bias, int bias_dtype,
                             void* q_out, const float* cos_table, const float* sin_table,
                             int table_positions, const int* positions, const int* token_seq,
                             const int* block_table, int table_stride, void* k_cache,
                             void* v_cache, int page_size, int n_q, int n_kv, int d, int rotate,
                             int M, int K, hipStream_t stream) {
  return qkv_skinny_any(x, nullptr, nullptr, MK_F32, 0.f, w, bias, bias_dtype, q_out, cos_table,
                        sin_table, table_positions, positions, token_seq, block_table,
                        table_stride, k_cache, v_cache, page_size, n_q, n_kv, d, rotate, M, K,
                        stream);
}

// mk_qkv_skinny on x = rmsnorm(h64) * norm_w, made by every workgroup for itself from the
// fixed-point residual stream h64 [M, K]; at most 16 tokens.
extern "C" int mk_qkv_skinny_normed(const long long* h64, const void* norm_w, int norm_dtype,
                                    float eps, const void* w, const void* bias, int bias_dtype,
                                    void* q_out, const float* cos_table, const float* sin_table,
                                    int table_positions, const int* positions,
                                    const int* token_seq, const int* block_table,
                                    int table_stride, void* k_cache, void* v_cache, int page_size,
                                    int n_q, int n_kv, int d, int rotate, int M, int K,
                                    hipStream_t stream) {
  MK_REQUIRE(h64, "qkv projection: null argument");
  return qkv_skinny_any(nullptr, h64, norm_w, norm_dtype, eps, w, bias, bias_dtype, q_out,
                        cos_table, sin_table, table_positions, positions, token_seq, block_table,
                        table_stride, k_cache, v_cache, page_size, n_q, n_kv, d, rotate, M, K,
                        stream);
}

// ------------------------------------------------------------------------------- tiled

enum { EPI_BF16 = 0, EPI_F32 = 1, EPI_ACC = 2, EPI_GATED = 3, EPI_QKV = 4 };

// a / b for 0 <= a < 2^22 and 0 < b: the float quotient is off by less than one, which one
// step either way repairs.  A dozen instructions where the general division is forty, on
// the way to a workgroup's first loads.
__device__ __forceinline__ int small_div(int a, int b) {
  const int q = (int)((float)a * __builtin_amdgcn_rcpf((float)b));
  const int r = a - q * b;
  return q + (r >= b ? 1 : 0) - (r < 0 ? 1 : 0);
}

#define TILE_K 64  // k per stage: a tile row is 128 bytes in LDS, one cache line of the operand

// Sixteen zero bytes: what a lane fetches for k past K, so that a last, partial stage
// multiplies zeros.
__device__ __attribute__((aligned(16))) const unsigned int tiled_zero_chunk[4] = {0u, 0u, 0u, 0u};

// The LDS buffer of stage S of the ring: x rows first, then W rows.  Static buffers, one per
// stage and instantiation.
template <int S, int ELEMS>
__device__ __forceinline__ bf16_t* tiled_stage_buffer() {
  __shared__ __attribute__((aligned(1024))) bf16_t buffer[ELEMS];
  return buffer;
}

// s_waitcnt immediate: at most `loads` vector-memory loads outstanding, every LDS operation
// complete (vmcnt is split over bits 3:0 and 15:14, lgkmcnt is bits 11:8, expcnt 6:4 unused).
#define TILED_WAIT(loads) (((loads) & 15) | (((loads) >> 4) << 14) | (7 << 4) | (0 << 8))

// One workgroup of WM x WN wavefronts computes a BM x BN tile of y.  K advances 64 per stage
// through a ring of STAGES LDS buffers.  The tiles travel from global memory straight into
// LDS (global_load_lds_dwordx4: each lane's 16 bytes land at M0 + 16 * lane, no register in
// between), so a stage's loads can be asked for STAGES - 1 stages before they are used at no
// cost in registers: the latency of a load under full traffic is more than a stage's worth
// of products.  One wavefront instruction fills 8 tile rows; which 16 bytes of its row a
// lane fetches is permuted by the row pair's index, so that the operand reads of 16 rows hit
// 16 different bank groups.  Per stage: wait until this wavefront's loads of the stage have
// landed, barrier (now everybody's have, and everybody is done with the previous stage's
// buffer), ask for the stage STAGES - 1 ahead into that buffer while multiplying.
//
// The loads are inline assembly: the compiler counts its own vector-memory operations only
// (there are none inside the loop), and the waits for these are written out by hand.  The
// compiler may move LDS reads past a load but not past the barrier, which is fenced: a load
// writes the buffer whose reads ended before the barrier.
//
// EPI_GATED: W is [gate rows | up rows] of N each.  A wavefront's BN / WN tile rows are half
// gate rows and half the matching up rows, so its accumulators hold both; the epilogue writes
// act[m][n] = silu(g) * u in bfloat16 (reference: mercury/model/qwen2.py:42).
//
// EPI_QKV: W is [q heads | k heads | v heads] of d rows each.  A wavefront's tile rows are
// half rows from the first halves of heads and half the rows d / 2 further, so its
// accumulators hold both members of every rotation pair; the epilogue adds the bias,
// rotates, and writes q and the paged cache (qkv_store).  N counts the rows of W.
template <int BM, int BN, int STAGES, int WM, int WN, int SPREAD, int EPI, typename TBIAS>
__global__ __launch_bounds__(64 * WM * WN) void gemm_tiled_kernel(const bf16_t* __restrict__ x,
                                                                  const bf16_t* __restrict__ w,
                                                                  const TBIAS* __restrict__ bias,
                                                                  void* __restrict__ out_, int M,
                                                                  int N, int K, int ldo,
                                                                  int slice_stages,
                                                                  QkvTarget target) {
  constexpr int WAVES = WM * WN, TK = TILE_K;
  constexpr int NI = (BM + BN) / 8 / WAVES;                 // load instructions per wavefront and stage
  static_assert((BM + BN) % (8 * WAVES) == 0 && WAVES % 2 == 0, "tile rows divide over the wavefronts");
  static_assert(BM % 16 == 0 && (STAGES - 2) * NI < 64, "tile shape");
  constexpr int ELEMS = (BM + BN) * TK;
  constexpr int TM = BM / WM / 16, TN = BN / WN / 16;       // MFMA tiles per wavefront
  constexpr bool PAIRED = EPI == EPI_GATED || EPI == EPI_QKV;
  static_assert(!PAIRED || TN % 2 == 0, "both members of a pair of rows in one wavefront");
  constexpr int WIDTH = BN / WN;                            // W rows per wavefront
  constexpr int COLS = PAIRED ? BN / 2 : BN;                // output columns (pairs) per tile
  // Where the 8 elements from k-chunk `chunk` of tile row `row` lie in a stage buffer.
  auto lds_at = [](int row, int chunk) { return row * TK + (((chunk ^ (row >> 1)) & 7) << 3); };

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, g4 = lane >> 4;
  const int wm = (wave / WN) * (BM / WM), wn = (wave % WN) * WIDTH;
  // Which tile: workgroups go to the 8 XCDs in turn, each with an L2 of its own, so the
  // launch index is first renumbered to give every XCD a contiguous stretch of tiles, and the
  // stretch is walked in bands of 8 tile rows, column by column, so that the tiles in flight
  // on an XCD share rows of x and rows of W in its L2.
  int tile_m, tile_n;
  {
    const int gx = gridDim.x, gy = gridDim.y, total = gx * gy;
    const int id = blockIdx.y * gx + blockIdx.x;
    const int per = (total + 7) / 8, tall = total % 8;
    const int xcd = id % 8, local = id / 8;
    const int renum = (tall == 0 || xcd < tall) ? xcd * per + local
                                                : tall * per + (xcd - tall) * (per - 1) + local;
    const int band = 8 * gx, first = renum / band * 8;
    const int height = min(gy - first, 8), in_band = renum % band;
    tile_m = first + in_band % height;
    tile_n = in_band / height;
  }
  const int m0 = tile_m * BM, n0 = tile_n * COLS;

  // Load instruction i of this wavefront fills buffer rows [8 j, 8 j + 8), j = wave + WAVES i;
  // lane l lands on chunk l % 8 of row 8 j + l / 8, and fetches the k-chunk that belongs
  // there.  (row >> 1) & 7 = (4 j + l / 16) & 7 has the same value for every i, WAVES being
  // even, and so has the k-chunk.
  const int chunk = ((lane & 7) ^ (4 * wave + (lane >> 4))) & 7;
  const bf16_t* src[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int row = (wave + WAVES * i) * 8 + (lane >> 3);
    if (row < BM) {
      src[i] = x + (size_t)min(m0 + row, M - 1) * K + chunk * 8;
    } else {
      int wrow = row - BM;
      if (EPI == EPI_GATED) {  // per wavefront: WIDTH / 2 gate rows, then the matching up rows
        const int col = min(n0 + wrow / WIDTH * (WIDTH / 2) + wrow % (WIDTH / 2), N - 1);
        wrow = (wrow % WIDTH < WIDTH / 2 ? 0 : N) + col;
      } else if (EPI == EPI_QKV) {  // WIDTH / 2 rows of heads' first halves, then their partners
        const int half = target.d / 2;
        const int pair = min(n0 + wrow / WIDTH * (WIDTH / 2) + wrow % (WIDTH / 2), N / 2 - 1);
        const int head = small_div(pair, half);     // (a model's q/k/v width is far below 2^22)
        wrow = head * target.d + (pair - head * half) + (wrow % WIDTH < WIDTH / 2 ? 0 : half);
      } else {
        wrow = min(n0 + wrow, N - 1);
      }
      src[i] = w + (size_t)wrow * K + chunk * 8;
    }
  }
  // gridDim.z slices of K, slice_stages stages each, every slice with a result of its own
  // (EPI_F32 only): out[slice][M][ldo].
  const int all_steps = (K + TK - 1) / TK;
  const int first_step = blockIdx.z * slice_stages;
  const int steps = min(slice_stages, all_steps - first_step);
  const bool ragged = K % TK != 0 && first_step + steps == all_steps;
  const bool past_k = (all_steps - 1) * TK + chunk * 8 >= K;  // this lane's part of a partial last stage
#pragma unroll
  for (int i = 0; i < NI; ++i) src[i] += (size_t)first_step * TK;
  if (EPI == EPI_F32) out_ = (float*)out_ + (size_t)blockIdx.z * M * ldo;

  f32x4 acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; ++a)
#pragma unroll
    for (int b = 0; b < TN; ++b) acc[a][b] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // Stages past the last are asked for as the last one again: they land in buffers nobody
  // reads any more, and every iteration has the same number of loads to count.
  // Load instructions [first, last) of stage s.
  auto fetch = [&](int s, bf16_t* buffer, int first, int last) __attribute__((always_inline)) {
    const int stage = min(s, steps - 1);
    const bool partial = ragged && stage == steps - 1;      // the same for the whole workgroup
#pragma unroll
    for (int i = first; i < last; ++i) {
      const unsigned int dst = (unsigned int)(uintptr_t)(
          __attribute__((address_space(3))) void*)(buffer + (wave + WAVES * i) * 512);
      const bf16_t* from = src[i] + stage * TK;
      if (partial) from = past_k ? (const bf16_t*)tiled_zero_chunk : from;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                   :
                   : "s"(dst), "v"(from)
                   : "m0");
    }
  };
  // The products of a stage, with the loads of stage `ahead` handed out between them: all up
  // front (SPREAD 0), half before each half of k (1), or a few before every row of MFMA
  // tiles (2).  Requests that arrive in one burst per stage take longer to be served, but a
  // stage asked for earlier is there earlier: the 256 x 256 tile, with one stage of
  // lookahead, is 2-5 % faster with all of them up front (8,192 cubed: 853 against 900 us).
  auto products = [&](const bf16_t* buffer, int ahead, bf16_t* into) __attribute__((always_inline)) {
    const bf16_t* xs = buffer;
    const bf16_t* ws = buffer + BM * TK;
    constexpr int HALVES = TK / 32, SLOTS = HALVES * TM;
    if (SPREAD == 0) fetch(ahead, into, 0, NI);
#pragma unroll
    for (int kk = 0; kk < TK; kk += 32) {
      if (SPREAD == 1) fetch(ahead, into, kk / 32 * NI / HALVES, (kk / 32 + 1) * NI / HALVES);
      Frag a[TM], b[TN];
#pragma unroll
      for (int t = 0; t < TM; ++t)
        a[t].u = *(const uint4*)(&xs[lds_at(wm + t * 16 + r, kk / 8 + g4)]);
#pragma unroll
      for (int t = 0; t < TN; ++t)
        b[t].u = *(const uint4*)(&ws[lds_at(wn + t * 16 + r, kk / 8 + g4)]);
#pragma unroll
      for (int ta = 0; ta < TM; ++ta) {
        const int slot = kk / 32 * TM + ta;
        if (SPREAD == 2) fetch(ahead, into, slot * NI / SLOTS, (slot + 1) * NI / SLOTS);
#pragma unroll
        for (int tb = 0; tb < TN; ++tb)
          // A = W rows (n), B = x rows (m): the result holds 4 consecutive n per lane.
          acc[ta][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[tb].v, a[ta].v, acc[ta][tb],
                                                                0, 0, 0);
      }
    }
  };

  bf16_t* ring[STAGES];
  ring[0] = tiled_stage_buffer<0, ELEMS>();
  ring[1] = tiled_stage_buffer<1, ELEMS>();
  if constexpr (STAGES > 2) ring[2] = tiled_stage_buffer<2, ELEMS>();
  if constexpr (STAGES > 3) ring[3] = tiled_stage_buffer<3, ELEMS>();
  static_assert(STAGES >= 2 && STAGES <= 4, "two to four stages");

#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s) fetch(s, ring[s], 0, NI);
  for (int s0 = 0; s0 < steps; s0 += STAGES) {
#pragma unroll
    for (int u = 0; u < STAGES; ++u) {   // unrolled: every buffer of the ring is a constant
      if (s0 + u < steps) {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(TILED_WAIT((STAGES - 2) * NI));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        products(ring[u], s0 + u + STAGES - 1, ring[(u + STAGES - 1) % STAGES]);
      }
    }
  }

  // acc[ta][tb][i] = y[m = m0 + wm + ta*16 + r][tile column wn + tb*16 + g4*4 + i]
  //
  // What the q/k/v epilogue reads (the tokens' places in the cache, their angles, the bias)
  // is asked for before its first store: for all the compiler knows a store may change what a
  // later load reads, so a load that follows a store in the program waits for it, and the
  // three trips to memory per row of tiles become three per tile (1152 x 896 at 2,048 rows:
  // 15.8 us against 17.6).
  if constexpr (EPI == EPI_QKV) {
    const int half = target.d / 2;
    QkvPlace place[TM];
#pragma unroll
    for (int ta = 0; ta < TM; ++ta) place[ta] = qkv_place(target, min(m0 + wm + ta * 16 + r, M - 1));
    // The widest tiles have no registers to spare for a row of tiles' bias and angles at
    // once: theirs are asked for tile by tile.
    constexpr bool AHEAD = TN / 2 <= 3;
    constexpr int HELD = AHEAD ? TN / 2 : 1;
    int head[TN / 2], dd[TN / 2];
    float blo[HELD][4], bhi[HELD][4];
    auto bias_of = [&](int tb, float (&lo)[4], float (&hi)[4]) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        lo[i] = bias ? Elem<TBIAS>::load(bias + head[tb] * target.d + dd[tb] + i) : 0.f;
        hi[i] = bias ? Elem<TBIAS>::load(bias + head[tb] * target.d + half + dd[tb] + i) : 0.f;
      }
    };
#pragma unroll
    for (int tb = 0; tb < TN / 2; ++tb) {
      const int pair = min(n0 + wn / 2 + tb * 16 + g4 * 4, N / 2 - 4);   // 4 pairs, all of one head
      head[tb] = small_div(pair, half);
      dd[tb] = pair - head[tb] * half;
      if constexpr (AHEAD) bias_of(tb, blo[tb], bhi[tb]);
    }
#pragma unroll
    for (int ta = 0; ta < TM; ++ta) {
      const int m = m0 + wm + ta * 16 + r;
      QkvAngles angles[HELD];
      if constexpr (AHEAD) {
#pragma unroll
        for (int tb = 0; tb < TN / 2; ++tb) angles[tb] = qkv_angles(target, place[ta], head[tb], dd[tb]);
      }
      if (m >= M) continue;
#pragma unroll
      for (int tb = 0; tb < TN / 2; ++tb) {
        if (n0 + wn / 2 + tb * 16 + g4 * 4 >= N / 2) continue;
        const int at = AHEAD ? tb : 0;
        if constexpr (!AHEAD) {
          bias_of(tb, blo[0], bhi[0]);
          angles[0] = qkv_angles(target, place[ta], head[tb], dd[tb]);
        }
        float lo[4], hi[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          lo[i] = acc[ta][tb][i] + blo[at][i];
          hi[i] = acc[ta][tb + TN / 2][i] + bhi[at][i];
        }
        qkv_store(target, place[ta], angles[at], m, head[tb], dd[tb], lo, hi);
      }
    }
    return;
  }
  // The bias of this lane's columns, asked for in one go and at clamped places (a load under
  // a condition is a branch that the compiler waits behind before the next load).
  float col_bias[EPI == EPI_GATED ? 1 : TN][4];
  if constexpr (EPI != EPI_GATED) {
#pragma unroll
    for (int tb = 0; tb < TN; ++tb)
#pragma unroll
      for (int i = 0; i < 4; ++i) col_bias[tb][i] = 0.f;
    if (bias != nullptr) {
#pragma unroll
      for (int tb = 0; tb < TN; ++tb)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          col_bias[tb][i] = Elem<TBIAS>::load(bias + min(n0 + wn + tb * 16 + g4 * 4 + i, N - 1));
    }
  }
#pragma unroll
  for (int ta = 0; ta < TM; ++ta) {
    const int m = m0 + wm + ta * 16 + r;
    // EPI_ACC: the values a row tile's results are added to, all of the tile's loads in
    // flight at once (one by one, each behind the store before it, a wavefront makes TM x TN
    // trips to memory in a row).  Rows and columns past the end read a clamped place that
    // nothing is made of.
    float4 old[EPI == EPI_ACC ? TN : 1];
    const bool old_held = EPI == EPI_ACC && (ldo & 3) == 0 && N >= 4;
    if constexpr (EPI == EPI_ACC) {
      if (old_held) {
        const float* row = (const float*)out_ + (size_t)min(m, M - 1) * ldo;
#pragma unroll
        for (int tb = 0; tb < TN; ++tb)
          old[tb] = *(const float4*)(row + min(n0 + wn + tb * 16 + g4 * 4, (N - 4) & ~3));
      }
    }
    if (m >= M) continue;
    if (EPI == EPI_GATED) {
#pragma unroll
      for (int tb = 0; tb < TN / 2; ++tb) {
        const int n = n0 + wn / 2 + tb * 16 + g4 * 4;
        bf16_t* dst = (bf16_t*)out_ + (size_t)m * ldo + n;
        float o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float g = Elem<bf16_t>::round(acc[ta][tb][i]);
          const float u = Elem<bf16_t>::round(acc[ta][tb + TN / 2][i]);
          o[i] = Elem<bf16_t>::round(silu_for_bf16(g)) * u;
        }
        if (n + 3 < N && (ldo & 3) == 0) {
          *(uint2*)dst = make_uint2(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]));
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < N) dst[i] = f32_to_bf16(o[i]);
        }
      }
      continue;
    }
#pragma unroll
    for (int tb = 0; tb < TN; ++tb) {
      const int n = n0 + wn + tb * 16 + g4 * 4;
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = acc[ta][tb][i] + col_bias[tb][i];
      const bool whole = n + 3 < N && (ldo & 3) == 0;
      if (EPI == EPI_BF16) {
        bf16_t* dst = (bf16_t*)out_ + (size_t)m * ldo + n;
        if (whole) {
          *(uint2*)dst = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < N) dst[i] = f32_to_bf16(v[i]);
        }
      } else {
        float* dst = (float*)out_ + (size_t)m * ldo + n;
        if (whole) {
          float4 o = make_float4(v[0], v[1], v[2], v[3]);
          if constexpr (EPI == EPI_ACC) {
            o.x += old[tb].x;
            o.y += old[tb].y;
            o.z += old[tb].z;
            o.w += old[tb].w;
          }
          *(float4*)dst = o;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < N) dst[i] = (EPI == EPI_ACC ? dst[i] : 0.f) + v[i];
        }
      }
    }
  }
}

// Tile configurations, by index.  `rate` is what one workgroup sustains on a busy chip in
// TFLOP/s, `alone` what it sustains with a compute unit to itself, `resident` how many
// workgroups a compute unit holds (LDS decides); measured on problems of many tiles with
// weights that no cache holds, as a model's are.
struct TiledConfig {
  int bm, bn, resident;
  float rate, alone;
};
#define TILED_CONFIGS 10
static const TiledConfig tiled_configs[TILED_CONFIGS] = {
    {256, 256, 1, 5.03f, 5.03f},  // 0: 2 stages (128 KB), 16 wavefronts
    {128, 256, 1, 4.7f, 4.7f},    // 1: 3 stages (144 KB), 8 wavefronts
    {128, 128, 1, 3.75f, 3.75f},  // 2: 3 stages (96 KB), 8 wavefronts
    {128, 128, 2, 2.03f, 2.8f},   // 3: 2 stages (64 KB), 4 wavefronts
    {64, 64, 2, 1.2f, 2.0f},      // 4: 4 stages (64 KB), 4 wavefronts
    {64, 128, 1, 2.14f, 2.14f},   // 5: 4 stages (96 KB), 4 wavefronts
    {256, 192, 1, 4.9f, 4.9f},    // 6: 2 stages (112 KB), 8 wavefronts: for widths that 256 divides badly
    {128, 192, 1, 4.45f, 4.45f},  // 7: 3 stages (120 KB), 8 wavefronts
    {64, 32, 3, 0.6f, 1.2f},      // 8: 4 stages (48 KB), 4 wavefronts: small matrices, few rows
    // 9: 2 stages (144 KB), 8 wavefronts of 64 x 160.  The most products per byte a stage
    // brings, which is what a kernel waiting for its stages wants: 18944 x 3584 gated at 2,048
    // rows 448 us against 488 in 256 x 256 tiles, 4864 x 896 45 against 54 in 256 x 192.
    {256, 320, 1, 5.5f, 5.5f},
};

template <int BM, int BN, int STAGES, int WM, int WN, int SPREAD, int EPI>
static void launch_tiled_cfg(const void* x, const void* w, const void* bias, int bias_dtype,
                             void* out, int M, int N, int K, int ldo, int slices,
                             const QkvTarget& target, hipStream_t stream) {
  constexpr int COLS = (EPI == EPI_GATED || EPI == EPI_QKV) ? BN / 2 : BN;
  const int cols = EPI == EPI_QKV ? N / 2 : N;   // q/k/v: the grid counts pairs of rows
  const int all_steps = (K + TILE_K - 1) / TILE_K;
  const int slice_stages = (all_steps + slices - 1) / slices;
  dim3 grid((cols + COLS - 1) / COLS, (M + BM - 1) / BM, (all_steps + slice_stages - 1) / slice_stages);
  if (bias && bias_dtype == MK_BF16)
    gemm_tiled_kernel<BM, BN, STAGES, WM, WN, SPREAD, EPI, bf16_t><<<grid, 64 * WM * WN, 0, stream>>>(
        (const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias, out, M, N, K, ldo, slice_stages, target);
  else
    gemm_tiled_kernel<BM, BN, STAGES, WM, WN, SPREAD, EPI, float><<<grid, 64 * WM * WN, 0, stream>>>(
        (const bf16_t*)x, (const bf16_t*)w, (const float*)bias, out, M, N, K, ldo, slice_stages, target);
}

template <int EPI>
static void launch_tiled(int config, const void* x, const void* w, const void* bias,
                         int bias_dtype, void* out, int M, int N, int K, int ldo, int slices,
                         hipStream_t stream, const QkvTarget& target = QkvTarget()) {
  switch (config) {
    case 0: launch_tiled_cfg<256, 256, 2, 4, 4, 0, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, slices, target, stream); break;
    case 1: launch_tiled_cfg<128, 256, 3, 2, 4, 2, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, slices, target, stream); break;
    case 2: launch_tiled_cfg<128, 128, 3, 2, 4, 2, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, slices, target, stream); break;
    case 3: launch_tiled_cfg<128, 128, 2, 2, 2, 1, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, slices, target, stream); break;
    case 4: launch_tiled_cfg<64, 64, 4, 2, 2, 2, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, slices, target, stream); break;
    case 5: launch_tiled_cfg<64, 128, 4, 1, 4, 0, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, slices, target, stream); break;
    case 6: launch_tiled_cfg<256, 192, 2, 4, 2, 1, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, slices, target, stream); break;
    case 7: launch_tiled_cfg<128, 192, 3, 4, 2, 2, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, slices, target, stream); break;
    case 9: launch_tiled_cfg<256, 320, 2, 4, 2, 1, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, slices, target, stream); break;
    default: launch_tiled_cfg<64, 32, 4, 4, 1, 0, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, slices, target, stream); break;
  }
}

// The estimated time, in microseconds, of y[M, cols] over K in configuration t with K cut
// into `slices`.  A tile covers `bn / halves` columns (halves = 2 when gate and up rows share
// a tile) and moves `out_bytes` per element in its epilogue.  Tiles are dealt to the 256
// compute units; a tile costs its products at the configuration's rate plus a start (the
// first loads' latency) and a finish (the epilogue, at what one workgroup streams: about
// 35 GB/s); of two resident workgroups one's start and finish hide behind the other's
// products, and an odd last one runs alone.
static double tiled_time(const TiledConfig& t, int M, int cols, int K, int halves, int out_bytes,
                         int slices) {
  const int width = t.bn / halves;
  const long tiles = (long)((M + t.bm - 1) / t.bm) * ((cols + width - 1) / width) * slices;
  const bool few = tiles <= 4 * 256;
  const double per_unit = few ? (double)((tiles + 255) / 256) : tiles / 256.0 + 0.5;
  const double products = 2.0 * t.bm * t.bn * K * 1e-6 / slices;        // MFLOP
  const double edges = 1.5 + (double)t.bm * width * out_bytes / 35e3;  // microseconds
  // With few rows of x the weights are the work: a compute unit's tiles stream their rows of
  // W at the unit's share of HBM bandwidth (about 26 GB/s; tiles of 64 rows a little less,
  // x being read again for each).  18944 x 3584 gated at 32 rows: 57.6 us in 64 x 64 tiles
  // (3 a unit), 66.8 in 64 x 128 (2 a unit); 27648 x 5120: 117.5 (4) against 108.4 (2).
  // (With several tile rows the rows of W are shared through the L2 and this is no bound.)
  // The largest tiles (8 wavefronts, three stages of 48 KB in flight) draw about 33 GB/s, and
  // the chip as a whole gives these kernels about 5.9 TB/s: 27648 x 5120 gated at 64 rows runs
  // 106 us in 128 x 256 tiles (216 units busy), 118 in 64 x 128, 135 in 64 x 64; 18944 x 3584:
  // 60, 70, 64.
  const double unit_rate = t.bm * t.bn >= 128 * 256 ? 33e3 : (t.bn >= 128 ? 26e3 : 22.5e3);
  const double tile_bytes = (double)t.bn * K * 2.0 / slices;
  const double streaming =
      M > t.bm ? 0.0 : fmax(per_unit * tile_bytes / unit_rate, tiles * tile_bytes / 5.9e6);
  // Paired rows (gate and up) halve the columns a tile covers, so x is read twice as often:
  // the small tiles, two to a unit, lose about a fifth of their rate to that
  // (512 x 18944 x 3584 gated: 194 us in 128 x 128 tiles, 167 in 128 x 256).
  const double slower = halves == 2 && t.resident == 2 ? 0.8 : 1.0;
  const double rate = t.rate * slower, alone = t.alone * slower;
  double time;
  if (t.resident == 1) {
    time = per_unit * (products / rate + edges);
  } else if (few) {
    const long n = (long)per_unit;
    time = (n / 2) * (products / rate + edges / 2) + (n % 2) * (products / alone + edges);
  } else {
    time = per_unit / 2 * (products / rate + edges / 2);
  }
  return time > streaming ? time : streaming;
}

// The configuration with the least estimated time, K whole.
static int tiled_config_for(int M, int cols, int K, int halves, int out_bytes) {
  int best = -1;
  double best_time = 0.0;
  for (int c = 0; c < TILED_CONFIGS; ++c) {
    // Few rows of x: tiles of 128 rows multiply padding, which costs nothing while the weights
    // are the work, but only the paired 128 x 256 and 128 x 192 tiles stream them faster than
    // the 64-row tiles do (the head, 152064 x 5120 at 64 rows: 319 us against 306 in 64 x 128);
    // of the two, the one whose tiles spread better over the compute units (18944 x 3584 gated
    // at 64 rows: 198 tiles of 192 rows 54 us, 148 of 256 rows 61; 27648 x 5120: 145 and 106).
    if (M <= 64 && tiled_configs[c].bm > 64 && !(halves == 2 && (c == 1 || c == 7))) continue;
    const double time = tiled_time(tiled_configs[c], M, cols, K, halves, out_bytes, 1);
    if (best < 0 || time < best_time) best = c, best_time = time;
  }
  return best;
}

// Configuration and number of slices of K (each with a float32 result of its own, for a
// consumer that adds them up) with the least estimated time: for few rows of x over a long K,
// where whole-K tiles are too few to occupy the chip.  Every slice keeps at least 8 stages.
static void tiled_plan_sliced(int M, int N, int K, int* config, int* slices) {
  const int all_steps = (K + TILE_K - 1) / TILE_K;
  double best_time = 0.0;
  *config = -1, *slices = 1;
  for (int c = 0; c < TILED_CONFIGS; ++c) {
    if (M <= 64 && tiled_configs[c].bm > 64) continue;
    for (int s = 1; s <= 16 && (s == 1 || all_steps / s >= 8); ++s) {
      const int per = (all_steps + s - 1) / s;
      if ((all_steps + per - 1) / per != s) continue;
      // a slice more costs a little by itself, and whoever adds the partial results up has to
      // read them (just written, they come at about 7 TB/s)
      const double adding = s > 1 ? (double)s * M * N * 4.0 / 7e6 : 0.0;
      const double time =
          tiled_time(tiled_configs[c], M, N, K, 1, 4, s) * (1.0 + 0.02 * (s - 1)) + adding;
      if (*config < 0 || time < best_time) *config = c, *slices = s, best_time = time;
    }
  }
}

extern "C" int mk_linear_tiled_configs(void) { return TILED_CONFIGS; }

extern "C" int mk_gated_tiled_config(int M, int inter, int K) {
  return tiled_config_for(M, inter, K, 2, 2);
}

extern "C" int mk_linear_tiled_config(int M, int N, int K, int out_bytes) {
  return tiled_config_for(M, N, K, 1, out_bytes);
}

extern "C" int mk_linear_tiled_slices(int M, int N, int K) {
  int config, slices;
  tiled_plan_sliced(M, N, K, &config, &slices);
  return slices;
}

// out[slices, M, N] (float32): partial sums of x W^T over `slices` slices of K
// (mk_linear_tiled_slices says how many pay), for a consumer that adds them in slice order.
extern "C" int mk_linear_tiled_partials(const void* x, const void* w, float* out, int M, int N,
                                        int K, int slices, hipStream_t stream) {
  MK_REQUIRE(M > 0 && N > 0 && K > 0 && K % 8 == 0,
             "tiled projection: K=%d must be a multiple of 8 (M=%d N=%d)", K, M, N);
  MK_REQUIRE((M + 63) / 64 <= 65535, "tiled projection: M=%d too large for one launch", M);
  int config, planned;
  tiled_plan_sliced(M, N, K, &config, &planned);
  const int all_steps = (K + TILE_K - 1) / TILE_K;
  const int per = (all_steps + (slices > 0 ? slices : 1) - 1) / (slices > 0 ? slices : 1);
  MK_REQUIRE(slices >= 1 && slices <= 1024 && (all_steps + per - 1) / per == slices,
             "tiled projection: %d stages of K do not divide into %d slices", all_steps, slices);
  if (slices != planned) config = tiled_config_for(M, N, (K + slices - 1) / slices, 1, 4);
  launch_tiled<EPI_F32>(config, x, w, nullptr, MK_F32, out, M, N, K, N, slices, stream);
  MK_LAUNCH_CHECK("linear_tiled_partials");
  return 0;
}

// act[M, inter] (bfloat16) = silu(x Wg^T) * (x Wu^T) for w = [Wg | Wu] stacked [2 inter, K].
extern "C" int mk_gated_tiled(const void* x, const void* w, void* act, int M, int inter, int K,
                              int config, hipStream_t stream) {
  MK_REQUIRE(M > 0 && inter > 0 && K > 0 && K % 8 == 0,
             "gated projection: K=%d must be a multiple of 8 (M=%d I=%d)", K, M, inter);
  MK_REQUIRE((M + 63) / 64 <= 65535, "gated projection: M=%d too large for one launch", M);
  if (config < 0) config = tiled_config_for(M, inter, K, 2, 2);
  MK_REQUIRE(config < TILED_CONFIGS, "gated projection: no configuration %d", config);
  launch_tiled<EPI_GATED>(config, x, w, nullptr, MK_F32, act, M, inter, K, inter, 1, stream);
  MK_LAUNCH_CHECK("gated_tiled");
  return 0;
}

// The q/k/v projection of any number of tokens with everything that follows it, as
// mk_qkv_skinny: bias, rotation of q and k by the token's position (full head width, or
// none), q [M, n_q d] out, k and v into the paged cache (n_kv = 0: queries only).
extern "C" int mk_qkv_tiled(const void* x, const void* w, const void* bias, int bias_dtype,
                            void* q_out, const float* cos_table, const float* sin_table,
                            int table_positions, const int* positions, const int* token_seq,
                            const int* block_table, int table_stride, void* k_cache,
                            void* v_cache, int page_size, int n_q, int n_kv, int d, int rotate,
                            int M, int K, int config, hipStream_t stream) {
  MK_REQUIRE(M >= 1 && (M + 63) / 64 <= 65535, "qkv projection: M=%d", M);
  MK_REQUIRE(n_q > 0 && n_kv >= 0 && d > 0 && d % 32 == 0,
             "qkv projection: head size %d is not a multiple of 32", d);
  MK_REQUIRE(K > 0 && K % 8 == 0, "qkv projection: K=%d must be a multiple of 8", K);
  MK_REQUIRE(!rotate || (cos_table && sin_table && table_positions > 0),
             "qkv projection: rotation needs the angle tables");
  MK_REQUIRE(n_kv == 0 || (k_cache && v_cache && block_table && mk_is_pow2(page_size)),
             "qkv projection: the cache and a power-of-two page size are required");
  MK_REQUIRE(bias_dtype == MK_F32 || bias_dtype == MK_BF16, "qkv projection: bias dtype");
  const int N = (n_q + 2 * n_kv) * d;
  QkvTarget t = {};
  t.q_out = (bf16_t*)q_out;
  t.cos_table = cos_table;
  t.sin_table = sin_table;
  t.positions = positions;
  t.token_seq = token_seq;
  t.block_table = block_table;
  t.table_stride = table_stride;
  t.k_cache = (bf16_t*)k_cache;
  t.v_cache = (bf16_t*)v_cache;
  t.page_shift = mk_log2(page_size > 0 ? page_size : 1);
  t.n_q = n_q;
  t.n_kv = n_kv;
  t.d = d;
  t.rotate = rotate;
  if (config < 0) config = tiled_config_for(M, N / 2, K, 2, 2);
  MK_REQUIRE(config < TILED_CONFIGS, "qkv projection: no configuration %d", config);
  launch_tiled<EPI_QKV>(config, x, w, bias, bias_dtype, nullptr, M, N, K, N, 1, stream, t);
  MK_LAUNCH_CHECK("qkv_tiled");
  return 0;
}

extern "C" int mk_linear_tiled(const void* x, const void* w, const void* bias, int bias_dtype,
                               void* out, int out_dtype, int accumulate, int M, int N, int K,
                               int ldo, int config, hipStream_t stream) {
  MK_REQUIRE(M > 0 && N > 0 && K > 0 && K % 8 == 0,
             "tiled projection: K=%d must be a multiple of 8 (M=%d N=%d)", K, M, N);
  MK_REQUIRE(ldo >= N, "tiled projection: leading dimension %d smaller than N=%d", ldo, N);
  MK_REQUIRE(!accumulate || out_dtype == MK_F32,
             "tiled projection: accumulation needs a float32 destination");
  MK_REQUIRE((M + 63) / 64 <= 65535, "tiled projection: M=%d too large for one launch", M);
  if (config < 0)
    config = mk_linear_tiled_config(M, N, K, accumulate ? 8 : (out_dtype == MK_F32 ? 4 : 2));
  MK_REQUIRE(config < TILED_CONFIGS, "tiled projection: no configuration %d", config);
  if (accumulate)
    launch_tiled<EPI_ACC>(config, x, w, bias, bias_dtype, out, M, N, K, ldo, 1, stream);
  else if (out_dtype == MK_F32)
    launch_tiled<EPI_F32>(config, x, w, bias, bias_dtype, out, M, N, K, ldo, 1, stream);
  else if (out_dtype == MK_BF16)
    launch_tiled<EPI_BF16>(config, x, w, bias, bias_dtype, out, M, N, K, ldo, 1, stream);
  else
    MK_REQUIRE(false, "tiled projection: unknown out dtype %d", out_dtype);
  MK_LAUNCH_CHECK("linear_tiled");
  return 0;
}
