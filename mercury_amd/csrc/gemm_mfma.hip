// bfloat16 projections on the matrix cores: y[M,N] = x[M,K] W[N,K]^T, float32 accumulate.
//
// Two kernels for the two regimes of an inference step:
//
//  * skinny (M <= 64, decoding): the weights are read once, straight from HBM into the A
//    operand of v_mfma_f32_16x16x32_bf16 (16 rows of W by 32 k per instruction); the few rows
//    of x are the B operand and come out of the L2.  A workgroup owns 16 or 32 rows of W, its
//    wavefronts taking the k-steps in turn.  Where those workgroups occupy the chip, or the
//    matrix is too small for bandwidth to matter, a workgroup keeps all of K and finishes the
//    job in its epilogue: adds into the float32 residual stream, gates (gate/up projection),
//    or adds the bias, rotates and writes q and the paged cache (q/k/v projection).
//    Otherwise K is split:
//    every slice writes its own float32 partial result [slice, M, N], and whichever kernel
//    consumes the projection (RMSNorm, rotary + cache write) adds the slices up in slice
//    order, so results are reproducible.
//
//  * tiled (M > 64, prompts): tiles of y per workgroup of four wavefronts (128 x 128, or
//    smaller when the matrix would otherwise leave compute units idle), K in stages through
//    two LDS buffers with the next stage's global loads in flight during the current stage's
//    products.  Epilogues: bfloat16 store with bias, float32 store, or float32 accumulate
//    into the residual stream.
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
enum { SK_PARTIAL = 0, SK_GATED = 1, SK_ACC = 2, SK_QKV = 3 };

struct SkinnyArgs {
  const bf16_t* x;  // [M, K]
  const bf16_t* w;
  void* out;
  int M, N, K, steps_per_slice;
  const void* bias;  // SK_ACC, SK_QKV: [N] or null
  int bias_bf16;
  // SK_QKV
  bf16_t* q_out;
  const float* cos_table;
  const float* sin_table;
  const int* positions;
  const int* token_seq;
  const int* block_table;
  int table_stride;
  bf16_t* k_cache;
  bf16_t* v_cache;
  int page_shift, n_q, n_kv, d, rotate;
};

__device__ __forceinline__ float load_scalar(const void* p, int is_bf16, int i) {
  return is_bf16 ? bf16_to_f32(((const bf16_t*)p)[i]) : ((const float*)p)[i];
}

// One workgroup: NT tiles of 16 rows of W, its four wavefronts taking the slice's 128-wide
// k-steps in turn (wave w: steps w, w + 4, ...), the next step's loads in flight during the
// current step's products; the wavefronts' results are added through LDS in wave order.
// Product j of a step takes k = step*128 + j*32 + g4*8 .. + 8 from a lane, so that one load
// instruction reads 64 contiguous bytes of each of its 16 rows.
template <int MT, int NT, int EPI, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void gemm_skinny_kernel(SkinnyArgs p) {
  static_assert((EPI != SK_GATED && EPI != SK_QKV) || NT == 2, "paired tiles");
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
  for (int t = 0; t < MT; ++t) xrow[t] = p.x + (size_t)min(t * 16 + r, M - 1) * K;

  constexpr int DEPTH = MT == 1 ? 3 : (MT == 2 ? 2 : 1);
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
      for (int t = 0; t < MT; ++t)
        b[buf][t][j].u = ok ? ld16(xrow[t] + kk + j * 32) : make_uint4(0, 0, 0, 0);
    }
  };

  int step = step_begin + wave;
  if (step < step_end) load_w(0, step);

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
        load_w(d, step + d * WAVES);
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
        o[i] = f32_to_bf16(Elem<bf16_t>::round(g / (1.f + expf(-g))) * u);
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
      const int d = p.d, half = d / 2, dd = dd0 + g4 * 4;
      const int pos = p.positions[m];
      float lo[4], hi[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float u = acc[0][tb][i], v = acc[1][tb][i];
        if (p.bias) {
          u += load_scalar(p.bias, p.bias_bf16, n0 + g4 * 4 + i);
          v += load_scalar(p.bias, p.bias_bf16, n0 + half + g4 * 4 + i);
        }
        lo[i] = Elem<bf16_t>::round(u);
        hi[i] = Elem<bf16_t>::round(v);
      }
      const bool is_v = head >= p.n_q + p.n_kv;
      if (p.rotate && !is_v) {
        const float4 c = *(const float4*)(p.cos_table + (size_t)pos * half + dd);
        const float4 s = *(const float4*)(p.sin_table + (size_t)pos * half + dd);
        const float cs[4] = {c.x, c.y, c.z, c.w}, sn[4] = {s.x, s.y, s.z, s.w};
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
      } else {
        const int page = p.block_table[(size_t)p.token_seq[m] * p.table_stride + (pos >> p.page_shift)];
        if (page < 0) continue;
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

// Slices of K for the plain skinny projection: enough workgroups to fill the chip (about
// 512), every wavefront of a workgroup with at least one k-step, and no more partial results
// than the weights are worth (slices * M * 4 bytes per output column against K * 2).
extern "C" int mk_linear_skinny_slices(int M, int N, int K) {
  const int tiles = (N + 31) / 32;
  const int steps = (K + 127) / 128;
  int slices = (512 + tiles - 1) / tiles;
  const int by_steps = (steps + SK_WAVES - 1) / SK_WAVES;
  if (slices > by_steps) slices = by_steps;
  const int cap = K / (8 * (M > 0 ? M : 1));
  if (slices > cap) slices = cap;
  if (slices < 1) slices = 1;
  const int per = (steps + slices - 1) / slices;
  return (steps + per - 1) / per;
}

// Whether a projection added straight into the residual stream should keep all of K in one
// workgroup (no partial results, one kernel less to wait for): for at most 16 rows of x,
// when 16-row workgroups alone occupy most of the chip, or when the matrix is so small that
// latency, not bandwidth, is what its kernel costs.  One workgroup alone pulls about 35 GB/s;
// with more rows of x every workgroup re-reads so much of x from the L2 that fewer, larger
// workgroups over slices of K are faster.
extern "C" int mk_linear_skinny_unsplit(int M, int N, int K) {
  const int tiles16 = (N + 15) / 16;
  return M <= 16 && (tiles16 >= 192 || (double)N * K * 2.0 <= 4.0e6);
}

template <int NT, int EPI>
static void launch_skinny(const SkinnyArgs& a, dim3 grid, hipStream_t stream) {
  // 8 wavefronts where the grid is small; with 3 or 4 tiles of x rows they would not fit
  // the register file.
  constexpr int W = (EPI == SK_ACC || EPI == SK_QKV) ? 8 : SK_WAVES;
  switch ((a.M + 15) / 16) {
    case 1: gemm_skinny_kernel<1, NT, EPI, W><<<grid, 64 * W, 0, stream>>>(a); break;
    case 2: gemm_skinny_kernel<2, NT, EPI, W><<<grid, 64 * W, 0, stream>>>(a); break;
    case 3: gemm_skinny_kernel<3, NT, EPI, SK_WAVES><<<grid, 64 * SK_WAVES, 0, stream>>>(a); break;
    default: gemm_skinny_kernel<4, NT, EPI, SK_WAVES><<<grid, 64 * SK_WAVES, 0, stream>>>(a); break;
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
  MK_REQUIRE(M >= 1 && M <= 64, "skinny projection: M=%d outside 1..64", M);
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

// out[M, N] (float32) += x W^T (+ bias), 1 <= M <= 64, all of K in each workgroup.
extern "C" int mk_linear_skinny_acc(const void* x, const void* w, const void* bias,
                                    int bias_dtype, float* out, int M, int N, int K,
                                    hipStream_t stream) {
  MK_REQUIRE(M >= 1 && M <= 64, "skinny projection: M=%d outside 1..64", M);
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

// act[M, I] = silu(x Wg^T) * (x Wu^T) for W = [Wg | Wu] stacked as [2 I, K], 1 <= M <= 64.
extern "C" int mk_gated_skinny(const void* x, const void* w, void* act, int M, int inter, int K,
                               hipStream_t stream) {
  MK_REQUIRE(M >= 1 && M <= 64, "gated projection: M=%d outside 1..64", M);
  MK_REQUIRE(inter > 0 && K > 0 && K % 8 == 0, "gated projection: K=%d must be a multiple of 8",
             K);
  launch_skinny<2, SK_GATED>(skinny_args(x, w, act, M, inter, K, (K + 127) / 128),
                             dim3((inter + 15) / 16, 1), stream);
  MK_LAUNCH_CHECK("gated_skinny");
  return 0;
}

// The q/k/v projection of 1 <= M <= 64 tokens with everything that follows it: bias, rotation
// of q and k by the token's position (full head width, or none), q [M, n_q d] out, k and v
// into the paged cache (n_kv = 0: queries only).  W is [(n_q + 2 n_kv) d, K].
// Formulas: reference mercury/model/qwen2.py:57-64, mercury/model/rope.py:19-29.
extern "C" int mk_qkv_skinny(const void* x, const void* w, const void* bias, int bias_dtype,
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
  launch_skinny<2, SK_QKV>(a, grid, stream);
  MK_LAUNCH_CHECK("qkv_skinny");
  return 0;
}

// ------------------------------------------------------------------------------- tiled

enum { EPI_BF16 = 0, EPI_F32 = 1, EPI_ACC = 2, EPI_GATED = 3 };

// One workgroup of 4 wavefronts (WM x WN) computes a BM x BN tile of y; K advances TK per
// stage through two LDS buffers, the next stage's global loads in flight during the current
// stage's products.  The 16-byte chunks of a tile row are permuted in LDS (or the row padded)
// so that operand reads of 16 rows and staging writes of 2 rows hit distinct banks.
// EPI_GATED: W is [gate rows | up rows] of N each; a tile holds BN / 2 gate rows and the BN / 2
// matching up rows, every wavefront spans the tile's whole width (WN = 1), and the epilogue
// writes act[m][n] = silu(g) * u in bfloat16 (reference: mercury/model/qwen2.py:42).
template <int BM, int BN, int TK, int WM, int WN, int EPI, typename TBIAS>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const bf16_t* __restrict__ x,
                                                         const bf16_t* __restrict__ w,
                                                         const TBIAS* __restrict__ bias,
                                                         void* __restrict__ out_, int M, int N,
                                                         int K, int ldo) {
  static_assert(WM * WN == 4, "four wavefronts");
  static_assert(EPI != EPI_GATED || WN == 1, "gating needs both halves in one wavefront");
  constexpr bool SWIZZLED = TK == 64;
  constexpr int LD = SWIZZLED ? TK : TK + 8;
  // Where the 8 elements from k (a multiple of 8) of a tile row lie in LDS.  Rows of 64
  // elements are 128 bytes, half the banks; the 16-byte chunks of a row are permuted by the
  // row pair's index, so that the 16 rows one operand read touches hit 16 different bank
  // groups, as do the two rows a staging write fills.  Other widths pad the row instead.
  auto lds_at = [](int row, int k) {
    return SWIZZLED ? row * LD + ((((k >> 3) ^ (row >> 1)) & 7) << 3) : row * LD + k;
  };
  constexpr int TM = BM / WM / 16, TN = BN / WN / 16;       // MFMA tiles per wavefront
  constexpr int CHUNKS_ROW = TK / 8;                        // 16-byte chunks per tile row
  constexpr int XCH = BM * CHUNKS_ROW / 256, WCH = BN * CHUNKS_ROW / 256;  // per thread
  static_assert(XCH >= 1 && WCH >= 1, "tile too small for 256 threads");
  __shared__ __attribute__((aligned(16))) bf16_t xs[2][BM * LD];
  __shared__ __attribute__((aligned(16))) bf16_t ws[2][BN * LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g4 = lane >> 4;
  const int wm = (wave / WN) * (BM / WM), wn = (wave % WN) * (BN / WN);
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
  const int m0 = tile_m * BM, n0 = tile_n * (EPI == EPI_GATED ? BN / 2 : BN);

  // Staging: thread t moves chunk t, t + 256, ... of each operand's tile.
  const bf16_t* xg[XCH];
  const bf16_t* wg[WCH];
  int xo[XCH], wo[WCH];
  const int sk = (tid % CHUNKS_ROW) * 8;
#pragma unroll
  for (int i = 0; i < XCH; ++i) {
    const int row = (tid + i * 256) / CHUNKS_ROW;
    xg[i] = x + (size_t)min(m0 + row, M - 1) * K + sk;
    xo[i] = lds_at(row, sk);
  }
#pragma unroll
  for (int i = 0; i < WCH; ++i) {
    const int row = (tid + i * 256) / CHUNKS_ROW;
    int wrow = min(n0 + row, N - 1);
    if (EPI == EPI_GATED)  // tile rows [0, BN/2) are gate rows, [BN/2, BN) the matching up rows
      wrow = row < BN / 2 ? min(n0 + row, N - 1) : N + min(n0 + row - BN / 2, N - 1);
    wg[i] = w + (size_t)wrow * K + sk;
    wo[i] = lds_at(row, sk);
  }

  f32x4 acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; ++a)
#pragma unroll
    for (int b = 0; b < TN; ++b) acc[a][b] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // A stage's loads are asked for one or two stages before it is needed, into registers (the
  // latency of a load is several stages' worth of products), and parked in LDS one stage
  // before.
  struct Staged {
    uint4 x[XCH], w[WCH];
  };
  auto fetch = [&](int k0) __attribute__((always_inline)) {
    Staged r;
    const bool ok = k0 + sk < K;
#pragma unroll
    for (int i = 0; i < XCH; ++i) r.x[i] = ok ? ld16(xg[i] + k0) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < WCH; ++i) r.w[i] = ok ? ld16(wg[i] + k0) : make_uint4(0, 0, 0, 0);
    return r;
  };
  auto stash = [&](const Staged& r, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < XCH; ++i) *(uint4*)(&xs[buf][xo[i]]) = r.x[i];
#pragma unroll
    for (int i = 0; i < WCH; ++i) *(uint4*)(&ws[buf][wo[i]]) = r.w[i];
  };
  auto products = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int kk = 0; kk < TK; kk += 32) {
      Frag a[TM], b[TN];
#pragma unroll
      for (int t = 0; t < TM; ++t)
        a[t].u = *(const uint4*)(&xs[buf][lds_at(wm + t * 16 + r, kk + g4 * 8)]);
#pragma unroll
      for (int t = 0; t < TN; ++t)
        b[t].u = *(const uint4*)(&ws[buf][lds_at(wn + t * 16 + r, kk + g4 * 8)]);
#pragma unroll
      for (int ta = 0; ta < TM; ++ta)
#pragma unroll
        for (int tb = 0; tb < TN; ++tb)
          // A = W rows (n), B = x rows (m): the result holds 4 consecutive n per lane.
          acc[ta][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[tb].v, a[ta].v, acc[ta][tb],
                                                                0, 0, 0);
    }
  };

  const int steps = (K + TK - 1) / TK;
  // Small tiles have the registers for a second set in flight (the loop is unrolled by two so
  // that no set is ever copied: a copy would wait for its loads); the 128 x 128 tile would
  // lose its second workgroup per compute unit to it, and asks one stage ahead only.
  constexpr bool TWO_AHEAD = BM * BN <= 64 * 128;
  Staged even = fetch(0);
  stash(even, 0);
  if constexpr (TWO_AHEAD) {
    Staged odd = fetch(TK);          // past K: zeros, never parked
    even = fetch(2 * TK);
    __syncthreads();
    for (int s = 0; s < steps; s += 2) {
      products(0);
      if (s + 1 < steps) stash(odd, 1);
      odd = fetch((s + 3) * TK);
      __syncthreads();
      if (s + 1 < steps) {
        products(1);
        if (s + 2 < steps) stash(even, 0);
        even = fetch((s + 4) * TK);
        __syncthreads();
      }
    }
  } else {
    __syncthreads();
    for (int s = 0; s < steps; ++s) {   // not unrolled: the loop body's registers are the limit
      const int buf = s & 1;
      if (s + 1 < steps) even = fetch((s + 1) * TK);
      products(buf);
      if (s + 1 < steps) stash(even, buf ^ 1);
      __syncthreads();
    }
  }

  // acc[ta][tb][i] = y[m = m0 + wm + ta*16 + r][n = n0 + wn + tb*16 + g4*4 + i]
#pragma unroll
  for (int ta = 0; ta < TM; ++ta) {
    const int m = m0 + wm + ta * 16 + r;
    if (m >= M) continue;
    if (EPI == EPI_GATED) {
#pragma unroll
      for (int tb = 0; tb < TN / 2; ++tb) {
        const int n = n0 + tb * 16 + g4 * 4;
        bf16_t* dst = (bf16_t*)out_ + (size_t)m * ldo + n;
        float o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float g = Elem<bf16_t>::round(acc[ta][tb][i]);
          const float u = Elem<bf16_t>::round(acc[ta][tb + TN / 2][i]);
          o[i] = Elem<bf16_t>::round(g / (1.f + expf(-g))) * u;
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
      for (int i = 0; i < 4; ++i) {
        v[i] = acc[ta][tb][i];
        if (bias != nullptr && n + i < N) v[i] += Elem<TBIAS>::load(bias + n + i);
      }
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
          if (EPI == EPI_ACC) {
            const float4 old = *(const float4*)dst;
            o.x += old.x;
            o.y += old.y;
            o.z += old.z;
            o.w += old.w;
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

template <int BM, int BN, int TK, int WM, int WN, int EPI>
static void launch_tiled_cfg(const void* x, const void* w, const void* bias, int bias_dtype,
                             void* out, int M, int N, int K, int ldo, hipStream_t stream) {
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  if (bias && bias_dtype == MK_BF16)
    gemm_tiled_kernel<BM, BN, TK, WM, WN, EPI, bf16_t><<<grid, 256, 0, stream>>>(
        (const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias, out, M, N, K, ldo);
  else
    gemm_tiled_kernel<BM, BN, TK, WM, WN, EPI, float><<<grid, 256, 0, stream>>>(
        (const bf16_t*)x, (const bf16_t*)w, (const float*)bias, out, M, N, K, ldo);
}

// Tile configurations, by index: 0 = 128x128, 1 = 64x128, 2 = 64x64 (k in stages of 64).
#define TILED_CONFIGS 3

template <int EPI>
static void launch_tiled(int config, const void* x, const void* w, const void* bias,
                         int bias_dtype, void* out, int M, int N, int K, int ldo,
                         hipStream_t stream) {
  switch (config) {
    case 0: launch_tiled_cfg<128, 128, 64, 2, 2, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, stream); break;
    case 1: launch_tiled_cfg<64, 128, 64, 1, 4, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, stream); break;
    default: launch_tiled_cfg<64, 64, 64, 2, 2, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, stream); break;
  }
}

// 128 x 128 tiles when they give every compute unit a workgroup, else 64 x 64 (measured:
// 2048 x 3584 x 18944 runs a quarter faster in 448 large tiles than in 1792 small ones,
// 2048 x 896 x 4864 a quarter slower in 112 large tiles than in 448 small ones).
// At most 64 rows: 64 x 128 tiles, no half of a tile idle.
extern "C" int mk_linear_tiled_config(int M, int N, int K) {
  if (M <= 64) return 1;
  const long groups = (long)((M + 127) / 128) * ((N + 127) / 128);
  return groups >= 256 ? 0 : 2;
}

// act[M, inter] (bfloat16) = silu(x Wg^T) * (x Wu^T) for w = [Wg | Wu] stacked [2 inter, K].
extern "C" int mk_gated_tiled(const void* x, const void* w, void* act, int M, int inter, int K,
                              hipStream_t stream) {
  MK_REQUIRE(M > 0 && inter > 0 && K > 0 && K % 8 == 0,
             "gated projection: K=%d must be a multiple of 8 (M=%d I=%d)", K, M, inter);
  MK_REQUIRE((M + 127) / 128 <= 65535, "gated projection: M=%d too large for one launch", M);
  dim3 grid((inter + 63) / 64, (M + 127) / 128);
  gemm_tiled_kernel<128, 128, 64, 4, 1, EPI_GATED, float><<<grid, 256, 0, stream>>>(
      (const bf16_t*)x, (const bf16_t*)w, (const float*)nullptr, act, M, inter, K, inter);
  MK_LAUNCH_CHECK("gated_tiled");
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
  if (config < 0) config = mk_linear_tiled_config(M, N, K);
  MK_REQUIRE(config < TILED_CONFIGS, "tiled projection: no configuration %d", config);
  if (accumulate)
    launch_tiled<EPI_ACC>(config, x, w, bias, bias_dtype, out, M, N, K, ldo, stream);
  else if (out_dtype == MK_F32)
    launch_tiled<EPI_F32>(config, x, w, bias, bias_dtype, out, M, N, K, ldo, stream);
  else if (out_dtype == MK_BF16)
    launch_tiled<EPI_BF16>(config, x, w, bias, bias_dtype, out, M, N, K, ldo, stream);
  else
    MK_REQUIRE(false, "tiled projection: unknown out dtype %d", out_dtype);
  MK_LAUNCH_CHECK("linear_tiled");
  return 0;
}
