// bfloat16 projections on the matrix cores: y[M,N] = x[M,K] W[N,K]^T, float32 accumulate.
//
// Two kernels for the two regimes of an inference step:
//
//  * skinny (M <= 64, decoding): the weights are read once, straight from HBM into the A
//    operand of v_mfma_f32_16x16x32_bf16 (16 rows of W by 32 k per instruction); the few rows
//    of x are the B operand and come out of the L2.  A workgroup owns 32 rows of W and one
//    slice of K, its wavefronts taking the slice's k-steps in turn.  Splitting K gives the
//    small matrices of a small model enough wavefronts to pull their bytes; every slice
//    writes its own float32 partial result [slice, M, N], and whichever kernel consumes the
//    projection (RMSNorm, rotary + cache write) adds the slices up in slice order, so results
//    are reproducible.  The gate/up projection keeps all of K in one workgroup and gates in
//    its epilogue.
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

#define SK_NT 2     // 16-row tiles of W per workgroup
#define SK_WAVES 4  // wavefronts of a workgroup; they share the rows and split the k-steps

// Each workgroup owns 32 rows of W (two 16-row tiles) and one slice of K; its four wavefronts
// take the slice's 128-wide k-steps in turn (wave w: steps w, w + 4, ...) and add their
// results up through LDS in wave order, so a slice yields one partial result.
//   GATED = 0: out[(slice * M + m) * N + n] float32, tiles are rows n0.. and n0 + 16..
//   GATED = 1: W is [gate rows | up rows] of N each; the two tiles are gate rows n0.. and the
//              matching up rows N + n0.., the slice must be all of K, and the epilogue writes
//              act[m][n] = silu(g) * u in bfloat16 (reference: mercury/model/qwen2.py:42).
template <int MT, int GATED>
__global__ __launch_bounds__(64 * SK_WAVES) void gemm_skinny_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, void* __restrict__ out_, int M,
    int N, int K, int steps_per_slice) {
  __shared__ float red[SK_WAVES - 1][SK_NT * MT * 4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, g4 = lane >> 4;
  const int n0 = blockIdx.x * (GATED ? 16 : 16 * SK_NT);
  const int slice = blockIdx.y;
  const int step_begin = slice * steps_per_slice;
  const int step_end = min((K + 127) / 128, step_begin + steps_per_slice);

  const bf16_t* wrow[SK_NT];
#pragma unroll
  for (int t = 0; t < SK_NT; ++t) {
    const int row = GATED ? t * N + min(n0 + r, N - 1) : min(n0 + t * 16 + r, N - 1);
    wrow[t] = w + (size_t)row * K;
  }
  const bf16_t* xrow[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) xrow[t] = x + (size_t)min(t * 16 + r, M - 1) * K;

  f32x4 acc[SK_NT][MT];
#pragma unroll
  for (int a = 0; a < SK_NT; ++a)
#pragma unroll
    for (int b = 0; b < MT; ++b) acc[a][b] = (f32x4){0.f, 0.f, 0.f, 0.f};

  for (int step = step_begin + wave; step < step_end; step += SK_WAVES) {
    // Product j of the step takes k = step*128 + j*32 + g4*8 .. + 8 from this lane, so that
    // one load instruction reads 64 contiguous bytes of each of its 16 rows.
    const int kk = step * 128 + g4 * 8;
    Frag a[SK_NT][4], b[MT][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool ok = kk + j * 32 < K;
#pragma unroll
      for (int t = 0; t < SK_NT; ++t)
        a[t][j].u = ok ? ld16(wrow[t] + kk + j * 32) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int t = 0; t < MT; ++t)
        b[t][j].u = ok ? ld16(xrow[t] + kk + j * 32) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int ta = 0; ta < SK_NT; ++ta)
#pragma unroll
        for (int tb = 0; tb < MT; ++tb)
          acc[ta][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ta][j].v, b[tb][j].v,
                                                                acc[ta][tb], 0, 0, 0);
  }

  if (wave > 0) {
#pragma unroll
    for (int ta = 0; ta < SK_NT; ++ta)
#pragma unroll
      for (int tb = 0; tb < MT; ++tb)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave - 1][(ta * MT + tb) * 4 + i][lane] = acc[ta][tb][i];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int v = 0; v < SK_WAVES - 1; ++v)
#pragma unroll
    for (int ta = 0; ta < SK_NT; ++ta)
#pragma unroll
      for (int tb = 0; tb < MT; ++tb)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[ta][tb][i] += red[v][(ta * MT + tb) * 4 + i][lane];

  // acc[ta][tb][i] = y[m = tb*16 + r][column g4*4 + i of tile ta]
#pragma unroll
  for (int tb = 0; tb < MT; ++tb) {
    const int m = tb * 16 + r;
    if (m >= M) continue;
    if (GATED) {
      bf16_t* dst = (bf16_t*)out_ + (size_t)m * N;
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
    } else {
      float* dst = (float*)out_ + ((size_t)slice * M + m) * N;
#pragma unroll
      for (int ta = 0; ta < SK_NT; ++ta) {
        const int n = n0 + ta * 16 + g4 * 4;
        if (n + 3 < N && (N & 3) == 0) {
          *(float4*)(dst + n) =
              make_float4(acc[ta][tb][0], acc[ta][tb][1], acc[ta][tb][2], acc[ta][tb][3]);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < N) dst[n + i] = acc[ta][tb][i];
        }
      }
    }
  }
}

// Slices of K for the plain skinny projection: enough workgroups to fill the chip (about
// 512), every wavefront of a workgroup with at least one k-step, and no more partial results
// than the weights are worth (slices * M * 4 bytes per output column against K * 2).
extern "C" int mk_linear_skinny_slices(int M, int N, int K) {
  const int tiles = (N + 16 * SK_NT - 1) / (16 * SK_NT);
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

template <int GATED>
static void launch_skinny(const bf16_t* x, const bf16_t* w, void* out, int M, int N, int K,
                          int per, dim3 grid, hipStream_t stream) {
  switch ((M + 15) / 16) {
    case 1: gemm_skinny_kernel<1, GATED><<<grid, 64 * SK_WAVES, 0, stream>>>(x, w, out, M, N, K, per); break;
    case 2: gemm_skinny_kernel<2, GATED><<<grid, 64 * SK_WAVES, 0, stream>>>(x, w, out, M, N, K, per); break;
    case 3: gemm_skinny_kernel<3, GATED><<<grid, 64 * SK_WAVES, 0, stream>>>(x, w, out, M, N, K, per); break;
    default: gemm_skinny_kernel<4, GATED><<<grid, 64 * SK_WAVES, 0, stream>>>(x, w, out, M, N, K, per); break;
  }
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
  const int tiles = (N + 16 * SK_NT - 1) / (16 * SK_NT);
  MK_REQUIRE(slices <= 65535, "skinny projection: too many slices");
  launch_skinny<0>((const bf16_t*)x, (const bf16_t*)w, out, M, N, K, per, dim3(tiles, slices),
                   stream);
  MK_LAUNCH_CHECK("linear_skinny");
  return 0;
}

// act[M, I] = silu(x Wg^T) * (x Wu^T) for W = [Wg | Wu] stacked as [2 I, K], 1 <= M <= 64.
extern "C" int mk_gated_skinny(const void* x, const void* w, void* act, int M, int inter, int K,
                               hipStream_t stream) {
  MK_REQUIRE(M >= 1 && M <= 64, "gated projection: M=%d outside 1..64", M);
  MK_REQUIRE(inter > 0 && K > 0 && K % 8 == 0, "gated projection: K=%d must be a multiple of 8",
             K);
  const int steps = (K + 127) / 128;
  launch_skinny<1>((const bf16_t*)x, (const bf16_t*)w, act, M, inter, K, steps,
                   dim3((inter + 15) / 16, 1), stream);
  MK_LAUNCH_CHECK("gated_skinny");
  return 0;
}

// ------------------------------------------------------------------------------- tiled

enum { EPI_BF16 = 0, EPI_F32 = 1, EPI_ACC = 2, EPI_GATED = 3 };

// One workgroup of 4 wavefronts (WM x WN) computes a BM x BN tile of y; K advances TK per
// stage through two LDS buffers, the next stage's global loads in flight during the current
// stage's products.  Rows of a tile lie in LDS with a stride of TK + 8 elements, which keeps
// 16-byte reads of 16 consecutive rows on distinct banks.
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
  constexpr int LD = TK + 8;
  constexpr int TM = BM / WM / 16, TN = BN / WN / 16;       // MFMA tiles per wavefront
  constexpr int CHUNKS_ROW = TK / 8;                        // 16-byte chunks per tile row
  constexpr int XCH = BM * CHUNKS_ROW / 256, WCH = BN * CHUNKS_ROW / 256;  // per thread
  static_assert(XCH >= 1 && WCH >= 1, "tile too small for 256 threads");
  __shared__ __attribute__((aligned(16))) bf16_t xs[2][BM * LD];
  __shared__ __attribute__((aligned(16))) bf16_t ws[2][BN * LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g4 = lane >> 4;
  const int wm = (wave / WN) * (BM / WM), wn = (wave % WN) * (BN / WN);
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * (EPI == EPI_GATED ? BN / 2 : BN);

  // Staging: thread t moves chunk t, t + 256, ... of each operand's tile.
  const bf16_t* xg[XCH];
  const bf16_t* wg[WCH];
  int xo[XCH], wo[WCH];
  const int sk = (tid % CHUNKS_ROW) * 8;
#pragma unroll
  for (int i = 0; i < XCH; ++i) {
    const int row = (tid + i * 256) / CHUNKS_ROW;
    xg[i] = x + (size_t)min(m0 + row, M - 1) * K + sk;
    xo[i] = row * LD + sk;
  }
#pragma unroll
  for (int i = 0; i < WCH; ++i) {
    const int row = (tid + i * 256) / CHUNKS_ROW;
    int wrow = min(n0 + row, N - 1);
    if (EPI == EPI_GATED)  // tile rows [0, BN/2) are gate rows, [BN/2, BN) the matching up rows
      wrow = row < BN / 2 ? min(n0 + row, N - 1) : N + min(n0 + row - BN / 2, N - 1);
    wg[i] = w + (size_t)wrow * K + sk;
    wo[i] = row * LD + sk;
  }

  f32x4 acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; ++a)
#pragma unroll
    for (int b = 0; b < TN; ++b) acc[a][b] = (f32x4){0.f, 0.f, 0.f, 0.f};

  uint4 xr[XCH], wr[WCH];
  auto fetch = [&](int k0) {
    const bool ok = k0 + sk < K;
#pragma unroll
    for (int i = 0; i < XCH; ++i) xr[i] = ok ? ld16(xg[i] + k0) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < WCH; ++i) wr[i] = ok ? ld16(wg[i] + k0) : make_uint4(0, 0, 0, 0);
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < XCH; ++i) *(uint4*)(&xs[buf][xo[i]]) = xr[i];
#pragma unroll
    for (int i = 0; i < WCH; ++i) *(uint4*)(&ws[buf][wo[i]]) = wr[i];
  };

  const int steps = (K + TK - 1) / TK;
  fetch(0);
  stash(0);
  __syncthreads();
  for (int s = 0; s < steps; ++s) {
    const int buf = s & 1;
    if (s + 1 < steps) fetch((s + 1) * TK);
#pragma unroll
    for (int kk = 0; kk < TK; kk += 32) {
      Frag a[TM], b[TN];
#pragma unroll
      for (int t = 0; t < TM; ++t)
        a[t].u = *(const uint4*)(&xs[buf][(wm + t * 16 + r) * LD + kk + g4 * 8]);
#pragma unroll
      for (int t = 0; t < TN; ++t)
        b[t].u = *(const uint4*)(&ws[buf][(wn + t * 16 + r) * LD + kk + g4 * 8]);
#pragma unroll
      for (int ta = 0; ta < TM; ++ta)
#pragma unroll
        for (int tb = 0; tb < TN; ++tb)
          // A = W rows (n), B = x rows (m): the result holds 4 consecutive n per lane.
          acc[ta][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[tb].v, a[ta].v, acc[ta][tb],
                                                                0, 0, 0);
    }
    if (s + 1 < steps) stash(buf ^ 1);
    __syncthreads();
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

// Tile configurations, by index: 0 = 128x128 (k 64), 1 = 64x128, 2 = 64x64, 3 = 128x128 (k 32).
#define TILED_CONFIGS 4

template <int EPI>
static void launch_tiled(int config, const void* x, const void* w, const void* bias,
                         int bias_dtype, void* out, int M, int N, int K, int ldo,
                         hipStream_t stream) {
  switch (config) {
    case 0: launch_tiled_cfg<128, 128, 64, 2, 2, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, stream); break;
    case 1: launch_tiled_cfg<64, 128, 64, 1, 4, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, stream); break;
    case 2: launch_tiled_cfg<64, 64, 64, 2, 2, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, stream); break;
    default: launch_tiled_cfg<128, 128, 32, 2, 2, EPI>(x, w, bias, bias_dtype, out, M, N, K, ldo, stream); break;
  }
}

// 128 x 128 tiles when they give every compute unit two workgroups or more, else 64 x 64.
extern "C" int mk_linear_tiled_config(int M, int N, int K) {
  const long groups = (long)((M + 127) / 128) * ((N + 127) / 128);
  return groups >= 512 ? 0 : 2;
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
