// bfloat16 projections on the matrix cores: y[M,N] = x[M,K] W[N,K]^T, float32 accumulate.
//
// Two kernels for the two regimes of an inference step:
//
//  * skinny (M <= 64, decoding): the weights are read once, straight from HBM into the A
//    operand of v_mfma_f32_16x16x32_bf16 (16 rows of W by 32 k per instruction); the few rows
//    of x are the B operand and come out of the L2.  One wavefront owns 32 rows of W and one
//    slice of K.  Splitting K gives the small matrices of a small model enough wavefronts to
//    pull their bytes; every slice writes its own float32 partial result [slice, M, N], and
//    whichever kernel consumes the projection (RMSNorm, rotary + cache write, SiLU gating)
//    adds the slices up in slice order, so results are reproducible.
//
//  * tiled (M > 64, prompts): 128 x 128 tiles of y per workgroup, K in steps of 32 through
//    LDS with the next step's global loads in flight during the current step's products;
//    4 wavefronts as 2 x 2, each 64 x 64 = 4 x 4 MFMA tiles.  Epilogues: bfloat16 store with
//    bias, float32 store, or float32 accumulate into the residual stream.
//
// In both, lane l of a wavefront holds row (l % 16) and k-slots (l / 16) * 8 .. + 8 of an
// operand; which k a slot means is free as long as A and B agree, and the skinny kernel uses
// that to let each lane read 64 contiguous bytes per 128 k.
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

#define SK_NT 2  // 16-row tiles of W per wavefront

// out[(slice * M + m) * N + n]; K % 8 == 0; a slice covers k_per_slice (a multiple of 128).
template <int MT>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const bf16_t* __restrict__ x,
                                                          const bf16_t* __restrict__ w,
                                                          float* __restrict__ out, int M, int N,
                                                          int K, int k_per_slice) {
  const int lane = threadIdx.x & 63, r = lane & 15, g4 = lane >> 4;
  const int n0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * (16 * SK_NT);
  if (n0 >= N) return;
  const int slice = blockIdx.y;
  const int k_begin = slice * k_per_slice, k_end = min(K, k_begin + k_per_slice);

  const bf16_t* wrow[SK_NT];
#pragma unroll
  for (int t = 0; t < SK_NT; ++t) wrow[t] = w + (size_t)min(n0 + t * 16 + r, N - 1) * K;
  const bf16_t* xrow[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) xrow[t] = x + (size_t)min(t * 16 + r, M - 1) * K;

  f32x4 acc[SK_NT][MT];
#pragma unroll
  for (int a = 0; a < SK_NT; ++a)
#pragma unroll
    for (int b = 0; b < MT; ++b) acc[a][b] = (f32x4){0.f, 0.f, 0.f, 0.f};

  for (int k0 = k_begin; k0 < k_end; k0 += 128) {
    const int kk = k0 + g4 * 32;  // this lane's 32 k of the 128
    Frag a[SK_NT][4], b[MT][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool ok = kk + j * 8 < k_end;
#pragma unroll
      for (int t = 0; t < SK_NT; ++t)
        a[t][j].u = ok ? ld16(wrow[t] + kk + j * 8) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int t = 0; t < MT; ++t)
        b[t][j].u = ok ? ld16(xrow[t] + kk + j * 8) : make_uint4(0, 0, 0, 0);
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

  // acc[ta][tb][i] = y[m = tb*16 + r][n = n0 + ta*16 + g4*4 + i]
#pragma unroll
  for (int tb = 0; tb < MT; ++tb) {
    const int m = tb * 16 + r;
    if (m >= M) continue;
    float* dst = out + ((size_t)slice * M + m) * N;
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

extern "C" int mk_linear_skinny_slices(int M, int N, int K) {
  // Enough slices of K (each a multiple of 128) for about 1024 wavefronts, but no more
  // partial results than the weights are worth: slices * M * 4 bytes per output column
  // against K * 2 bytes of weights.
  const int tiles = (N + 16 * SK_NT - 1) / (16 * SK_NT);
  const int steps = (K + 127) / 128;
  int slices = (1024 + tiles - 1) / tiles;
  if (slices > steps) slices = steps;
  const int cap = K / (8 * (M > 0 ? M : 1));
  if (slices > cap) slices = cap;
  if (slices < 1) slices = 1;
  const int per = ((steps + slices - 1) / slices);
  return (steps + per - 1) / per;
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
  dim3 grid((tiles + 3) / 4, slices);
  const bf16_t* xp = (const bf16_t*)x;
  const bf16_t* wp = (const bf16_t*)w;
  switch ((M + 15) / 16) {
    case 1: gemm_skinny_kernel<1><<<grid, 256, 0, stream>>>(xp, wp, out, M, N, K, per * 128); break;
    case 2: gemm_skinny_kernel<2><<<grid, 256, 0, stream>>>(xp, wp, out, M, N, K, per * 128); break;
    case 3: gemm_skinny_kernel<3><<<grid, 256, 0, stream>>>(xp, wp, out, M, N, K, per * 128); break;
    default: gemm_skinny_kernel<4><<<grid, 256, 0, stream>>>(xp, wp, out, M, N, K, per * 128); break;
  }
  MK_LAUNCH_CHECK("linear_skinny");
  return 0;
}

// ------------------------------------------------------------------------------- tiled

#define TB 128  // tile of y, both ways
#define TK 32   // k per LDS stage
#define TLD 40  // LDS row stride in elements (80 bytes: conflict-free 16-byte reads)

enum { EPI_BF16 = 0, EPI_F32 = 1, EPI_ACC = 2 };

template <int EPI, typename TBIAS>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const bf16_t* __restrict__ x,
                                                         const bf16_t* __restrict__ w,
                                                         const TBIAS* __restrict__ bias,
                                                         void* __restrict__ out_, int M, int N,
                                                         int K, int ldo) {
  __shared__ __attribute__((aligned(16))) bf16_t xs[2][TB * TLD];
  __shared__ __attribute__((aligned(16))) bf16_t ws[2][TB * TLD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g4 = lane >> 4;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
  const int m0 = blockIdx.y * TB, n0 = blockIdx.x * TB;

  // Staging: 128 rows x 32 k = 512 chunks of 16 bytes per operand, two per thread.
  const int srow = tid >> 2, sk = (tid & 3) * 8;
  const bf16_t* xg[2];
  const bf16_t* wg[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    xg[i] = x + (size_t)min(m0 + srow + i * 64, M - 1) * K + sk;
    wg[i] = w + (size_t)min(n0 + srow + i * 64, N - 1) * K + sk;
  }

  f32x4 acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[a][b] = (f32x4){0.f, 0.f, 0.f, 0.f};

  uint4 xr[2], wr[2];
  auto fetch = [&](int k0) {
    const bool ok = k0 + sk < K;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      xr[i] = ok ? ld16(xg[i] + k0) : make_uint4(0, 0, 0, 0);
      wr[i] = ok ? ld16(wg[i] + k0) : make_uint4(0, 0, 0, 0);
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      *(uint4*)(&xs[buf][(srow + i * 64) * TLD + sk]) = xr[i];
      *(uint4*)(&ws[buf][(srow + i * 64) * TLD + sk]) = wr[i];
    }
  };

  const int steps = (K + TK - 1) / TK;
  fetch(0);
  stash(0);
  __syncthreads();
  for (int s = 0; s < steps; ++s) {
    const int buf = s & 1;
    if (s + 1 < steps) fetch((s + 1) * TK);
    Frag a[4], b[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      a[t].u = *(const uint4*)(&xs[buf][(wm + t * 16 + r) * TLD + g4 * 8]);
      b[t].u = *(const uint4*)(&ws[buf][(wn + t * 16 + r) * TLD + g4 * 8]);
    }
#pragma unroll
    for (int ta = 0; ta < 4; ++ta)
#pragma unroll
      for (int tb = 0; tb < 4; ++tb)
        // A = W rows (n), B = x rows (m): the result holds 4 consecutive n per lane.
        acc[ta][tb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[tb].v, a[ta].v, acc[ta][tb], 0,
                                                              0, 0);
    if (s + 1 < steps) stash(buf ^ 1);
    __syncthreads();
  }

  // acc[ta][tb][i] = y[m = m0 + wm + ta*16 + r][n = n0 + wn + tb*16 + g4*4 + i]
#pragma unroll
  for (int ta = 0; ta < 4; ++ta) {
    const int m = m0 + wm + ta * 16 + r;
    if (m >= M) continue;
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) {
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
          ushort4 o;
          o.x = f32_to_bf16(v[0]);
          o.y = f32_to_bf16(v[1]);
          o.z = f32_to_bf16(v[2]);
          o.w = f32_to_bf16(v[3]);
          *(ushort4*)dst = o;
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

template <int EPI>
static void launch_tiled(const void* x, const void* w, const void* bias, int bias_dtype, void* out,
                         int M, int N, int K, int ldo, hipStream_t stream) {
  dim3 grid((N + TB - 1) / TB, (M + TB - 1) / TB);
  if (bias && bias_dtype == MK_BF16)
    gemm_tiled_kernel<EPI, bf16_t><<<grid, 256, 0, stream>>>(
        (const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias, out, M, N, K, ldo);
  else
    gemm_tiled_kernel<EPI, float><<<grid, 256, 0, stream>>>(
        (const bf16_t*)x, (const bf16_t*)w, (const float*)bias, out, M, N, K, ldo);
}

extern "C" int mk_linear_tiled(const void* x, const void* w, const void* bias, int bias_dtype,
                               void* out, int out_dtype, int accumulate, int M, int N, int K,
                               int ldo, hipStream_t stream) {
  MK_REQUIRE(M > 0 && N > 0 && K > 0 && K % 8 == 0,
             "tiled projection: K=%d must be a multiple of 8 (M=%d N=%d)", K, M, N);
  MK_REQUIRE(ldo >= N, "tiled projection: leading dimension %d smaller than N=%d", ldo, N);
  MK_REQUIRE(!accumulate || out_dtype == MK_F32,
             "tiled projection: accumulation needs a float32 destination");
  MK_REQUIRE((M + TB - 1) / TB <= 65535, "tiled projection: M=%d too large for one launch", M);
  if (accumulate)
    launch_tiled<EPI_ACC>(x, w, bias, bias_dtype, out, M, N, K, ldo, stream);
  else if (out_dtype == MK_F32)
    launch_tiled<EPI_F32>(x, w, bias, bias_dtype, out, M, N, K, ldo, stream);
  else if (out_dtype == MK_BF16)
    launch_tiled<EPI_BF16>(x, w, bias, bias_dtype, out, M, N, K, ldo, stream);
  else
    MK_REQUIRE(false, "tiled projection: unknown out dtype %d", out_dtype);
  MK_LAUNCH_CHECK("linear_tiled");
  return 0;
}
