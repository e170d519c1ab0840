// y[M,N] = x[M,K] * W[N,K]^T (+ bias), float32 multiply-add on the vector units.
//
// This is the projection kernel of the true 32-bit path and the fallback for any size the
// matrix-core kernels refuse.  Every output element is produced by one thread that walks K
// in ascending order, so a row's result does not depend on how many other rows are in the
// batch or where the row sits in it.
#include "common.h"
#include "mercury_kernels.h"

#define GT 64   // tile of C, both ways
#define GK 16   // depth of one LDS stage

template <typename T, typename TO, int ACCUMULATE, typename TB>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const T* __restrict__ x,
                                                           const T* __restrict__ w,
                                                           const TB* __restrict__ bias,
                                                           TO* __restrict__ out, int M, int N,
                                                           int K, int lda, int ldo) {
  __shared__ float xs[GK][GT + 4];
  __shared__ float ws[GK][GT + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
  const int lrow = tid >> 2;        // 0..63: the tile row this thread stages
  const int lk = (tid & 3) * 4;     // 0,4,8,12: first of its four k

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += GK) {
    {
      const int m = m0 + lrow;
      const T* src = x + (size_t)m * lda + k0 + lk;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        xs[lk + i][lrow] = (m < M && k0 + lk + i < K) ? Elem<T>::load(src + i) : 0.f;
      const int n = n0 + lrow;
      const T* wsrc = w + (size_t)n * K + k0 + lk;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        ws[lk + i][lrow] = (n < N && k0 + lk + i < K) ? Elem<T>::load(wsrc + i) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += Elem<TB>::load(bias + n);
      TO* dst = out + (size_t)m * ldo + n;
      if (ACCUMULATE)
        Elem<TO>::store(dst, Elem<TO>::load(dst) + v);
      else
        Elem<TO>::store(dst, v);
    }
  }
}

template <typename T, typename TO, int ACC>
static void launch_generic(const void* x, const void* w, const void* bias, int bias_dtype,
                           void* out, int M, int N, int K, int lda, int ldo,
                           hipStream_t stream) {
  dim3 grid((N + GT - 1) / GT, (M + GT - 1) / GT);
  if (bias && bias_dtype == MK_BF16)
    gemm_generic_kernel<T, TO, ACC, bf16_t><<<grid, 256, 0, stream>>>(
        (const T*)x, (const T*)w, (const bf16_t*)bias, (TO*)out, M, N, K, lda, ldo);
  else
    gemm_generic_kernel<T, TO, ACC, float><<<grid, 256, 0, stream>>>(
        (const T*)x, (const T*)w, (const float*)bias, (TO*)out, M, N, K, lda, ldo);
}

extern "C" int mk_linear_generic(const void* x, const void* w, int dtype, const void* bias,
                                 int bias_dtype, void* out, int out_dtype, int accumulate,
                                 int M, int N, int K, int lda, int ldo, hipStream_t stream) {
  MK_REQUIRE(M >= 0 && N > 0 && K > 0, "linear: bad sizes M=%d N=%d K=%d", M, N, K);
  MK_REQUIRE(lda >= K && ldo >= N, "linear: leading dimensions %d/%d smaller than K=%d/N=%d",
             lda, ldo, K, N);
  MK_REQUIRE(!accumulate || out_dtype == MK_F32,
             "linear: accumulation needs a float32 destination");
  MK_REQUIRE((M + GT - 1) / GT <= 65535, "linear: M=%d too large for one launch", M);
  if (M == 0) return 0;
  if (dtype == MK_F32 && out_dtype == MK_F32) {
    if (accumulate)
      launch_generic<float, float, 1>(x, w, bias, bias_dtype, out, M, N, K, lda, ldo, stream);
    else
      launch_generic<float, float, 0>(x, w, bias, bias_dtype, out, M, N, K, lda, ldo, stream);
  } else if (dtype == MK_BF16 && out_dtype == MK_F32) {
    if (accumulate)
      launch_generic<bf16_t, float, 1>(x, w, bias, bias_dtype, out, M, N, K, lda, ldo, stream);
    else
      launch_generic<bf16_t, float, 0>(x, w, bias, bias_dtype, out, M, N, K, lda, ldo, stream);
  } else if (dtype == MK_BF16 && out_dtype == MK_BF16) {
    launch_generic<bf16_t, bf16_t, 0>(x, w, bias, bias_dtype, out, M, N, K, lda, ldo, stream);
  } else {
    MK_REQUIRE(false, "linear: unsupported dtypes in=%d out=%d", dtype, out_dtype);
  }
  MK_LAUNCH_CHECK("linear_generic");
  return 0;
}
