// y[M, N] = x[M, K] . w[N, K]^T (+ bias[N]) for any M, N, K, in float or bfloat16
// with float accumulation. Every output element is summed over k = 0..K-1 in that
// order by one thread, so a row's result does not depend on how many other rows
// there are. This is the matrix product of the 32-bit path and the fallback of the
// bfloat16 path for sizes that the faster kernels refuse.
#include "nhv_common.h"

#define TM 64
#define TN 64
#define TK 16

template <typename TIn, typename TOut>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TIn* __restrict__ x, const TIn* __restrict__ w,
                                                           const TIn* __restrict__ bias, TOut* __restrict__ y,
                                                           int M, int N, int K) {
  __shared__ float xs[TK][TM + 4];
  __shared__ float ws[TK][TN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  const int lr = tid / 4;          // row of the tile that this thread loads
  const int lk = (tid % 4) * 4;    // first of its four k
  for (int k0 = 0; k0 < K; k0 += TK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + lk + i;
      const int m = m0 + lr, n = n0 + lr;
      xs[lk + i][lr] = (m < M && k < K) ? to_f32(x[(size_t)m * K + k]) : 0.f;
      ws[lk + i][lr] = (n < N && k < K) ? to_f32(w[(size_t)n * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
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
      if (bias) v += to_f32(bias[n]);
      y[(size_t)m * N + n] = from_f32<TOut>(v);
    }
  }
}

extern "C" int nhv_gemm_generic(const void* x, const void* w, const void* bias, void* y, int M, int N, int K,
                                int in_dtype, int out_dtype, void* stream) {
  NHV_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
  dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
  NHV_REQUIRE(grid.y <= 65535, "gemm: too many rows (%d)", M);
  hipStream_t s = (hipStream_t)stream;
#define LAUNCH(TI, TO) \
  hipLaunchKernelGGL((gemm_generic_kernel<TI, TO>), grid, dim3(256), 0, s, (const TI*)x, (const TI*)w, (const TI*)bias, (TO*)y, M, N, K)
  if (in_dtype == NHV_F32 && out_dtype == NHV_F32) LAUNCH(float, float);
  else if (in_dtype == NHV_BF16 && out_dtype == NHV_BF16) LAUNCH(bf16_t, bf16_t);
  else if (in_dtype == NHV_BF16 && out_dtype == NHV_F32) LAUNCH(bf16_t, float);
  else return nhv_fail("gemm: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
#undef LAUNCH
  NHV_LAUNCH_CHECK("gemm_generic");
  return 0;
}
