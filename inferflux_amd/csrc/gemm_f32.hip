// True 32-bit matrix product:  C[M,N] = A[M,K] * W[N,K]^T (+ bias[N]).
//
// The weight is float and every multiply-add is a float fmaf: no matrix-core instruction, no
// reduced-precision mode.  Each output element is accumulated over k in ascending order by one
// thread, so its value does not depend on M, on the element's place in the batch or on what
// else runs.  This is the matrix product of the 32-bit path; the reference has no 32-bit path
// (runtime/backends/cuda/native/transformer_forward.cu:4600-4601 instantiates half and bf16
// only), its library call with float accumulation is runtime/backends/cuda/native/cublas_gemm.cpp:99-117.
#include "common.h"

IFX_DEFINE_LAST_ERROR()

#define BM 64
#define BN 64
#define BK 16

template <typename TA, typename TO>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const TA* __restrict__ A, const float* __restrict__ W,
                                                       const float* __restrict__ bias, TO* __restrict__ C,
                                                       int M, int N, int K) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  const int lr = tid / 4;        // tile row this thread loads (0..63)
  const int lk = (tid % 4) * 4;  // first of its 4 k values
  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int k = k0 + lk + q;
      const int m = m0 + lr, n = n0 + lr;
      As[lk + q][lr] = (m < M && k < K) ? to_f(A[(size_t)m * K + k]) : 0.f;
      Ws[lk + q][lr] = (n < N && k < K) ? W[(size_t)n * K + k] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
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
      if (bias) v += bias[n];
      C[(size_t)m * N + n] = from_f<TO>(v);
    }
  }
}

extern "C" int ifx_gemm_f32(const void* A, int a_dtype, const float* W, const float* bias, void* C,
                            int c_dtype, int M, int N, int K, void* stream) {
  IFX_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
  if (M == 0) return 0;
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  IFX_REQUIRE(grid.y <= 65535, "gemm_f32: M=%d too large for one launch", M);
  hipStream_t s = (hipStream_t)stream;
#define LAUNCH(TA, TO) \
  hipLaunchKernelGGL((gemm_f32_kernel<TA, TO>), grid, dim3(256), 0, s, (const TA*)A, W, bias, (TO*)C, M, N, K)
  if (a_dtype == DT_F32 && c_dtype == DT_F32) LAUNCH(float, float);
  else if (a_dtype == DT_BF16 && c_dtype == DT_BF16) LAUNCH(bf16_t, bf16_t);
  else if (a_dtype == DT_BF16 && c_dtype == DT_F32) LAUNCH(bf16_t, float);
  else if (a_dtype == DT_F32 && c_dtype == DT_BF16) LAUNCH(float, bf16_t);
  else IFX_FAIL("gemm_f32: unknown dtypes a=%d c=%d", a_dtype, c_dtype);
#undef LAUNCH
  IFX_LAUNCH_CHECK();
}
