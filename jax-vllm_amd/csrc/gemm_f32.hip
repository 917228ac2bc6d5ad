// C[M,N] = A[M,K] * W[N,K]^T in true 32-bit: float inputs, float FMA, float
// accumulation, no reduced-precision matrix mode.  Each output element sums its
// K products in ascending k, whatever M and N are, so a row's result does not
// depend on which other rows are in the batch.
// 64x64 output tile per 256-thread block, K in slabs of 16 through LDS, 4x4
// outputs per thread.
#include "common.h"

#define G32_BM 64
#define G32_BN 64
#define G32_BK 16

__global__ void __launch_bounds__(256)
gemm_f32_kernel(float* __restrict__ C, const float* __restrict__ A, const float* __restrict__ W,
                int M, int N, int K, long long lda, long long ldw, long long ldc) {
  __shared__ float As[G32_BK][G32_BM + 4];
  __shared__ float Ws[G32_BK][G32_BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;      // 16 x 16 threads
  const int m0 = blockIdx.y * G32_BM, n0 = blockIdx.x * G32_BN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += G32_BK) {
    // 64 rows x 16 k = 1024 elements per operand, 4 per thread
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int idx = tid + e * 256;
      const int r = idx >> 4, kk = idx & 15;
      const int k = k0 + kk;
      const int am = m0 + r, wn = n0 + r;
      As[kk][r] = (am < M && k < K) ? A[(long long)am * lda + k] : 0.f;
      Ws[kk][r] = (wn < N && k < K) ? W[(long long)wn * ldw + k] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < G32_BK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
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
      if (n < N) C[(long long)m * ldc + n] = acc[i][j];
    }
  }
}

extern "C" int jv_gemm_f32(float* C, const float* A, const float* W, int M, int N, int K,
                           long long lda, long long ldw, long long ldc, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K < 0) return (int)hipErrorInvalidValue;
  const unsigned gy = (M + G32_BM - 1) / G32_BM;
  if (gy > 65535u) return (int)hipErrorInvalidValue;
  dim3 grid((N + G32_BN - 1) / G32_BN, gy);
  hipLaunchKernelGGL(gemm_f32_kernel, grid, dim3(256), 0, (hipStream_t)stream, C, A, W, M, N, K,
                     lda, ldw, ldc);
  return JV_LAUNCH_CHECK();
}
