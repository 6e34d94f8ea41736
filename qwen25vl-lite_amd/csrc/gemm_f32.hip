// True float32 matrix product  C[M,N] = A[M,K] * W[N,K]^T (+ bias[N]),  W as a Linear stores it.
// Plain FMA arithmetic, no matrix-core input formats.  Every output element sums its K products
// in index order 0..K-1 in one accumulator, so a row's result does not depend on M or on the
// tile it falls in.  64x64 tile per block, 16x16 threads, 4x4 outputs per thread, K step 16.
#include "common.h"

#define TM 64
#define TN 64
#define TK 16

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ A, int lda,
                                                       const float* __restrict__ W, int ldw,
                                                       const float* __restrict__ bias, float* __restrict__ C, int ldc,
                                                       int M, int N, int K) {
  __shared__ float sa[TK][TM + 4];
  __shared__ float sw[TK][TN + 4];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += TK) {
    // 64 rows x 16 k per operand: 1024 elements, 4 per thread
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int idx = threadIdx.x + 256 * e;
      const int rr = idx / TK, kk = idx % TK;
      const int gm = m0 + rr, gn = n0 + rr, gk = k0 + kk;
      sa[kk][rr] = (gm < M && gk < K) ? A[(size_t)gm * lda + gk] : 0.f;
      sw[kk][rr] = (gn < N && gk < K) ? W[(size_t)gn * ldw + gk] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = sa[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = sw[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + ty * 4 + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn < N) C[(size_t)gm * ldc + gn] = acc[i][j] + (bias ? bias[gn] : 0.f);
    }
  }
}

extern "C" int qvl_gemm_f32(const void* A, int lda, const void* W, int ldw, const void* bias, void* C, int ldc, int M,
                            int N, int K, hipStream_t stream) {
  if (M <= 0 || N <= 0) return QVL_OK;
  if (K <= 0 || lda < K || ldw < K || ldc < N) return QVL_ERR_SHAPE;
  const dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
  if (grid.y > 65535) return QVL_ERR_LIMIT;
  hipLaunchKernelGGL(gemm_f32_kernel, grid, dim3(256), 0, stream, (const float*)A, lda, (const float*)W, ldw,
                     (const float*)bias, (float*)C, ldc, M, N, K);
  return qvl_launch_status();
}
