// C[M, N] = A[M, K] * W[N, K]^T in true float32: plain fused multiply-adds on the
// vector units, no matrix-core mode of reduced precision.  W has the layout of a
// bias-free linear layer's weight ([out, in], src/halite/transformers/feedforward.py:
// 204-212; src/halite/transformers/infer/attention.py:21-24).  Each output element
// is one chain of K multiply-adds in index order, whatever M is, so a token's
// result does not depend on what else is in the batch.
#include "hal_common.h"
#include "hal_api.h"

#define GF_BM 64
#define GF_BN 64
#define GF_BK 16
#define GF_PAD 4

__global__ void __launch_bounds__(256)
gemm_f32_kernel(const float* __restrict__ A, int lda, const float* __restrict__ W, int ldw,
                float* __restrict__ C, int ldc, int M, int N, int K) {
  __shared__ float As[GF_BK][GF_BM + GF_PAD];
  __shared__ float Ws[GF_BK][GF_BN + GF_PAD];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * GF_BM, n0 = blockIdx.x * GF_BN;
  const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;  // this thread's 4x4 outputs

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += GF_BK) {
    // 64 rows x 16 k of each operand: 1024 elements, four per thread
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int idx = tid + e * 256;
      const int r = idx / GF_BK, kk = idx % GF_BK;
      const int gm = m0 + r, gn = n0 + r, gk = k0 + kk;
      As[kk][r] = (gm < M && gk < K) ? A[(size_t)gm * lda + gk] : 0.f;
      Ws[kk][r] = (gn < N && gk < K) ? W[(size_t)gn * ldw + gk] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GF_BK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][tm + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tn + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + tm + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tn + j;
      if (gn < N) C[(size_t)gm * ldc + gn] = acc[i][j];
    }
  }
}

extern "C" int hal_gemm_f32(const float* A, int lda, const float* W, int ldw, float* C, int ldc,
                            int M, int N, int K, hipStream_t stream) {
  HAL_REQUIRE(M >= 0 && N > 0 && K > 0, "hal_gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
  HAL_REQUIRE(lda >= K && ldw >= K && ldc >= N, "hal_gemm_f32: leading dimensions %d %d %d", lda,
              ldw, ldc);
  if (M == 0) return 0;
  dim3 grid((N + GF_BN - 1) / GF_BN, (M + GF_BM - 1) / GF_BM);
  HAL_REQUIRE(grid.y <= 65535, "hal_gemm_f32: M=%d exceeds the grid limit", M);
  hipLaunchKernelGGL(gemm_f32_kernel, grid, dim3(256), 0, stream, A, lda, W, ldw, C, ldc, M, N, K);
  HAL_LAUNCH_CHECK();
  return 0;
}
