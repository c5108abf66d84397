// C[M, N] = A[M, K] * W[N, K]^T in true float32: plain fused multiply-adds on the
// vector units, no matrix-core mode of reduced precision.  W has the layout of a
// bias-free linear layer's weight ([out, in], src/halite/transformers/feedforward.py:
// 204-212; src/halite/transformers/infer/attention.py:21-24).
//
// Two kernels.  The tiled one (any M): each output element is one chain of K multiply-adds
// in index order.  The one for at most 16 rows (decode steps), which the tiled one serves
// at 1/64 to 1/4 of its tile: a wave takes a few columns of the output, its lanes take
// every 64th group of four k each (the rows of A come through LDS, shared by the workgroup's
// four waves), and the lanes' partial sums are added in a fixed tree.
// In both a token's result depends on its own row alone, not on what else is in the batch;
// between the two the order of the additions differs, i.e. the last bits may.
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

// ---- at most 16 rows ------------------------------------------------------------------------
// A wave computes MB x NC outputs (MB * NC = 64).  Lane l holds the partial sums of the k's
// 4 (l + 64 i) .. + 3, added in rising k.  Then the 64 sums of a wave are added across the
// lanes in six halving steps (a lane keeps the half of the values that its bit picks and
// hands the other half to its partner), after which lane l holds output l whole.
template <int MB, int NC>
__global__ void __launch_bounds__(256)
gemm_f32_skinny_kernel(const float* __restrict__ A, int lda, const float* __restrict__ W, int ldw,
                       float* __restrict__ C, int ldc, int M, int N, int K) {
  static_assert(MB * NC == HAL_WAVE, "one output per lane");
  // The rows of A go through LDS in pieces of CH k, brought by all four waves together (a
  // wave that read them itself would ask memory for as many bytes of A as of W); the next
  // piece is on its way to registers while this one is worked on.
  constexpr int CH = 8192 / MB;                // k of a piece: 32 KB of LDS
  constexpr int AV = MB * CH / 4 / 256;        // 16-byte vectors of a piece per thread
  __shared__ __align__(16) float a_s[MB][CH];
  const int tid = threadIdx.x, lane = tid % HAL_WAVE, wave = tid / HAL_WAVE;
  const int n0 = (blockIdx.x * 4 + wave) * NC;
  const bool have_columns = n0 < N;  // (a wave without columns still helps with A)
  const float* wrow[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) wrow[c] = W + (size_t)(n0 + c < N ? n0 + c : N - 1) * ldw;
  float v[MB * NC];
#pragma unroll
  for (int i = 0; i < MB * NC; ++i) v[i] = 0.f;
  float4 a_next[AV];
  auto ask_piece = [&](int k0) {  // vector e of the piece: row e / (CH/4), k0 + 4 (e % (CH/4))
#pragma unroll
    for (int u = 0; u < AV; ++u) {
      const int e = tid + u * 256, m = e / (CH / 4), k = k0 + (e % (CH / 4)) * 4;
      a_next[u] = (m < M && k < K) ? *(const float4*)(A + (size_t)m * lda + k) : float4{0.f, 0.f, 0.f, 0.f};
    }
  };
  ask_piece(0);
  for (int k0 = 0; k0 < K; k0 += CH) {
    __syncthreads();  // the piece before is read
#pragma unroll
    for (int u = 0; u < AV; ++u) {
      const int e = tid + u * 256;
      *(float4*)&a_s[e / (CH / 4)][(e % (CH / 4)) * 4] = a_next[u];
    }
    if (k0 + CH < K) ask_piece(k0 + CH);
    __syncthreads();
    if (!have_columns) continue;
    const int k_end = k0 + CH < K ? k0 + CH : K;
    for (int k = k0 + lane * 4; k < k_end; k += HAL_WAVE * 4) {  // K is a multiple of 4
      float4 w[NC], a[MB];
#pragma unroll
      for (int c = 0; c < NC; ++c) w[c] = *(const float4*)(wrow[c] + k);
#pragma unroll
      for (int m = 0; m < MB; ++m) a[m] = *(const float4*)&a_s[m][k - k0];
#pragma unroll
      for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          float s = v[m * NC + c];
          s = fmaf(a[m].x, w[c].x, s);
          s = fmaf(a[m].y, w[c].y, s);
          s = fmaf(a[m].z, w[c].z, s);
          s = fmaf(a[m].w, w[c].w, s);
          v[m * NC + c] = s;
        }
    }
  }
  if (!have_columns) return;
#pragma unroll
  for (int half = HAL_WAVE / 2; half >= 1; half /= 2) {
    const bool upper = (lane & half) != 0;
#pragma unroll
    for (int i = 0; i < half; ++i) {
      const float keep = upper ? v[i + half] : v[i];
      const float give = upper ? v[i] : v[i + half];
      v[i] = keep + __shfl_xor(give, half, HAL_WAVE);
    }
  }
  const int m = lane / NC, c = lane % NC;
  if (m < M && n0 + c < N) C[(size_t)m * ldc + n0 + c] = v[0];
}

extern "C" int hal_gemm_f32(const float* A, int lda, const float* W, int ldw, float* C, int ldc,
                            int M, int N, int K, hipStream_t stream) {
  HAL_REQUIRE(M >= 0 && N > 0 && K > 0, "hal_gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
  HAL_REQUIRE(lda >= K && ldw >= K && ldc >= N, "hal_gemm_f32: leading dimensions %d %d %d", lda,
              ldw, ldc);
  if (M == 0) return 0;
  if (M <= 16 && K % 4 == 0 && lda % 4 == 0 && ldw % 4 == 0 && ((uintptr_t)A % 16) == 0 &&
      ((uintptr_t)W % 16) == 0) {
    if (M <= 8) {
      hipLaunchKernelGGL((gemm_f32_skinny_kernel<8, 8>), dim3((N + 31) / 32), dim3(256), 0, stream, A, lda,
                         W, ldw, C, ldc, M, N, K);
    } else {
      hipLaunchKernelGGL((gemm_f32_skinny_kernel<16, 4>), dim3((N + 15) / 16), dim3(256), 0, stream, A, lda,
                         W, ldw, C, ldc, M, N, K);
    }
    HAL_LAUNCH_CHECK();
    return 0;
  }
  dim3 grid((N + GF_BN - 1) / GF_BN, (M + GF_BM - 1) / GF_BM);
  HAL_REQUIRE(grid.y <= 65535, "hal_gemm_f32: M=%d exceeds the grid limit", M);
  hipLaunchKernelGGL(gemm_f32_kernel, grid, dim3(256), 0, stream, A, lda, W, ldw, C, ldc, M, N, K);
  HAL_LAUNCH_CHECK();
  return 0;
}
