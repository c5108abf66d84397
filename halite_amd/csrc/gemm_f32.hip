// C[M, N] = A[M, K] * W[N, K]^T in true float32: float32 multiply-adds on the vector units
// or the matrix cores' float32 instruction, no mode of reduced precision.  W has the layout
// of a bias-free linear layer's weight ([out, in], src/halite/transformers/feedforward.py:
// 204-212; src/halite/transformers/infer/attention.py:21-24).
//
// Four kernels.  At most 16 rows (decode steps): a wave takes a few columns of the output,
// its lanes take every 64th group of four k each (the rows of A come through LDS, shared by
// the workgroup's four waves), and the partial sums of the lanes, and of the waves that share
// columns, are added in a fixed order.  17 to about 100 rows: the matrix cores, k split over a
// workgroup's waves, each staging whole rows through LDS of its own.  More rows: tiles of 128 rows and 128 or 32
// columns on the matrix cores, through LDS.  For sizes and addresses that are no multiples of
// four: tiles of 64 x 64 on the vector units, each output element one chain of K
// multiply-adds in index order.
// In all of them a token's result depends on its own row alone, not on what else is in the
// batch; between them the order of the additions differs, i.e. the last bits may.
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

// ---- many rows: the matrix cores' float32 instruction -----------------------------------------
// v_mfma_f32_32x32x2_f32 multiplies and adds in float32 (it is the instruction behind the
// published float32 matrix rate, not one of the reduced-precision modes), at twice the rate of
// the vector units' multiply-adds.  A workgroup of four waves takes 128 x 128 outputs, a wave
// 64 x 64 as 2 x 2 products of 32 x 32; k goes through LDS 32 at a time, in two buffers, the
// next stage on its way to registers while this one is multiplied.
//
// The instruction takes, from lane l, A[row l % 32][k l / 32] and B[k l / 32][column l % 32],
// two k a call.  Which two k of the stage a call gets is free as long as A and B agree: the
// lower half of the lanes takes the k's 8 s .. 8 s + 3, the upper half 8 s + 4 .. 8 s + 7
// (s = 0 .. 3), one 16-byte LDS read per operand block and four calls each.  An output element
// is the sum over k in that order, in stretches of 512 that each start from nothing (see the
// kernel), rounded as the instruction rounds; it depends on its own row of A alone.
#define MF_BM 128
#define MF_BN 128
#define MF_BK 32
#define MF_KQ (MF_BK / 4)
#define MF_STRETCH 512  // k of a stretch that is summed from nothing
#define MF_XCDS 8  // dies of the gfx950 parts that this library is built for (a wrong count costs cache hits only)
typedef __attribute__((ext_vector_type(16))) float f32x16;

// BN: columns of a workgroup's tile, 128 (a wave takes 64 x 64 as 2 x 2 products) or 32 (a wave
// takes 32 x 32): the narrow tile is for products of so few rows and columns that tiles of 128
// columns would leave most of the chip empty.  An output element's sum is the same in both.
template <int BN>
__global__ void __launch_bounds__(256, 2)
gemm_f32_mfma_kernel(const float* __restrict__ A, int lda, const float* __restrict__ W, int ldw,
                     float* __restrict__ C, int ldc, int M, int N, int K, int tiles_m, int tiles_n) {
  constexpr int NB = BN == 128 ? 2 : 1;     // 32 x 32 products of a wave, each way
  constexpr int WV = BN * MF_KQ / 256;      // 16-byte vectors of W's stage per thread
  static_assert(BN == 128 || BN == 32, "tiles of 128 or 32 columns");
  // [buffer][k / 4][row], a row more than there are so that the stores of a wave (a row's
  // eight vectors side by side) spread over the banks
  __shared__ float4 a_s[2][MF_KQ][MF_BM + 1];
  __shared__ float4 w_s[2][MF_KQ][BN + 1];
  const int tid = threadIdx.x, lane = tid % HAL_WAVE, wave = tid / HAL_WAVE;
  // Workgroups go to the eight dies in turn, each die with a cache of its own: renumber them
  // so that a die's workgroups are neighbours in the order of tiles (the same columns of W,
  // rows of A one after the other).
  int id = blockIdx.x;
  const int n_tiles = tiles_m * tiles_n;
  if (n_tiles % MF_XCDS == 0) id = (id % MF_XCDS) * (n_tiles / MF_XCDS) + id / MF_XCDS;
  const int m0 = (id % tiles_m) * MF_BM, n0 = (id / tiles_m) * BN;

  float4 a_next[4], w_next[WV];
  auto ask = [&](int k0) {  // vector e of a stage: row e / 8, k0 + 4 (e % 8)
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = tid + u * 256, r = e / MF_KQ, k = k0 + (e % MF_KQ) * 4;
      const bool in = k < K && m0 + r < M;  // (K is a multiple of 4)
      a_next[u] = in ? *(const float4*)(A + (size_t)(m0 + r) * lda + k) : float4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int u = 0; u < WV; ++u) {
      const int e = tid + u * 256, r = e / MF_KQ, k = k0 + (e % MF_KQ) * 4;
      const bool in = k < K && n0 + r < N;
      w_next[u] = in ? *(const float4*)(W + (size_t)(n0 + r) * ldw + k) : float4{0.f, 0.f, 0.f, 0.f};
    }
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = tid + u * 256;
      a_s[buf][e % MF_KQ][e / MF_KQ] = a_next[u];
    }
#pragma unroll
    for (int u = 0; u < WV; ++u) {
      const int e = tid + u * 256;
      w_s[buf][e % MF_KQ][e / MF_KQ] = w_next[u];
    }
  };

  // An output element is summed in stretches of MF_STRETCH k, each from nothing, and the
  // stretches' sums are added in order: one chain of K additions would round K / 2 times on top
  // of each other (measured: four times the error of this at K = 14,336).
  f32x16 acc[NB][NB], total[NB][NB];
#pragma unroll
  for (int i = 0; i < NB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = total[i][j][v] = 0.f;
  // this wave's corner of the tile
  const int wm = BN == 128 ? (wave / 2) * 64 : wave * 32, wn = BN == 128 ? (wave % 2) * 64 : 0;
  const int rows = wm + lane % 32, cols = wn + lane % 32, half = lane / 32;
  const bool wave_has_rows = m0 + wm < M;  // (a wave whose rows are all beyond M only helps to load)

  ask(0);
  put(0);
  __syncthreads();
  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += MF_BK, buf ^= 1) {
    const bool more = k0 + MF_BK < K;
    if (more) ask(k0 + MF_BK);
    if (wave_has_rows) {
#pragma unroll
      for (int s = 0; s < MF_KQ / 2; ++s) {
        const int kq = 2 * s + half;
        float av[NB][4], bv[NB][4];
#pragma unroll
        for (int i = 0; i < NB; ++i) {
          const float4 a = a_s[buf][kq][rows + 32 * i], b = w_s[buf][kq][cols + 32 * i];
          av[i][0] = a.x, av[i][1] = a.y, av[i][2] = a.z, av[i][3] = a.w;
          bv[i][0] = b.x, bv[i][1] = b.y, bv[i][2] = b.z, bv[i][3] = b.w;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
          for (int i = 0; i < NB; ++i)
#pragma unroll
            for (int j = 0; j < NB; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i][e], bv[j][e], acc[i][j], 0, 0, 0);
      }
    }
    if ((k0 + MF_BK) % MF_STRETCH == 0 || !more) {  // (the same for every thread)
#pragma unroll
      for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            total[i][j][v] += acc[i][j][v];
            acc[i][j][v] = 0.f;
          }
    }
    if (more) put(buf ^ 1);  // (read last in the stage before the one that just ended)
    __syncthreads();
  }
  // element v of a lane's 16: row 8 (v / 4) + 4 (lane / 32) + v % 4, column lane % 32
#pragma unroll
  for (int i = 0; i < NB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int gn = n0 + wn + j * 32 + lane % 32;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int gm = m0 + wm + i * 32 + 8 * (v / 4) + 4 * half + v % 4;
        if (gm < M && gn < N) C[(size_t)gm * ldc + gn] = total[i][j][v];
      }
    }
}

// ---- 17 to 128 rows: the same instruction, k split over a workgroup's waves -----------------
// Too many rows for the vector units' kernel below, too few for tiles to fill the chip: what
// counts is that W streams.  A workgroup takes 32 columns (rows of W) and all rows of A; its
// waves split k into stretches, one each, and work on their own from there: no barrier until
// the end.  A wave brings a stage (32 k) of its 32 rows of W and of the rows of A in whole rows
// (a load instruction reads eight rows of 128 bytes: eight cache lines; read in the operands'
// own order, lane = row, it would touch 32 lines for the same bytes, which measured half the
// rate), DEPTH stages ahead of the products, puts it into LDS of its own in the order of the
// tiles above ([k / 4][row]) and reads the operands from there; a wave's LDS operations keep
// their order, so one buffer will do.  W is the first operand, so a lane ends with one row of
// A and sixteen columns; the waves' sums meet in LDS and are added in rising wave number.
// MB: blocks of 32 rows of A (M <= 32 MB).  An output element's sum depends on K and on the
// number of waves, i.e. on the matrix and on MB, and not on the rows beside it.
// LDS that one lane of a wave writes and another reads: the wave's LDS operations are done in
// the order they were issued; this keeps the compiler from moving them across.
__device__ __forceinline__ void rows_wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int MB, int ROWS_WAVES>
__global__ void __launch_bounds__(64 * ROWS_WAVES)
gemm_f32_rows_kernel(const float* __restrict__ A, int lda, const float* __restrict__ W, int ldw,
                     float* __restrict__ C, int ldc, int M, int N, int K) {
  constexpr int DEPTH = MB == 1 ? 4 : 2;  // stages in registers
  constexpr int WS = 33, AS = 32 * MB + 1;  // rows of a stage and one more (the stores spread over the banks)
  // per wave: W's stage [8][WS] and A's [8][AS] vectors; afterwards the waves' sums [32][33] floats
  constexpr int PART = MF_KQ * (WS + AS);  // vectors of a wave
  extern __shared__ float4 stage_s[];      // [ROWS_WAVES][PART]
  static_assert(sizeof(float4) * PART >= sizeof(float) * 32 * 33, "the sums fit where the stages were");
  const int tid = threadIdx.x, lane = tid % HAL_WAVE, wave = tid / HAL_WAVE;
  const int col = lane % 32, half = lane / 32;
  const int n0 = blockIdx.x * 32;
  float4* w_s = stage_s + wave * PART;
  float4* a_s = w_s + MF_KQ * WS;
  // this wave's stretch of k: whole stages of 32
  const int stages = (K + 31) / 32, each = (stages + ROWS_WAVES - 1) / ROWS_WAVES;
  const int k_begin = wave * each * 32, k_end = min(K, (wave + 1) * each * 32);
  // vector e = lane + 64 u of a stage: row e / 8, k 4 (e % 8)
  const int r0 = lane / MF_KQ, kq0 = lane % MF_KQ;
  float4 wr[DEPTH][4], ar[DEPTH][4 * MB];
  auto ask = [&](int d, int k) {  // (K is a multiple of 4: a vector is inside or outside)
    const bool k_in = k + 4 * kq0 < k_end;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int r = r0 + 8 * u;
      wr[d][u] = (k_in && n0 + r < N) ? *(const float4*)(W + (size_t)(n0 + r) * ldw + k + 4 * kq0) : float4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int u = 0; u < 4 * MB; ++u) {
      const int r = r0 + 8 * u;
      ar[d][u] = (k_in && r < M) ? *(const float4*)(A + (size_t)r * lda + k + 4 * kq0) : float4{0.f, 0.f, 0.f, 0.f};
    }
  };
  f32x16 acc[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[b][v] = 0.f;
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) ask(d, k_begin + 32 * d);
  for (int k = k_begin; k < k_end; k += 32 * DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {  // (stages beyond the stretch hold zeros)
#pragma unroll
      for (int u = 0; u < 4; ++u) w_s[kq0 * WS + r0 + 8 * u] = wr[d][u];
#pragma unroll
      for (int u = 0; u < 4 * MB; ++u) a_s[kq0 * AS + r0 + 8 * u] = ar[d][u];
      rows_wave_sync();  // what one lane put down another reads
      ask(d, k + 32 * (d + DEPTH));  // (the other stages are on their way meanwhile)
#pragma unroll
      for (int s4 = 0; s4 < MF_KQ / 2; ++s4) {
        const int kq = 2 * s4 + half;
        const float4 w = w_s[kq * WS + col];
        const float wv[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int b = 0; b < MB; ++b) {
          const float4 a = a_s[kq * AS + 32 * b + col];
          const float av[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(wv[e], av[e], acc[b], 0, 0, 0);
        }
      }
      rows_wave_sync();  // the stage is read before the next one is put down
    }
  }
  // element v of a lane's 16: column 8 (v / 4) + 4 half + v % 4 of the workgroup's 32, row `col` of the block
  float* sums = (float*)stage_s;  // [wave][32][33], a wave's part where its stages were
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    __syncthreads();  // the block before is added up (and, the first time, every wave is done with its stages)
#pragma unroll
    for (int v = 0; v < 16; ++v) sums[wave * 4 * PART + col * 33 + 8 * (v / 4) + 4 * half + v % 4] = acc[b][v];
    __syncthreads();
    for (int e = tid; e < 32 * 32; e += 64 * ROWS_WAVES) {
      const int m = 32 * b + e / 32, n = n0 + e % 32;
      float total = sums[(e / 32) * 33 + e % 32];
#pragma unroll
      for (int w = 1; w < ROWS_WAVES; ++w) total += sums[w * 4 * PART + (e / 32) * 33 + e % 32];
      if (m < M && n < N) C[(size_t)m * ldc + n] = total;
    }
  }
}

template <int MB, int WAVES>
static int launch_rows_with(const float* A, int lda, const float* W, int ldw, float* C, int ldc, int M, int N,
                            int K, hipStream_t stream) {
  const size_t smem = (size_t)WAVES * MF_KQ * (33 + 32 * MB + 1) * sizeof(float4);
  static bool raised = false;  // more than 64 KB of LDS has to be asked for, once per kernel
  if (!raised && smem > 64 * 1024) {
    HAL_CHECK_HIP(hipFuncSetAttribute((const void*)gemm_f32_rows_kernel<MB, WAVES>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    raised = true;
  }
  hipLaunchKernelGGL((gemm_f32_rows_kernel<MB, WAVES>), dim3((N + 31) / 32), dim3(64 * WAVES), smem, stream, A,
                     lda, W, ldw, C, ldc, M, N, K);
  return 0;
}

// eight waves a workgroup where few columns leave compute units idle, four otherwise
template <int MB>
static int launch_rows(const float* A, int lda, const float* W, int ldw, float* C, int ldc, int M, int N,
                       int K, hipStream_t stream) {
  if ((N + 31) / 32 < 256) return launch_rows_with<MB, 8>(A, lda, W, ldw, C, ldc, M, N, K, stream);
  return launch_rows_with<MB, 4>(A, lda, W, ldw, C, ldc, M, N, K, stream);
}

// ---- at most 16 rows ------------------------------------------------------------------------
// A wave computes partial sums of MB x NC outputs (MB * NC = 64).  k is cut into blocks of 256;
// KW waves of a workgroup share a set of columns and take every KW-th block each (KW = 1: a
// wave has its columns to itself), and inside a block lane l has the k's 4 l .. 4 l + 3.  A lane
// adds its products up in rising k.  Then the 64 sums of a wave are added across the lanes in
// six halving steps (a lane keeps the half of the values that its bit picks and hands the other
// half to its partner), after which lane l holds output l of its wave's blocks, and the KW
// waves' sums are added in rising wave number.  The order depends on KW, i.e. on the weight's
// size, and not on the number of rows.
//
// Why KW: a matrix of few columns gives few workgroups (4096 columns: 128 of four waves with
// eight columns each), and with one wave on half of the compute units, each waiting for 8 KB
// at a time, memory is asked for too little at once (measured 1.2 TB/s on 4096 x 4096).  With
// the k's split over the waves such a matrix gives four times the workgroups, and every wave
// asks for its next block before it works on the one it has.
template <int MB, int NC, int KW>
__global__ void __launch_bounds__(256, 2)
gemm_f32_skinny_kernel(const float* __restrict__ A, int lda, const float* __restrict__ W, int ldw,
                       float* __restrict__ C, int ldc, int M, int N, int K) {
  static_assert(MB * NC == HAL_WAVE, "one output per lane");
  // The rows of A go through LDS in pieces of CH k, brought by all four waves together (a
  // wave that read them itself would ask memory for as many bytes of A as of W); the next
  // piece is on its way to registers while this one is worked on.
  constexpr int CH = 1024;                     // k of a piece: 4 KB of LDS a row
  constexpr int AV = MB * CH / 4 / 256;        // 16-byte vectors of a piece per thread
  constexpr int BLOCK = HAL_WAVE * 4;          // k of a block
  constexpr int NB = CH / BLOCK / KW;          // blocks of a piece per wave
  static_assert(NB >= 1, "a piece has a block for every wave");
  __shared__ __align__(16) float a_s[MB][CH];
  __shared__ float sums[4][HAL_WAVE];
  const int tid = threadIdx.x, lane = tid % HAL_WAVE, wave = tid / HAL_WAVE;
  const int kw = wave % KW;  // which of the blocks, and
  const int n0 = (blockIdx.x * (4 / KW) + wave / KW) * NC;  // which columns
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
  // this wave's b-th block of the piece at k0 begins at k0 + (b * KW + kw) * BLOCK
  float4 w_next[NC];
  auto ask_block = [&](int k) {  // (K is a multiple of 4: a lane's four k are there or not)
#pragma unroll
    for (int c = 0; c < NC; ++c)
      w_next[c] = (have_columns && k < K) ? *(const float4*)(wrow[c] + k) : float4{0.f, 0.f, 0.f, 0.f};
  };
  ask_block(kw * BLOCK + lane * 4);
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
#pragma unroll 1  // (unrolled, the blocks' values of A would wait in registers that are not there)
    for (int b = 0; b < NB; ++b) {
      const int at = (b * KW + kw) * BLOCK + lane * 4;  // inside the piece
      float4 w[NC];
#pragma unroll
      for (int c = 0; c < NC; ++c) w[c] = w_next[c];
      // the block after this one, in this piece or the next (beyond K: zeros, never used)
      ask_block(b + 1 < NB ? k0 + at + KW * BLOCK : k0 + CH + kw * BLOCK + lane * 4);
#pragma unroll
      for (int m = 0; m < MB; ++m) {
        const float4 a = *(const float4*)&a_s[m][at];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          float s = v[m * NC + c];
          s = fmaf(a.x, w[c].x, s);
          s = fmaf(a.y, w[c].y, s);
          s = fmaf(a.z, w[c].z, s);
          s = fmaf(a.w, w[c].w, s);
          v[m * NC + c] = s;
        }
      }
    }
  }
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
  float total = v[0];
  if (KW > 1) {
    sums[wave][lane] = total;
    __syncthreads();
    if (kw != 0) return;
    total = sums[wave][lane];
#pragma unroll
    for (int j = 1; j < KW; ++j) total += sums[wave + j][lane];
  }
  const int m = lane / NC, c = lane % NC;
  if (m < M && n0 + c < N) C[(size_t)m * ldc + n0 + c] = total;
}

template <int MB, int NC>
static void launch_skinny(const float* A, int lda, const float* W, int ldw, float* C, int ldc, int M,
                          int N, int K, hipStream_t stream) {
  // as many waves on a set of columns as it takes for 512 workgroups or more, counted for eight
  // columns a wave whatever NC is: the order of the additions is the same for every M
  const int alone = (N + 31) / 32;
  if (alone >= 512)
    hipLaunchKernelGGL((gemm_f32_skinny_kernel<MB, NC, 1>), dim3((N + 4 * NC - 1) / (4 * NC)), dim3(256), 0,
                       stream, A, lda, W, ldw, C, ldc, M, N, K);
  else if (alone >= 256)
    hipLaunchKernelGGL((gemm_f32_skinny_kernel<MB, NC, 2>), dim3((N + 2 * NC - 1) / (2 * NC)), dim3(256), 0,
                       stream, A, lda, W, ldw, C, ldc, M, N, K);
  else
    hipLaunchKernelGGL((gemm_f32_skinny_kernel<MB, NC, 4>), dim3((N + NC - 1) / NC), dim3(256), 0, stream,
                       A, lda, W, ldw, C, ldc, M, N, K);
}

extern "C" int hal_gemm_f32(const float* A, int lda, const float* W, int ldw, float* C, int ldc,
                            int M, int N, int K, hipStream_t stream) {
  HAL_REQUIRE(M >= 0 && N > 0 && K > 0, "hal_gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
  HAL_REQUIRE(lda >= K && ldw >= K && ldc >= N, "hal_gemm_f32: leading dimensions %d %d %d", lda,
              ldw, ldc);
  if (M == 0) return 0;
  if (M <= 16 && K % 4 == 0 && lda % 4 == 0 && ldw % 4 == 0 && ((uintptr_t)A % 16) == 0 &&
      ((uintptr_t)W % 16) == 0) {
    if (M <= 8)
      launch_skinny<8, 8>(A, lda, W, ldw, C, ldc, M, N, K, stream);
    else
      launch_skinny<16, 4>(A, lda, W, ldw, C, ldc, M, N, K, stream);
    HAL_LAUNCH_CHECK();
    return 0;
  }
  if (K % 4 == 0 && lda % 4 == 0 && ldw % 4 == 0 && ((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0) {
    // up to 96 rows, and up to 128 on matrices of few columns: k split over a workgroup's waves (measured
    // against the tiles below on the 8B shape's matrices: o-proj 31 / 50 / 74 / 100 us at 32 / 64 / 96 / 128
    // rows against 120; gate and up together 129 / 204 / 287 / 414 us against 275 to 368)
    if (M <= 96 || (M <= 128 && (N + 127) / 128 < 128)) {
      if (M <= 32 ? launch_rows<1>(A, lda, W, ldw, C, ldc, M, N, K, stream)
          : M <= 64 ? launch_rows<2>(A, lda, W, ldw, C, ldc, M, N, K, stream)
          : M <= 96 ? launch_rows_with<3, 4>(A, lda, W, ldw, C, ldc, M, N, K, stream)
                    : launch_rows_with<4, 4>(A, lda, W, ldw, C, ldc, M, N, K, stream))
        return 1;
      HAL_LAUNCH_CHECK();
      return 0;
    }
    // more rows: the matrix cores, in tiles of 128 columns where those fill the chip
    const long long tiles_m = (M + MF_BM - 1) / MF_BM, wide = (N + 127) / 128, narrow = (N + 31) / 32;
    const bool use_wide = tiles_m * wide >= 256;
    const long long tiles_n = use_wide ? wide : narrow;
    HAL_REQUIRE(tiles_m * tiles_n < (1ll << 31), "hal_gemm_f32: M=%d N=%d exceed the grid limit", M, N);
    if (use_wide)
      hipLaunchKernelGGL(gemm_f32_mfma_kernel<128>, dim3((unsigned)(tiles_m * tiles_n)), dim3(256), 0, stream, A,
                         lda, W, ldw, C, ldc, M, N, K, (int)tiles_m, (int)tiles_n);
    else
      hipLaunchKernelGGL(gemm_f32_mfma_kernel<32>, dim3((unsigned)(tiles_m * tiles_n)), dim3(256), 0, stream, A,
                         lda, W, ldw, C, ldc, M, N, K, (int)tiles_m, (int)tiles_n);
    HAL_LAUNCH_CHECK();
    return 0;
  }
  dim3 grid((N + GF_BN - 1) / GF_BN, (M + GF_BM - 1) / GF_BM);
  HAL_REQUIRE(grid.y <= 65535, "hal_gemm_f32: M=%d exceeds the grid limit", M);
  hipLaunchKernelGGL(gemm_f32_kernel, grid, dim3(256), 0, stream, A, lda, W, ldw, C, ldc, M, N, K);
  HAL_LAUNCH_CHECK();
  return 0;
}
