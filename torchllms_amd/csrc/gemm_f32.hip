// C[M, N] = A[M, K] * W[N, K]^T in true 32-bit: float inputs, float FMA accumulation, no matrix-core
// reduced-precision mode.  Each output element is accumulated by one thread over k = 0..K-1 in
// ascending order (in groups of 16 that are added up first), so its value does not depend on M or on
// where the row sits in the batch.
// Throughput is secondary: this is the matrix product of the 32-bit path.
#include "common.h"

namespace {

constexpr int BM = 64, BN = 64, BK = 16, TM = 4, TN = 4;
constexpr int kThreads = (BM / TM) * (BN / TN);  // 256

__global__ void __launch_bounds__(kThreads)
gemm_f32_kernel(const float* __restrict__ A, int lda, const float* __restrict__ W, int ldw,
                float* __restrict__ C, int ldc, int M, int N, int K) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % (BN / TN);  // column group
  const int ty = tid / (BN / TN);  // row group
  const int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * BN;

  float acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += BK) {
    // each thread loads 4 elements of each tile: tile row = tid / 4, k offsets (tid % 4) * 4 .. +3
    {
      const int r = tid / 4;
      const int kk = (tid % 4) * 4;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = k0 + kk + u;
        const int m = m0 + r;
        As[kk + u][r] = (m < M && k < K) ? A[(size_t)m * lda + k] : 0.f;
        const int n = n0 + r;
        Ws[kk + u][r] = (n < N && k < K) ? W[(size_t)n * ldw + k] : 0.f;
      }
    }
    __syncthreads();
    // the BK products of this step are added among themselves first and then to the running sum:
    // the rounding error of a long sum grows with the number of additions to one accumulator, and
    // this way there are K / BK + BK of them instead of K (at K = 1024 the 32-bit model's distance
    // from a 64-bit computation halves); the order is still fixed by K alone
    float part[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) part[i][j] = 0.f;
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float a[TM], w[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = As[k][ty * TM + i];
#pragma unroll
      for (int j = 0; j < TN; ++j) w[j] = Ws[k][tx * TN + j];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) part[i][j] = fmaf(a[i], w[j], part[i][j]);
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] += part[i][j];
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + ty * TM + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + tx * TN + j;
      if (n < N) C[(size_t)m * ldc + n] = acc[i][j];
    }
  }
}

// ----------------------------------------------------------------------------- few rows (decode steps)
// The kernel above gives a block 64 rows of A; a decode step has one to sixteen, and its grid is then
// N / 64 blocks that walk all of K in steps of 16 with two barriers each: a 4096 x 14336 matrix took
// over a millisecond.  This kernel computes the very same arithmetic for every output element (groups
// of 16 products, chained by fused multiply-adds from k ascending, each group's sum added to the
// running sum in the order of the groups), so its results are the same bits, but spreads the groups
// of an element over the lanes of a wave:
//   * a block of 4 waves takes 16 columns of the result, 4 per wave, and all rows (at most MR);
//   * K is walked in rounds of 1,024 = 64 groups: lane j computes group j of the round for its wave's
//     4 columns and every row (W: 64 contiguous bytes per lane and column, the wave reads 4 KB on end;
//     A: the round's slice of every row lies in LDS, loaded once per block, transposed so that the 64
//     lanes read 64 consecutive words);
//   * the groups' sums then have to join the running sums in the order of the groups: they go through
//     LDS, transposed, and lane p of the wave adds the 64 sums of (column, row) pair p one after the other.
constexpr int kRowsCols = 4;               // columns per wave
constexpr int kRowsWaves = 4;              // waves per block
constexpr int kRound = 64 * BK;            // k per round
constexpr int kPad = 65;                   // row stride of transposed tables in LDS (odd: no bank conflicts)

template <int MR>
__global__ void __launch_bounds__(kRowsWaves * kWave)
gemm_f32_rows_kernel(const float* __restrict__ A, int lda, const float* __restrict__ W, int ldw,
                     float* __restrict__ C, int ldc, int M, int N, int K) {
  constexpr int kPairs = kRowsCols * MR;   // (column, row) pairs of a wave: at most 64
  extern __shared__ float lds[];
  float* xs = lds;                                          // [MR][BK][kPad]: element u of group j of row m at (m * BK + u) * kPad + j
  float* ps = lds + MR * BK * kPad;                         // [waves][kPairs][kPad]
  const int tid = threadIdx.x;
  const int wave = tid / kWave;
  const int lane = tid % kWave;
  float* my_ps = ps + wave * kPairs * kPad;
  const int n0 = (blockIdx.x * kRowsWaves + wave) * kRowsCols;

  float acc = 0.f;  // lane p < kPairs: running sum of pair p = (column p / MR, row p % MR)

  for (int k0 = 0; k0 < K; k0 += kRound) {
    __syncthreads();  // everybody has finished with the slice of the round before
    for (int i = tid; i < MR * kRound; i += kRowsWaves * kWave) {
      const int m = i / kRound, kk = i % kRound, k = k0 + kk;
      xs[(m * BK + kk % BK) * kPad + kk / BK] = (m < M && k < K) ? A[(size_t)m * lda + k] : 0.f;
    }
    __syncthreads();
    const int kg = k0 + BK * lane;  // this lane's group of the round
    float part[kRowsCols][MR];
#pragma unroll
    for (int c = 0; c < kRowsCols; ++c)
#pragma unroll
      for (int m = 0; m < MR; ++m) part[c][m] = 0.f;
    float w[kRowsCols][BK];
#pragma unroll
    for (int c = 0; c < kRowsCols; ++c) {
      const int n = n0 + c;
      const float* wrow = W + (size_t)(n < N ? n : N - 1) * ldw;
      if (kg + BK <= K && (ldw % 4) == 0 && ((uintptr_t)W % 16) == 0) {
#pragma unroll
        for (int u = 0; u < BK; u += 4) {
          const float4 v = *reinterpret_cast<const float4*>(wrow + kg + u);
          w[c][u] = v.x; w[c][u + 1] = v.y; w[c][u + 2] = v.z; w[c][u + 3] = v.w;
        }
      } else {
#pragma unroll
        for (int u = 0; u < BK; ++u) w[c][u] = kg + u < K ? wrow[kg + u] : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < BK; ++u) {
#pragma unroll
      for (int m = 0; m < MR; ++m) {
        const float a = xs[(m * BK + u) * kPad + lane];
#pragma unroll
        for (int c = 0; c < kRowsCols; ++c) part[c][m] = fmaf(a, w[c][u], part[c][m]);
      }
    }
    // the sums of this lane's group, transposed: pair p's 64 sums lie side by side
#pragma unroll
    for (int c = 0; c < kRowsCols; ++c)
#pragma unroll
      for (int m = 0; m < MR; ++m) my_ps[(c * MR + m) * kPad + lane] = part[c][m];
    __syncthreads();
    if (lane < kPairs) {
      const float* mine = my_ps + lane * kPad;
      const int groups = min(64, (K - k0 + BK - 1) / BK);  // groups of this round that exist
      for (int g = 0; g < groups; ++g) acc += mine[g];
    }
  }
  if (lane < kPairs) {
    const int n = n0 + lane / MR, m = lane % MR;
    if (n < N && m < M) C[(size_t)m * ldc + n] = acc;
  }
}

}  // namespace

TL_EXPORT int tl_gemm_f32(const float* A, int lda, const float* W, int ldw, float* C, int ldc, int M, int N,
                          int K, hipStream_t stream) {
  TL_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
  TL_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_f32: leading dimensions too small");
  if (M == 0) return TL_OK;
  if (M <= 16) {
    // decode steps: the same sums, spread over a wave (see above)
    const unsigned blocks = (N + kRowsWaves * kRowsCols - 1) / (kRowsWaves * kRowsCols);
#define TL_ROWS_LAUNCH(MR)                                                                               \
  do {                                                                                                   \
    const size_t lds = ((size_t)MR * BK * kPad + (size_t)kRowsWaves * kRowsCols * MR * kPad) * sizeof(float); \
    if (lds > 48 * 1024) {                                                                               \
      hipError_t e = hipFuncSetAttribute((const void*)gemm_f32_rows_kernel<MR>,                          \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);          \
      if (e != hipSuccess) return tl_fail(TL_ERR_HIP, "gemm_f32: %s", hipGetErrorString(e));             \
    }                                                                                                    \
    gemm_f32_rows_kernel<MR><<<blocks, kRowsWaves * kWave, lds, stream>>>(A, lda, W, ldw, C, ldc, M, N, K); \
  } while (0)
    if (M == 1) TL_ROWS_LAUNCH(1);
    else if (M == 2) TL_ROWS_LAUNCH(2);
    else if (M <= 4) TL_ROWS_LAUNCH(4);
    else if (M <= 8) TL_ROWS_LAUNCH(8);
    else TL_ROWS_LAUNCH(16);
#undef TL_ROWS_LAUNCH
    return tl_check_launch("gemm_f32_rows");
  }
  const unsigned gy = (M + BM - 1) / BM;
  TL_REQUIRE(gy <= 65535, "gemm_f32: M=%d exceeds the grid limit of one launch", M);
  dim3 grid((N + BN - 1) / BN, gy);
  gemm_f32_kernel<<<grid, kThreads, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K);
  return tl_check_launch("gemm_f32");
}
