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

}  // namespace

TL_EXPORT int tl_gemm_f32(const float* A, int lda, const float* W, int ldw, float* C, int ldc, int M, int N,
                          int K, hipStream_t stream) {
  TL_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
  TL_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_f32: leading dimensions too small");
  if (M == 0) return TL_OK;
  const unsigned gy = (M + BM - 1) / BM;
  TL_REQUIRE(gy <= 65535, "gemm_f32: M=%d exceeds the grid limit of one launch", M);
  dim3 grid((N + BN - 1) / BN, gy);
  gemm_f32_kernel<<<grid, kThreads, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K);
  return tl_check_launch("gemm_f32");
}
