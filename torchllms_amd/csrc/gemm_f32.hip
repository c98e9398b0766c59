// C[M, N] = A[M, K] * W[N, K]^T in true 32-bit: float inputs, float FMA accumulation, no matrix-core
// reduced-precision mode.  Each output element is accumulated by one thread over k = 0..K-1 in
// ascending order (in groups of 16 that are added up first), so its value does not depend on M or on
// where the row sits in the batch.
// Throughput is secondary: this is the matrix product of the 32-bit path.
#include <type_traits>

#include "common.h"

namespace {

constexpr int BK = 16;  // products that are added among themselves before they join the running sum

// A block computes a BM x BN tile of C with (BM / TM) x (BN / TN) = 256 threads, each a TM x TN piece of it
// (its rows and columns in runs of four, so that operands come from LDS sixteen bytes at a time).  Tiles of A
// and W, BK wide, pass through LDS transposed (k-major); the next tiles travel from memory into registers
// while the current ones are multiplied, and two sets of LDS tiles leave one barrier a step.
// Two shapes: 64 x 64 with 4 x 4 a thread for steps of a few dozen rows, 128 x 128 with 8 x 8 a thread for
// prompts (twice the arithmetic per byte read from LDS).  The arithmetic of an output element is the same in
// both, and in the kernel for few rows below: the BK products of a step chained by fused multiply-adds from k
// ascending, starting from zero, then added to the running sum.
template <int BM, int BN, int TM, int TN>
__global__ void __launch_bounds__((BM / TM) * (BN / TN))
gemm_f32_kernel(const float* __restrict__ A, int lda, const float* __restrict__ W, int ldw,
                float* __restrict__ C, int ldc, int M, int N, int K) {
  constexpr int kThreads = (BM / TM) * (BN / TN);
  static_assert(kThreads == 256 && TM % 4 == 0 && TN % 4 == 0, "256 threads, pieces in runs of four");
  constexpr int kPerA = BM * BK / kThreads;  // elements of a tile that one thread moves: a run along k
  constexpr int kPerW = BN * BK / kThreads;
  static_assert(kPerA % 4 == 0 && kPerW % 4 == 0 && BK % kPerA == 0 && BK % kPerW == 0, "runs of whole float4s");
  constexpr int kPitchA = BM + 4, kPitchW = BN + 4;
  constexpr int kAhead = TM * TN >= 64 ? 2 : 4;  // steps of k whose operands are in registers together
  __shared__ __attribute__((aligned(16))) float As[2][BK][kPitchA];
  __shared__ __attribute__((aligned(16))) float Ws[2][BK][kPitchW];
  const int tid = threadIdx.x;
  const int tx = tid % (BN / TN);  // column group
  const int ty = tid / (BN / TN);  // row group
  // consecutive blocks share their columns: the tile of W is read from memory once for all of them
  const int m0 = blockIdx.x * BM;
  const int n0 = blockIdx.y * BN;
  // run r of the thread's rows is rows (BM / (TM / 4)) * r + 4 * ty ... + 3 of the tile; columns likewise
  constexpr int kRowRun = BM / (TM / 4), kColRun = BN / (TN / 4);

  float acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;

  // what this thread moves: row (of A or of W) and the run of k within the step
  const int ar = tid / (BK / kPerA), ak = (tid % (BK / kPerA)) * kPerA;
  const int wr = tid / (BK / kPerW), wk = (tid % (BK / kPerW)) * kPerW;
  const bool a_vec = (lda % 4) == 0 && ((uintptr_t)A % 16) == 0;
  const bool w_vec = (ldw % 4) == 0 && ((uintptr_t)W % 16) == 0;
  const float* a_row = A + (size_t)min(m0 + ar, M - 1) * lda;
  const float* w_row = W + (size_t)min(n0 + wr, N - 1) * ldw;
  const bool a_in = m0 + ar < M, w_in = n0 + wr < N;
  float ra[kPerA], rw[kPerW];
  auto fetch_run = [&](const float* row, bool inside, bool vec, int k, float* dst, auto per) {
    constexpr int kPer = decltype(per)::value;
    if (inside && vec && k + kPer <= K) {
#pragma unroll
      for (int u = 0; u < kPer; u += 4) {
        const float4 v = *reinterpret_cast<const float4*>(row + k + u);
        dst[u] = v.x; dst[u + 1] = v.y; dst[u + 2] = v.z; dst[u + 3] = v.w;
      }
    } else {
#pragma unroll
      for (int u = 0; u < kPer; ++u) dst[u] = (inside && k + u < K) ? row[k + u] : 0.f;
    }
  };
  auto fetch = [&](int k0) {
    fetch_run(a_row, a_in, a_vec, k0 + ak, ra, std::integral_constant<int, kPerA>{});
    fetch_run(w_row, w_in, w_vec, k0 + wk, rw, std::integral_constant<int, kPerW>{});
  };
  auto store = [&](int buffer) {
#pragma unroll
    for (int u = 0; u < kPerA; ++u) As[buffer][ak + u][ar] = ra[u];
#pragma unroll
    for (int u = 0; u < kPerW; ++u) Ws[buffer][wk + u][wr] = rw[u];
  };

  fetch(0);
  store(0);
  __syncthreads();
  int buffer = 0;
  for (int k0 = 0; k0 < K; k0 += BK) {
    const bool more = k0 + BK < K;
    if (more) fetch(k0 + BK);
    // the BK products of this step are added among themselves first and then to the running sum:
    // the rounding error of a long sum grows with the number of additions to one accumulator, and
    // this way there are K / BK + BK of them instead of K (at K = 1024 the 32-bit model's distance
    // from a 64-bit computation halves); the order is still fixed by K alone
    float part[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) part[i][j] = 0.f;
    // (unrolled by kAhead only: unrolled whole, the compiler asks for all sixteen steps' operands at once
    // and the large tile takes 405 registers)
#pragma unroll kAhead
    for (int k = 0; k < BK; ++k) {
      float a[TM], w[TN];
#pragma unroll
      for (int r = 0; r < TM / 4; ++r) {
        const float4 v = *reinterpret_cast<const float4*>(&As[buffer][k][kRowRun * r + 4 * ty]);
        a[4 * r] = v.x; a[4 * r + 1] = v.y; a[4 * r + 2] = v.z; a[4 * r + 3] = v.w;
      }
#pragma unroll
      for (int r = 0; r < TN / 4; ++r) {
        const float4 v = *reinterpret_cast<const float4*>(&Ws[buffer][k][kColRun * r + 4 * tx]);
        w[4 * r] = v.x; w[4 * r + 1] = v.y; w[4 * r + 2] = v.z; w[4 * r + 3] = v.w;
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) part[i][j] = fmaf(a[i], w[j], part[i][j]);
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] += part[i][j];
    if (more) store(buffer ^ 1);
    __syncthreads();
    buffer ^= 1;
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + kRowRun * (i / 4) + 4 * ty + i % 4;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + kColRun * (j / 4) + 4 * tx + j % 4;
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
//     4 columns and every row (W: the wave reads a column's 4 KB of the round 1 KB per instruction and
//     turns it through a piece of LDS of its own, so that lane j holds elements 16 j .. 16 j + 15;
//     A: the round's slice of every row lies in LDS, loaded once per block, transposed so that the 64
//     lanes read 64 consecutive words); what the next round needs travels from memory into registers
//     while this round is multiplied;
//   * the groups' sums then have to join the running sums in the order of the groups: they go through
//     LDS, transposed, and lane p of the wave adds the 64 sums of (column, row) pair p one after the other.
constexpr int kRowsCols = 4;               // columns per wave
constexpr int kRowsWaves = 4;              // waves per block
constexpr int kRound = 64 * BK;            // k per round
constexpr int kPad = 65;                   // row stride of transposed tables in LDS (odd: no bank conflicts)
constexpr int kTurned = kRound + kRound / 4;  // a column's round of W in LDS: four words of padding behind every group

template <int MR, bool kVec>
__global__ void __launch_bounds__(kRowsWaves * kWave)
gemm_f32_rows_kernel(const float* __restrict__ A, int lda, const float* __restrict__ W, int ldw,
                     float* __restrict__ C, int ldc, int M, int N, int K) {
  constexpr int kPairs = kRowsCols * MR;   // (column, row) pairs of a wave: at most 64
  constexpr int kWaveRegion = kPairs * kPad > kTurned ? kPairs * kPad : kTurned;
  extern __shared__ float lds[];
  float* xs = lds;                                          // [MR][BK][kPad]: element u of group j of row m at (m * BK + u) * kPad + j
  float* ps = lds + MR * BK * kPad;                         // [waves][kWaveRegion]: a wave's own piece
  const int tid = threadIdx.x;
  const int wave = tid / kWave;
  const int lane = tid % kWave;
  float* my_ps = ps + wave * kWaveRegion;                   // [kPairs][kPad] sums, or a column's round of W being turned
  const int n0 = (blockIdx.x * kRowsWaves + wave) * kRowsCols;

  float acc = 0.f;  // lane p < kPairs: running sum of pair p = (column p / MR, row p % MR)

  // What a round needs from memory is asked for a round ahead and waits in registers while the round
  // before it is multiplied.  Thread t moves elements 4 t .. 4 t + 3 of every row's slice of A; lane l
  // moves, of each of the wave's four columns of W, elements 256 q + 4 l .. + 3 for q = 0 .. 3 (the wave
  // reads 1 KB on end per instruction).
  // Two kernels (kVec): with rows of A and W on 16-byte boundaries and K a multiple of 4 everything is
  // fetched sixteen bytes a lane, otherwise element by element (one kernel with both forms under a branch
  // came out of the compiler with the element-wise loads for both).  Rows past M and elements past K are
  // read from a valid place (the row's last elements) and replaced by zeros when the round begins:
  // nothing here looks at a loaded value, or the wave would wait for each load in turn.
  float a_next[MR][4];
  float w_next[kRowsCols][BK];
  auto fetch = [&](int k0) {
    const int ka = k0 + 4 * tid;
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const float* arow = A + (size_t)(m < M ? m : 0) * lda;
      if constexpr (kVec) {
        const float4 v = *reinterpret_cast<const float4*>(arow + min(ka, K - 4));
        a_next[m][0] = v.x; a_next[m][1] = v.y; a_next[m][2] = v.z; a_next[m][3] = v.w;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) a_next[m][e] = arow[min(ka + e, K - 1)];
      }
    }
#pragma unroll
    for (int c = 0; c < kRowsCols; ++c) {
      const int n = n0 + c;
      const float* wrow = W + (size_t)(n < N ? n : N - 1) * ldw;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int k = k0 + 256 * q + 4 * lane;
        if constexpr (kVec) {
          const float4 v = *reinterpret_cast<const float4*>(wrow + min(k, K - 4));
          w_next[c][4 * q] = v.x; w_next[c][4 * q + 1] = v.y; w_next[c][4 * q + 2] = v.z; w_next[c][4 * q + 3] = v.w;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) w_next[c][4 * q + e] = wrow[min(k + e, K - 1)];
        }
      }
    }
  };

  fetch(0);
  for (int k0 = 0; k0 < K; k0 += kRound) {
    __syncthreads();  // everybody has finished with the slice of the round before
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int kk = 4 * tid + e;
        xs[(m * BK + kk % BK) * kPad + kk / BK] = (m < M && k0 + kk < K) ? a_next[m][e] : 0.f;
      }
    // the wave turns its columns of W through its own piece of LDS (free: the sums of the round before
    // have been added): lane j gets group j, elements 16 j .. 16 j + 15 of the round.  A wave's LDS
    // instructions are carried out in their order, so no barrier stands between the writes and the reads.
    float w[kRowsCols][BK];
#pragma unroll
    for (int c = 0; c < kRowsCols; ++c) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int kk = 256 * q + 4 * lane;
        const int left = K - (k0 + kk);  // elements of the row from here on: past them, zeros
        *reinterpret_cast<float4*>(my_ps + kk + 4 * (kk / BK)) =
            float4{left > 0 ? w_next[c][4 * q] : 0.f, left > 1 ? w_next[c][4 * q + 1] : 0.f,
                   left > 2 ? w_next[c][4 * q + 2] : 0.f, left > 3 ? w_next[c][4 * q + 3] : 0.f};
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int u = 0; u < BK; u += 4) {
        const float4 v = *reinterpret_cast<const float4*>(my_ps + (BK + 4) * lane + u);
        w[c][u] = v.x; w[c][u + 1] = v.y; w[c][u + 2] = v.z; w[c][u + 3] = v.w;
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
    // (asked for as soon as the registers are free, before the barrier: the fewer cycles a wave has no
    // load under way, the better; with two blocks a CU nobody else fills the gap)
    if (k0 + kRound < K) fetch(k0 + kRound);
    __syncthreads();
    float part[kRowsCols][MR];
#pragma unroll
    for (int c = 0; c < kRowsCols; ++c)
#pragma unroll
      for (int m = 0; m < MR; ++m) part[c][m] = 0.f;
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
      if (groups == 64) {
        // all 64 sums are asked for before the first is added (a loop would wait for LDS 64 times in a row)
        float sums[64];
#pragma unroll
        for (int g = 0; g < 64; ++g) sums[g] = mine[g];
#pragma unroll
        for (int g = 0; g < 64; ++g) acc += sums[g];
      } else {
        for (int g = 0; g < groups; ++g) acc += mine[g];
      }
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
    const bool vec = K % 4 == 0 && lda % 4 == 0 && ldw % 4 == 0 && ((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0;
#define TL_ROWS_LAUNCH(MR)                                                                               \
  do {                                                                                                   \
    const size_t region = (size_t)kRowsCols * MR * kPad > (size_t)kTurned ? (size_t)kRowsCols * MR * kPad : (size_t)kTurned; \
    const size_t lds = ((size_t)MR * BK * kPad + (size_t)kRowsWaves * region) * sizeof(float);               \
    if (lds > 48 * 1024) {                                                                               \
      hipError_t e = hipFuncSetAttribute(vec ? (const void*)gemm_f32_rows_kernel<MR, true>               \
                                             : (const void*)gemm_f32_rows_kernel<MR, false>,             \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);          \
      if (e != hipSuccess) return tl_fail(TL_ERR_HIP, "gemm_f32: %s", hipGetErrorString(e));             \
    }                                                                                                    \
    if (vec)                                                                                             \
      gemm_f32_rows_kernel<MR, true><<<blocks, kRowsWaves * kWave, lds, stream>>>(A, lda, W, ldw, C, ldc, M, N, K); \
    else                                                                                                 \
      gemm_f32_rows_kernel<MR, false><<<blocks, kRowsWaves * kWave, lds, stream>>>(A, lda, W, ldw, C, ldc, M, N, K); \
  } while (0)
    if (M == 1) TL_ROWS_LAUNCH(1);
    else if (M == 2) TL_ROWS_LAUNCH(2);
    else if (M <= 4) TL_ROWS_LAUNCH(4);
    else if (M <= 8) TL_ROWS_LAUNCH(8);
    else TL_ROWS_LAUNCH(16);
#undef TL_ROWS_LAUNCH
    return tl_check_launch("gemm_f32_rows");
  }
  // prompts take the large tile, if that still makes a block for every CU (both give the same sums)
  if (M > 96 && (size_t)((M + 127) / 128) * ((N + 127) / 128) >= 256) {
    const unsigned gy = (N + 127) / 128;
    TL_REQUIRE(gy <= 65535, "gemm_f32: N=%d exceeds the grid limit of one launch", N);
    gemm_f32_kernel<128, 128, 8, 8><<<dim3((M + 127) / 128, gy), 256, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K);
  } else {
    const unsigned gy = (N + 63) / 64;
    TL_REQUIRE(gy <= 65535, "gemm_f32: N=%d exceeds the grid limit of one launch", N);
    gemm_f32_kernel<64, 64, 4, 4><<<dim3((M + 63) / 64, gy), 256, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K);
  }
  return tl_check_launch("gemm_f32");
}
