// C[M, N] = A[M, K] * W[N, K]^T for few rows (M <= 64), bfloat16 inputs, 32-bit accumulation:
// the matrix products of decode steps, whose cost is reading W once from HBM.
//
//   * a block owns a strip of 16 output columns (16 rows of W); its waves split K between them and
//     add their partial sums through LDS in a fixed order (no atomics).
//   * C^T[16 columns x 16 rows of A] by MFMA 16x16x16 bf16: the A operand is W exactly as it lies in
//     memory (a lane loads 64 contiguous bytes of its row per step, four lanes cover 256 bytes), the B
//     operand is A, read through the cache with the same addressing.  M > 16 takes up to four MFMA
//     column blocks that reuse each W load.
//   * the result leaves as bfloat16 or as 32-bit (logits).
#include "common.h"

namespace {

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

union Pack16 {
  uint4 u;
  u32x4_t v;
  short4_t s[2];
};

constexpr int kStrip = 16;   // output columns per block
constexpr int kStepK = 128;  // k covered by one wave step: 4 lane groups x 32 contiguous elements

// MB: MFMA column blocks (M <= 16 * MB).  WAVES: waves per block = splits of K.
template <int MB, int WAVES, typename OutT>
__global__ void __launch_bounds__(WAVES* kWave)
gemm_skinny_kernel(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, int ldw,
                   OutT* __restrict__ C, int ldc, int M, int N, int K) {
  __shared__ float red[WAVES][MB][kWave][4];
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int n16 = lane % 16;
  const int g4 = lane / 16;
  const int n0 = blockIdx.x * kStrip;

  // K is walked in steps of 128; the waves of the block share the whole steps between them and the
  // last wave also takes the partial step at the end, if there is one
  const int steps_full = K / kStepK;
  const int steps_per_wave = (steps_full + WAVES - 1) / WAVES;
  const int step_lo = min(wave * steps_per_wave, steps_full);
  const int step_hi = min(step_lo + steps_per_wave, steps_full);

  const int wrow = min(n0 + n16, N - 1);  // rows past N are clamped; their results are not stored
  const bf16_t* wp = W + (size_t)wrow * ldw + 32 * g4;
  // rows of A past M are read from row 0: they only feed output columns that are never stored
  const bf16_t* ap[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    const int m = 16 * b + n16;
    ap[b] = A + (size_t)(m < M ? m : 0) * lda + 32 * g4;
  }

  float4_t acc[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) acc[b] = float4_t{0.f, 0.f, 0.f, 0.f};

  // whole steps: plain loads, nothing between a load and its use but the other stage's MFMAs
  auto load = [&](int st, Pack16* w, Pack16 (*a)[4]) {
    const int k0 = st * kStepK;
#pragma unroll
    for (int u = 0; u < 4; ++u) w[u].v = *reinterpret_cast<const u32x4_t*>(wp + k0 + 8 * u);
#pragma unroll
    for (int b = 0; b < MB; ++b)
#pragma unroll
      for (int u = 0; u < 4; ++u) a[b][u].v = *reinterpret_cast<const u32x4_t*>(ap[b] + k0 + 8 * u);
  };
  auto mma = [&](const Pack16* w, const Pack16 (*a)[4]) {
#pragma unroll
    for (int b = 0; b < MB; ++b) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(w[u].s[0], a[b][u].s[0], acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(w[u].s[1], a[b][u].s[1], acc[b], 0, 0, 0);
      }
    }
  };
  Pack16 w0[4], w1[4];
  Pack16 a0[MB][4], a1[MB][4];
  // Rows of W lie a power of two apart, so blocks that walk K in step would all press on the same
  // memory channels at once; every block therefore starts its walk at a different step and wraps
  // around.  Two steps per trip so that both buffers are named statically (they stay in registers).
  const int nst = step_hi - step_lo;
  const int rot = nst > 0 ? (int)((blockIdx.x * 5u + wave * 3u) % (unsigned)nst) : 0;
  auto step_of = [&](int i) {
    int s = i + rot;
    if (s >= nst) s -= nst;
    return step_lo + s;
  };
  // The prefetches are unconditional (past the end they repeat the last step and are ignored): a
  // load under a branch would make the wait before the MFMAs cover both paths, that is, wait for
  // the prefetch itself.
  if (nst > 0) {
    load(step_of(0), w0, a0);
    int i = 0;
    for (; i + 1 < nst; i += 2) {  // two steps per trip, nothing conditional inside
      load(step_of(i + 1), w1, a1);
      mma(w0, a0);
      load(step_of(min(i + 2, nst - 1)), w0, a0);
      mma(w1, a1);
    }
    if (i < nst) mma(w0, a0);  // an odd number of steps: the last one is already loaded
  }
  // the partial step: addresses past K are clamped into the row and the A side is zeroed, so the
  // out-of-range products vanish
  if (wave == WAVES - 1 && steps_full * kStepK < K) {
    const int kmax = K - 8;
    const int k0 = steps_full * kStepK + 32 * g4;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = k0 + 8 * u;
      w0[u].v = *reinterpret_cast<const u32x4_t*>(wp - 32 * g4 + min(k, kmax));
      const uint32_t keep = k < K ? 0xFFFFFFFFu : 0u;
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(ap[b] - 32 * g4 + min(k, kmax));
        a0[b][u].v = u32x4_t{v[0] & keep, v[1] & keep, v[2] & keep, v[3] & keep};
      }
    }
    mma(w0, a0);
  }

  // acc[b][i] = C^T[n0 + 4 g4 + i][16 b + n16]; add the waves' shares in wave order
  if (WAVES > 1) {
#pragma unroll
    for (int b = 0; b < MB; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][b][lane][i] = acc[b][i];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int b = 0; b < MB; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float s = red[0][b][lane][i];
#pragma unroll
        for (int w2 = 1; w2 < WAVES; ++w2) s += red[w2][b][lane][i];
        acc[b][i] = s;
      }
  }
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    const int m = 16 * b + n16;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + 4 * g4 + i;
      if (n < N) C[(size_t)m * ldc + n] = from_f32<OutT>(acc[b][i]);
    }
  }
}

template <int MB, int WAVES>
int launch(const bf16_t* A, int lda, const bf16_t* W, int ldw, void* C, int ldc, int M, int N, int K,
           int out_dtype, hipStream_t stream) {
  const dim3 grid((N + kStrip - 1) / kStrip);
  if (out_dtype == TL_BF16)
    gemm_skinny_kernel<MB, WAVES, bf16_t><<<grid, WAVES * kWave, 0, stream>>>(A, lda, W, ldw, (bf16_t*)C, ldc, M, N, K);
  else
    gemm_skinny_kernel<MB, WAVES, float><<<grid, WAVES * kWave, 0, stream>>>(A, lda, W, ldw, (float*)C, ldc, M, N, K);
  return tl_check_launch("gemm_skinny");
}

template <int MB>
int launch_waves(int waves, const bf16_t* A, int lda, const bf16_t* W, int ldw, void* C, int ldc, int M, int N,
                 int K, int out_dtype, hipStream_t stream) {
  switch (waves) {
    case 1: return launch<MB, 1>(A, lda, W, ldw, C, ldc, M, N, K, out_dtype, stream);
    case 2: return launch<MB, 2>(A, lda, W, ldw, C, ldc, M, N, K, out_dtype, stream);
    case 4: return launch<MB, 4>(A, lda, W, ldw, C, ldc, M, N, K, out_dtype, stream);
    default: return launch<MB, 8>(A, lda, W, ldw, C, ldc, M, N, K, out_dtype, stream);
  }
}

}  // namespace

// A [M, K] and W [N, K] bfloat16, row-major with leading dimensions lda / ldw (multiples of 8, bases
// 16-byte aligned); C [M, N] bfloat16 (out_dtype 1) or 32-bit (out_dtype 0).  M <= 64, K a multiple of 8.
// waves = 0 picks the number of K splits from the sizes.
TL_EXPORT int tl_gemm_skinny(const void* A, int lda, const void* W, int ldw, void* C, int ldc, int M, int N,
                             int K, int out_dtype, int waves, hipStream_t stream) {
  TL_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_skinny: bad sizes M=%d N=%d K=%d", M, N, K);
  if (M > 64) return tl_fail(TL_ERR_UNSUPPORTED, "gemm_skinny: M=%d exceeds 64", M);
  if (K % 8) return tl_fail(TL_ERR_UNSUPPORTED, "gemm_skinny: K=%d is not a multiple of 8", K);
  TL_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_skinny: leading dimensions too small");
  TL_REQUIRE(lda % 8 == 0 && ldw % 8 == 0 && ((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0,
             "gemm_skinny: rows must start on 16-byte boundaries");
  TL_REQUIRE(out_dtype == TL_BF16 || out_dtype == TL_F32, "gemm_skinny: out_dtype must be 0 or 1");
  if (M == 0) return TL_OK;
  if (waves == 0) {
    // enough waves to keep loads in flight on 256 CUs: about 4096 in all, at least one step each
    const int strips = (N + kStrip - 1) / kStrip;
    const int steps = (K + kStepK - 1) / kStepK;
    waves = 1;
    while (waves < 8 && strips * waves < 4096 && steps >= 2 * waves * 2) waves *= 2;
  }
  TL_REQUIRE(waves == 1 || waves == 2 || waves == 4 || waves == 8, "gemm_skinny: waves must be 1, 2, 4 or 8");
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  if (M <= 16) return launch_waves<1>(waves, a, lda, w, ldw, C, ldc, M, N, K, out_dtype, stream);
  if (M <= 32) return launch_waves<2>(waves, a, lda, w, ldw, C, ldc, M, N, K, out_dtype, stream);
  return launch_waves<4>(waves, a, lda, w, ldw, C, ldc, M, N, K, out_dtype, stream);
}
