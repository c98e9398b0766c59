// C[M, N] = A[M, K] * W[N, K]^T for 17 to 128 rows, bfloat16 inputs, 32-bit accumulation: the matrix
// products of decode steps with many requests.  Their cost is still reading W once from HBM, but
// the rows of A are now a quarter of a megabyte and more, so the blocks must share what they read
// of A instead of each wave fetching it for its own strip of columns.
//
//   * a block of four waves owns 64 * NCW rows of W (output columns); wave w owns the strips of 16
//     rows w * NCW .. w * NCW + NCW - 1 of them.  K is walked in steps of 128.  The step's slice of
//     A (all rows x 128) is fetched once per block into LDS, every wave a quarter of it, and read as
//     operands by all four; the slices of W go to a piece of LDS of the wave's own.
//   * everything is fetched by `global_load_lds` (a wave's instruction puts 4 rows x 256 contiguous
//     bytes, the coalesced shape, straight into 1 KB of LDS without passing through registers) into
//     one of two or three buffers: the loads of the next steps are in flight while one step is
//     multiplied.
//   * LDS rows are 256 bytes, one after the other.  The 16 lanes that read the same 16-byte piece
//     of 16 different rows would all fall on the same banks, so piece p of row r lies at slot
//     p ^ (r % 16): the fetch asks every lane for the piece that belongs into its slot.
//   * C^T[16 columns x 16 rows] by MFMA 16x16x32 bf16 (A operand = W, B operand = rows of A).
//   * grid (column blocks, splits of K).  Products with few columns (4,096 of them are 64 blocks)
//     are split along K over several blocks, whose 32-bit partial sums a second kernel adds in a
//     fixed order; for the query/key/value projection that second kernel also rotates the heads
//     and writes keys and values into their pages.
//   * gated variant (GLU): W = gate rows | up rows.  Waves 0 and 1 take gate strips, waves 2 and 3
//     the up strips of the same columns; at the end the up halves pass through LDS and the gate
//     waves store silu(gate) * up with the roundings of the unfused sequence.
#include "common.h"
#include "qkv_epilogue.h"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kWaves = 4;
constexpr int kStepK = 128;            // k per step: 16 pieces of 8 elements
constexpr int kRowElems = kStepK;      // an LDS row holds one step of one row
constexpr int kStripElems = 16 * kRowElems;

// 64 lanes x 16 bytes from `src` (per lane) to LDS at byte offset `lds_at` (wave-uniform) + 16 * lane.
// Written as assembly, not as the compiler's builtin: the compiler knows that the builtin writes LDS
// and, unable to tell the buffers apart, waits for every outstanding load before the first LDS read
// that follows, which would leave no load in flight during the multiplication.  The kernel counts
// its loads itself (s_waitcnt vmcnt) and has no other vector memory loads.
__device__ __forceinline__ void load_to_lds(const bf16_t* src, uint32_t lds_at) {
  asm volatile(
      "s_mov_b32 m0, %1\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %0, off"
      :
      : "v"(src), "s"(lds_at)
      : "m0", "memory");
}

// MC: chunks of 16 rows of A (M <= 16 MC).  NCW: strips of 16 columns per wave.
// STAGES: buffers; the loads of STAGES - 1 steps are in flight while one step is multiplied.
template <int MC, int NCW, int STAGES>
struct Shape {
  static constexpr int kATile = MC * kStripElems;
  static constexpr int kStage = kATile + kWaves * NCW * kStripElems;  // elements of one buffer
  static constexpr int kLdsBytes = STAGES * kStage * (int)sizeof(bf16_t);
  static constexpr int kBlockRows = kWaves * NCW * 16;  // rows of W per block
  static constexpr int kLoads = MC + 4 * NCW;  // load instructions of a wave per step
  // s_waitcnt that lets the loads of the STAGES - 2 latest steps stay outstanding (gfx9 encoding:
  // vmcnt in bits 3:0 and 15:14, the other counters left at their maxima)
  static constexpr int kPending = (STAGES - 2) * kLoads;
  static_assert(kPending < 64, "vmcnt has six bits");
  static constexpr int kWaitOldest = (kPending & 0xF) | (0x7 << 4) | (0xF << 8) | ((kPending >> 4) << 14);
};

// GATED: W holds 2 N rows, gate rows then up rows; C[M, N] = silu(A gate^T) * (A up^T), bfloat16.
template <int MC, int NCW, int STAGES, typename OutT, bool GATED>
__global__ void __launch_bounds__(kWaves* kWave)
gemm_wide_kernel(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, int ldw, OutT* __restrict__ C,
                 int ldc, float* __restrict__ partial, int M, int N, int K, int steps_per_split) {
  using S = Shape<MC, NCW, STAGES>;
  extern __shared__ __attribute__((aligned(16))) bf16_t lds[];
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int n16 = lane % 16;  // operand layout: row
  const int g4 = lane / 16;   // operand layout: piece within a group of four
  const int q = lane / 16;    // fetch layout: row within a group of four
  const int slot = lane % 16; // fetch layout: 16-byte slot of the LDS row
  // first output column of the wave's strips
  const int half = GATED ? wave / 2 : 0;  // gated: 0 = gate rows, 1 = up rows
  const int n0 = GATED ? blockIdx.x * (S::kBlockRows / 2) + (wave % 2) * NCW * 16 : blockIdx.x * S::kBlockRows + wave * NCW * 16;

  const int steps_total = K / kStepK;
  const int step_lo = blockIdx.y * steps_per_split;
  const int nst = min(steps_per_split, steps_total - step_lo);

  // what this lane fetches: MC loads of A (rows 4 (wave MC + j) + q) and 4 NCW loads of W; rows of
  // W past N are clamped and rows of A past M read row 0: neither result is stored
  const bf16_t* asrc[MC];
#pragma unroll
  for (int j = 0; j < MC; ++j) {
    const int r = 4 * (wave * MC + j) + q;
    asrc[j] = A + (size_t)(r < M ? r : 0) * lda + 8 * (slot ^ (r & 15));
  }
  const bf16_t* wsrc[4 * NCW];
#pragma unroll
  for (int j = 0; j < 4 * NCW; ++j) {
    const int r = 4 * j + q;  // row within the wave's NCW strips
    wsrc[j] = W + (size_t)(half * N + min(n0 + r, N - 1)) * ldw + 8 * (slot ^ (r & 15));
  }
  // byte offsets within the block's LDS of what this wave fills: its quarter of the A tile, its W strips
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;  // low half of the address = offset within LDS
  const uint32_t a_at = __builtin_amdgcn_readfirstlane(lds_base + 4 * wave * MC * kRowElems * (int)sizeof(bf16_t));
  const uint32_t w_at = __builtin_amdgcn_readfirstlane(lds_base + (S::kATile + wave * NCW * kStripElems) * (int)sizeof(bf16_t));
  auto issue = [&](int step, int buffer) {
    const uint32_t stage = buffer * S::kStage * (int)sizeof(bf16_t);
    const int k0 = step * kStepK;
#pragma unroll
    for (int j = 0; j < MC; ++j) load_to_lds(asrc[j] + k0, a_at + stage + 4 * j * kRowElems * (int)sizeof(bf16_t));
#pragma unroll
    for (int j = 0; j < 4 * NCW; ++j) load_to_lds(wsrc[j] + k0, w_at + stage + 4 * j * kRowElems * (int)sizeof(bf16_t));
  };

  float4_t acc[NCW][MC];
#pragma unroll
  for (int t = 0; t < NCW; ++t)
#pragma unroll
    for (int c = 0; c < MC; ++c) acc[t][c] = float4_t{0.f, 0.f, 0.f, 0.f};

  // Rows of W lie a power of two apart, so blocks that walk K in step would all press on the same
  // memory channels at once: every block starts its walk at a different step and wraps around.
  const int rot = (int)((blockIdx.x * 5u + blockIdx.y * 3u) % (unsigned)nst);
  auto step_of = [&](int i) {
    int s = i + rot;
    if (s >= nst) s -= nst;
    return step_lo + s;
  };

  // all loads are unconditional (past the end the last step is fetched again and never used): a
  // wave's count of outstanding loads must be the same in every trip, and a load under a branch
  // would make a wait cover both paths
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s) issue(step_of(min(s, nst - 1)), s);
  int buffer = 0;
  for (int i = 0; i < nst; ++i) {
    // this wave's loads of step i have landed (loads complete in order); after the barrier
    // everybody's have, and everybody has finished reading the buffer of step i - 1, which the
    // next loads overwrite
    __builtin_amdgcn_s_waitcnt(S::kWaitOldest);
    __syncthreads();
    const int refill = buffer == 0 ? STAGES - 1 : buffer - 1;
    issue(step_of(min(i + STAGES - 1, nst - 1)), refill);
    const bf16_t* stage = lds + buffer * S::kStage;
    buffer = buffer + 1 == STAGES ? 0 : buffer + 1;
    const bf16_t* mine = stage + S::kATile + wave * NCW * kStripElems;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int at = n16 * kRowElems + 8 * ((4 * u + g4) ^ n16);
      bf16x8_t wop[NCW], aop[MC];
#pragma unroll
      for (int t = 0; t < NCW; ++t) wop[t] = *reinterpret_cast<const bf16x8_t*>(mine + t * kStripElems + at);
#pragma unroll
      for (int c = 0; c < MC; ++c) aop[c] = *reinterpret_cast<const bf16x8_t*>(stage + c * kStripElems + at);
#pragma unroll
      for (int t = 0; t < NCW; ++t)
#pragma unroll
        for (int c = 0; c < MC; ++c) acc[t][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wop[t], aop[c], acc[t][c], 0, 0, 0);
    }
  }
  __builtin_amdgcn_s_waitcnt(0);  // the last, unused fetch must not land after the block has gone

  // acc[t][c][i] = C[16 c + n16][n0 + 16 t + 4 g4 + i]
  if constexpr (GATED) {
    // every wave has waited for its loads; after the barrier nobody reads or fills the buffers,
    // and the up waves hand their sums over through them
    float4_t* exchange = reinterpret_cast<float4_t*>(lds);
    __syncthreads();
    if (half == 1) {
#pragma unroll
      for (int t = 0; t < NCW; ++t)
#pragma unroll
        for (int c = 0; c < MC; ++c) exchange[(((wave % 2) * NCW + t) * MC + c) * kWave + lane] = acc[t][c];
    }
    __syncthreads();
    if (half == 1) return;
#pragma unroll
    for (int t = 0; t < NCW; ++t)
#pragma unroll
      for (int c = 0; c < MC; ++c) {
        const int m = 16 * c + n16;
        const int n = n0 + 16 * t + 4 * g4;
        if (m >= M) continue;
        const float4_t up = exchange[(((wave % 2) * NCW + t) * MC + c) * kWave + lane];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (n + i >= N) continue;
          const float g = to_f32(from_f32<OutT>(acc[t][c][i]));
          const float u = to_f32(from_f32<OutT>(up[i]));
          const float act = to_f32(from_f32<OutT>(g / (1.0f + expf(-g))));
          C[(size_t)m * ldc + n + i] = from_f32<OutT>(act * u);
        }
      }
  } else {
#pragma unroll
    for (int t = 0; t < NCW; ++t)
#pragma unroll
      for (int c = 0; c < MC; ++c) {
        const int m = 16 * c + n16;
        const int n = n0 + 16 * t + 4 * g4;
        if (m >= M || n >= N) continue;
        if (partial != nullptr) {
          float* dst = partial + ((size_t)blockIdx.y * M + m) * N + n;
          if (n + 4 <= N && (N % 4) == 0) {
            *reinterpret_cast<float4_t*>(dst) = acc[t][c];
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (n + i < N) dst[i] = acc[t][c][i];
          }
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < N) C[(size_t)m * ldc + n + i] = from_f32<OutT>(acc[t][c][i]);
        }
      }
  }
}

// C[m][n] = sum over the splits, in their order, of partial[s][m][n].  These kernels run between two
// large ones and every load of theirs misses the caches: the splits are asked for several at a time
// (a split past the last is the last once more, and not added), not one after the other.
constexpr int kReduceAhead = 8;

template <typename OutT>
__global__ void __launch_bounds__(256) gemm_wide_reduce_kernel(const float* __restrict__ partial, OutT* __restrict__ C,
                                                               int ldc, int M, int N, int splits) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t total = (size_t)M * N;
  if (idx >= total) return;
  float sum = 0.f;
  for (int s = 0; s < splits; s += kReduceAhead) {
    float part[kReduceAhead];
#pragma unroll
    for (int u = 0; u < kReduceAhead; ++u) part[u] = partial[(size_t)min(s + u, splits - 1) * total + idx];
#pragma unroll
    for (int u = 0; u < kReduceAhead; ++u) sum = s + u < splits ? sum + part[u] : sum;
  }
  C[(idx / N) * ldc + idx % N] = from_f32<OutT>(sum);
}

// The same for the query/key/value projection: a thread sums four neighbouring columns (two
// rotary pairs of one head) and finishes them.
__global__ void __launch_bounds__(256) gemm_wide_reduce_qkv_kernel(const float* __restrict__ partial, bf16_t* __restrict__ C,
                                                                   int ldc, int M, int N, int splits, QkvArgs qa) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // over M * N / 4
  const int quads = N / 4;
  if (idx >= (size_t)M * quads) return;
  const int m = (int)(idx / quads);
  const int n = 4 * (int)(idx % quads);
  const size_t total = (size_t)M * N;
  const float* mine = partial + (size_t)m * N + n;
  const QkvOperands operands = qkv_fetch(m, n, qa);
  float4_t sum = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < splits; s += kReduceAhead) {
    float4_t part[kReduceAhead];
#pragma unroll
    for (int u = 0; u < kReduceAhead; ++u) part[u] = *reinterpret_cast<const float4_t*>(mine + (size_t)min(s + u, splits - 1) * total);
#pragma unroll
    for (int u = 0; u < kReduceAhead; ++u) sum = s + u < splits ? sum + part[u] : sum;
  }
  const float sums[4] = {sum[0], sum[1], sum[2], sum[3]};
  qkv_finish(sums, m, n, qa, C, ldc, operands);
}

struct Launch {
  const bf16_t* A; int lda;
  const bf16_t* W; int ldw;
  void* C; int ldc;
  float* partial;
  int M, N, K;
  int out_dtype;
  int splits;          // blocks along K
  bool reduce;         // false: the splits' sums stay in `partial` (always written then) and C is not touched
  bool gated;
  const QkvArgs* qkv;  // non-null: the split product ends in the query/key/value epilogue
  hipStream_t stream;
};

template <int MC, int NCW, int STAGES, typename OutT, bool GATED>
int launch_kernel(const Launch& l) {
  using S = Shape<MC, NCW, STAGES>;
  static bool raised = false;  // blocks past 64 KB of LDS have to be allowed once per kernel
  if (S::kLdsBytes > 64 * 1024 && !raised) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_wide_kernel<MC, NCW, STAGES, OutT, GATED>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, S::kLdsBytes);
    if (e != hipSuccess) return tl_fail(TL_ERR_HIP, "gemm_wide: cannot reserve %d bytes of LDS: %s", S::kLdsBytes, hipGetErrorString(e));
    raised = true;
  }
  const int steps_total = l.K / kStepK;
  const int steps_per_split = (steps_total + l.splits - 1) / l.splits;
  const int used = (steps_total + steps_per_split - 1) / steps_per_split;  // no split is empty
  // the query/key/value epilogue lives in the second kernel; a caller that adds the splits itself gets
  // them even when there is only one
  const bool split = used > 1 || l.qkv != nullptr || !l.reduce;
  const int block_cols = GATED ? S::kBlockRows / 2 : S::kBlockRows;
  const dim3 grid((l.N + block_cols - 1) / block_cols, used);
  gemm_wide_kernel<MC, NCW, STAGES, OutT, GATED><<<grid, kWaves * kWave, S::kLdsBytes, l.stream>>>(
      l.A, l.lda, l.W, l.ldw, (OutT*)l.C, l.ldc, split ? l.partial : nullptr, l.M, l.N, l.K, steps_per_split);
  int rc = tl_check_launch("gemm_wide");
  if (rc != TL_OK || !split || !l.reduce) return rc;
  if (l.qkv != nullptr) {
    const size_t quads = (size_t)l.M * (l.N / 4);
    gemm_wide_reduce_qkv_kernel<<<(unsigned)((quads + 255) / 256), 256, 0, l.stream>>>(l.partial, (bf16_t*)l.C, l.ldc, l.M,
                                                                                       l.N, used, *l.qkv);
  } else {
    const size_t total = (size_t)l.M * l.N;
    gemm_wide_reduce_kernel<OutT><<<(unsigned)((total + 255) / 256), 256, 0, l.stream>>>(l.partial, (OutT*)l.C, l.ldc, l.M, l.N, used);
  }
  return tl_check_launch("gemm_wide_reduce");
}

template <int MC, int NCW, int STAGES>
int launch_stages(const Launch& l) {
  if constexpr (Shape<MC, NCW, STAGES>::kLdsBytes > 160 * 1024) {  // (more than gfx950 has: not compiled at all)
    return tl_fail(TL_ERR_UNSUPPORTED, "gemm_wide: %d buffers for %d rows and %d strips per wave do not fit into LDS", STAGES, 16 * MC, NCW);
  } else {
    if (Shape<MC, NCW, STAGES>::kLdsBytes > tl_device_facts().lds_bytes)
      return tl_fail(TL_ERR_UNSUPPORTED, "gemm_wide: %d buffers for %d rows and %d strips per wave take %d bytes of LDS, this device has %d",
                     STAGES, 16 * MC, NCW, (int)Shape<MC, NCW, STAGES>::kLdsBytes, tl_device_facts().lds_bytes);
    if (l.gated) return launch_kernel<MC, NCW, STAGES, bf16_t, true>(l);
    if (l.out_dtype == TL_BF16) return launch_kernel<MC, NCW, STAGES, bf16_t, false>(l);
    return launch_kernel<MC, NCW, STAGES, float, false>(l);
  }
}

template <int MC>
int launch_rows(int ncw, int stages, const Launch& l) {
  if (ncw == 1) return stages == 2 ? launch_stages<MC, 1, 2>(l) : launch_stages<MC, 1, 3>(l);
  return stages == 2 ? launch_stages<MC, 2, 2>(l) : launch_stages<MC, 2, 3>(l);
}

int run(Launch l, int strips_per_wave, int stages) {
  TL_REQUIRE(l.M >= 0 && l.N > 0 && l.K > 0, "gemm_wide: bad sizes M=%d N=%d K=%d", l.M, l.N, l.K);
  if (l.M > 128) return tl_fail(TL_ERR_UNSUPPORTED, "gemm_wide: M=%d exceeds 128", l.M);
  if (l.K % kStepK) return tl_fail(TL_ERR_UNSUPPORTED, "gemm_wide: K=%d is not a multiple of %d", l.K, kStepK);
  TL_REQUIRE(l.lda >= l.K && l.ldw >= l.K && l.ldc >= l.N, "gemm_wide: leading dimensions too small");
  TL_REQUIRE(l.lda % 8 == 0 && l.ldw % 8 == 0 && ((uintptr_t)l.A % 16) == 0 && ((uintptr_t)l.W % 16) == 0,
             "gemm_wide: rows must start on 16-byte boundaries");
  TL_REQUIRE(l.out_dtype == TL_BF16 || l.out_dtype == TL_F32, "gemm_wide: out_dtype must be 0 or 1");
  TL_REQUIRE(strips_per_wave == 1 || strips_per_wave == 2, "gemm_wide: strips_per_wave must be 1 or 2");
  TL_REQUIRE(l.splits >= 1 && l.splits <= 64, "gemm_wide: k_splits must be 1..64");
  TL_REQUIRE(stages == 2 || stages == 3, "gemm_wide: stages must be 2 or 3");
  const bool needs_partial = l.splits > 1 || l.qkv != nullptr || !l.reduce;
  TL_REQUIRE(!needs_partial || (l.partial != nullptr && ((uintptr_t)l.partial % 16) == 0),
             "gemm_wide: a split product needs the 16-byte aligned partial buffer");
  if (l.M == 0) return TL_OK;
  if (l.M <= 32) return launch_rows<2>(strips_per_wave, stages, l);
  if (l.M <= 64) return launch_rows<4>(strips_per_wave, stages, l);
  return launch_rows<8>(strips_per_wave, stages, l);
}

}  // namespace

// A [M, K] and W [N, K] bfloat16, row-major with leading dimensions lda / ldw (multiples of 8, bases
// 16-byte aligned); C [M, N] bfloat16 (out_dtype 1) or 32-bit (out_dtype 0).  M <= 128, K a multiple
// of 128.  strips_per_wave: 1 or 2 (a block owns 64 or 128 columns).  k_splits >= 1: blocks along
// K; with more than one, `partial` must hold k_splits * M * N floats.  stages: 2 or 3 buffers of LDS
// (a buffer is 4 KB for every 16 rows of A, 32, 64 or 128 of them, plus 16 KB for every strip per
// wave; three buffers of 128 rows and two strips do not fit the 160 KB and are refused).
// reduce = 0: the second kernel is left out; `partial` then holds tl_gemm_wide_splits(K, k_splits)
// slices [M, N] for the caller to add (in their order, for the same result), and C is not touched.
TL_EXPORT int tl_gemm_wide(const void* A, int lda, const void* W, int ldw, void* C, int ldc, int M, int N, int K,
                           int out_dtype, int strips_per_wave, int k_splits, int stages, int reduce, void* partial,
                           hipStream_t stream) {
  Launch l{(const bf16_t*)A, lda, (const bf16_t*)W, ldw, C, ldc, (float*)partial, M, N, K, out_dtype, k_splits, reduce != 0, false, nullptr, stream};
  return run(l, strips_per_wave, stages);
}

// How many splits a product over K with `k_splits` asked for really has (no split is empty).
TL_EXPORT int tl_gemm_wide_splits(int K, int k_splits) {
  if (K <= 0 || k_splits <= 0) return 0;
  const int steps_total = K / kStepK;
  const int steps_per_split = (steps_total + k_splits - 1) / k_splits;
  return steps_per_split > 0 ? (steps_total + steps_per_split - 1) / steps_per_split : 0;
}

// C [M, N] (bfloat16 or 32-bit) = the sum of `splits` slices [M, N] of `partial`, added in their order.
TL_EXPORT int tl_gemm_wide_reduce(const void* partial, void* C, int ldc, int M, int N, int splits, int out_dtype,
                                  hipStream_t stream) {
  TL_REQUIRE(M >= 0 && N > 0 && splits >= 1 && ldc >= N, "gemm_wide_reduce: bad sizes M=%d N=%d splits=%d", M, N, splits);
  TL_REQUIRE(out_dtype == TL_BF16 || out_dtype == TL_F32, "gemm_wide_reduce: out_dtype must be 0 or 1");
  if (M == 0) return TL_OK;
  const size_t total = (size_t)M * N;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (out_dtype == TL_BF16)
    gemm_wide_reduce_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const float*)partial, (bf16_t*)C, ldc, M, N, splits);
  else
    gemm_wide_reduce_kernel<float><<<blocks, 256, 0, stream>>>((const float*)partial, (float*)C, ldc, M, N, splits);
  return tl_check_launch("gemm_wide_reduce");
}

// The gated pair of products: W [2 N, K] = gate rows | up rows; C [M, N] bfloat16 =
// silu(A gate^T) * (A up^T), rounded as the two products, the activation and the final product
// would be if each were stored in bfloat16.  A block owns 32 or 64 columns (strips_per_wave 1 or 2).
TL_EXPORT int tl_gemm_wide_glu(const void* A, int lda, const void* W, int ldw, void* C, int ldc, int M, int N, int K,
                               int strips_per_wave, int stages, hipStream_t stream) {
  Launch l{(const bf16_t*)A, lda, (const bf16_t*)W, ldw, C, ldc, nullptr, M, N, K, TL_BF16, 1, true, true, nullptr, stream};
  return run(l, strips_per_wave, stages);
}

// The query/key/value projection, split along K, with the rotary kernel's work in the kernel that
// adds the splits.  W [(Hq + 2 Hkv) * head_dim, K]; C [M, that width] receives the rotated queries
// (and keys and values when no pages are given).  cos_sin [M][rotary_dim / 2][2]: cosine and sine of
// each row's position (interleaved pairs only).  k_pages / v_pages [page][Hkv][page_size][head_dim];
// slot_mapping [M].  head_dim % 4 == 0.  `partial` holds k_splits * M * width floats (also for one split).
TL_EXPORT int tl_gemm_wide_qkv(const void* A, int lda, const void* W, int ldw, void* C, int ldc, int M, int K,
                               int n_q_heads, int n_kv_heads, int head_dim, int rotary_dim, const float* cos_sin,
                               void* k_pages, void* v_pages, const int32_t* slot_mapping, int page_size,
                               int strips_per_wave, int k_splits, int stages, void* partial, hipStream_t stream) {
  QkvArgs qa;
  const int rc = qkv_args("gemm_wide_qkv", n_q_heads, n_kv_heads, head_dim, rotary_dim, cos_sin, k_pages, v_pages,
                          slot_mapping, page_size, C, ldc, &qa);
  if (rc != TL_OK) return rc;
  const int N = (n_q_heads + 2 * n_kv_heads) * head_dim;
  Launch l{(const bf16_t*)A, lda, (const bf16_t*)W, ldw, C, ldc, (float*)partial, M, N, K, TL_BF16, k_splits, true, false, &qa, stream};
  return run(l, strips_per_wave, stages);
}
