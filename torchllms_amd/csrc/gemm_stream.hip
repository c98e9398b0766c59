// C[M, N] = A[M, K] * W[N, K]^T for up to 16 rows, bfloat16 inputs, 32-bit accumulation: the matrix
// products of decode steps, whose cost is reading W once from HBM.
//
// The vector memory path is bound by the cache lines an instruction touches, not by its bytes, so
// W is fetched the coalesced way: one load instruction takes 4 rows x 256 contiguous bytes (8 cache
// lines per KB; a load in the MFMA operand's own layout, 16 rows x 64 bytes, touches twice as many).
// The MFMA wants the other layout (lane = row), so every wave passes its tile through a private
// piece of LDS: written as loaded, read back as operands.  A wave's LDS instructions run in order,
// so no barrier is needed, only fences that keep the compiler from reordering them.
//
//   * a block owns a strip of 16 output columns (16 rows of W); its waves split K between them and
//     add their partial sums through LDS in a fixed order (no atomics).
//   * C^T[16 columns x 16 rows of A] by MFMA 16x16x16 bf16: A operand = W, B operand = the rows of A,
//     fetched and transposed the same way (only as many groups of four rows as M needs).
//   * the LDS rows are 272 bytes apart: the 16 lanes that read one 16-byte piece of 16 different
//     rows then fall on different banks.
//   * gated variant (GLU), in two shapes.  Half: the block's 16 rows of W are 8 gate rows and the 8 up
//     rows of the same columns, so the launch looks like the plain product's (as many blocks, each
//     fetching as much) and costs the same; the lanes that hold gate sums fetch the up sums from the
//     lanes 32 further on.  With 16 rows of A, whose fetch every block repeats, twice as many blocks
//     cost more than they gain, hence the other shape.  Full:
//     W = gate rows | up rows; a block computes the same 16 columns of both
//     products from one fetch of A and stores silu(gate) * up, with the roundings of the unfused
//     sequence (both products rounded to bfloat16, the activation rounded, then the product).
//   * query/key/value variant (QKV): the columns are query heads | key heads | value heads; query and
//     key heads are rotated by position (interleaved pairs, cosines and sines from a table), keys
//     and values go straight into their cache pages, queries into C: the rotary kernel's work, done
//     on the 32-bit sums after the rounding the unfused product would have applied.
//   * a root-mean-square norm around the products, without a kernel of its own.  norm(x) W^T =
//     ((x * gain) W^T) / sqrt(mean(x^2) + eps): the gain is applied to the rows, the factor per row
//     commutes with the product.  The product that ends a branch adds its result to the residual rows
//     (residual variant), stores the new rows, the new rows times the next norm's gain, and the sums
//     of squares of the new rows, one per block of 16 columns; the gated and the query/key/value
//     variants, which read the rows with the gain as A, add the pieces up (each lane a few, asked
//     for before the walk along K, then lanes and waves in a fixed order) and scale their 32-bit sums
//     by the factor before anything else happens to them.
#include "common.h"
#include "qkv_epilogue.h"

namespace {

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kStrip = 16;    // output columns per block
constexpr int kStepK = 128;   // k per wave step: 16 pieces of 8 elements
constexpr int kPitch = 136;   // elements between LDS rows: 128 + 8 of padding (272 bytes)
constexpr int kTileElems = 16 * kPitch;

__device__ __forceinline__ short4_t lo_half(u32x4_t v) { return __builtin_bit_cast(short4_t, u32x2_t{v[0], v[1]}); }
__device__ __forceinline__ short4_t hi_half(u32x4_t v) { return __builtin_bit_cast(short4_t, u32x2_t{v[2], v[3]}); }

enum Epilogue { kPlain = 0, kGated = 1, kQkv = 2, kGatedHalf = 3, kResidual = 4 };

// What the variants need that stand in for a norm.
struct NormArgs {
  // kGated, kGatedHalf, kQkv: the rows of A are to be read as A[m] / sqrt(sum[m] / width + eps);
  // row_sums [n_row_sums][16] are pieces of sum[m] (piece by piece, the 16 rows side by side).  Null: A as it is.
  const float* row_sums;
  int n_row_sums;
  float width, eps;
  // kResidual: C = residual + product (the product rounded to bfloat16 first, then the sum),
  // gained = C * gain (rounded; same leading dimension as C), and sums_out [blocks][16] receives
  // sum(C[m][block's columns]^2) of the rounded rows.
  const bf16_t* residual;
  int ldr;
  const bf16_t* gain;  // [N]
  bf16_t* gained;
  float* sums_out;
};

constexpr int kSumRows = 16;   // rows side by side in a piece of the sums of squares
// Pieces of a row's sum of squares that a lane asks for before the walk along K (any others it fetches at the
// end, and waits for each): with sixteen rows (MR = 4) the registers allow fewer blocks a CU anyway.
constexpr int held_sums(int mr) { return mr == 4 ? 16 : 8; }
// Pieces that a block of `waves` waves takes in without that wait: its lanes share out the pieces of 4 MR rows.
constexpr int sums_taken_ahead(int mr, int waves) { return held_sums(mr) * (kWave / (4 * mr)) * waves; }

// MR: groups of four rows of A that are fetched (M <= 4 * MR).  WAVES: waves per block = splits of K.
// EPI kGated, kGatedHalf: W holds 2 N rows, gate rows then up rows; C[M, N] = silu(A gate^T) * (A up^T);
// a block owns 16 (kGated) or 8 (kGatedHalf) columns of C.
template <int MR, int WAVES, typename OutT, int EPI>
__global__ void __launch_bounds__(WAVES* kWave)
gemm_stream_kernel(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, int ldw,
                   OutT* __restrict__ C, int ldc, int M, int N, int K, QkvArgs qa, NormArgs na) {
  constexpr bool GLU = EPI == kGated;
  constexpr int NW = GLU ? 2 : 1;  // W tiles per step
  // per wave: a tile of W [16][kPitch], then a tile of A [4 MR][kPitch] (rows past 4 MR are read as
  // whatever the neighbour holds: they only feed output columns that are never stored)
  extern __shared__ __attribute__((aligned(16))) bf16_t lds[];
  constexpr int kWaveElems = kTileElems + kTileElems;
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int n16 = lane % 16;  // operand layout: row
  const int g4 = lane / 16;   // operand layout: piece within a group of four
  const int q = lane / 16;    // fetch layout: row within a group of four
  const int piece = lane % 16;  // fetch layout: 16-byte piece of the row's 256 bytes
  constexpr bool HALF = EPI == kGatedHalf;
  const int n0 = blockIdx.x * (HALF ? kStrip / 2 : kStrip);
  bf16_t* w_lds = lds + (size_t)wave * kWaveElems;
  bf16_t* a_lds = w_lds + kTileElems;

  // K is walked in steps of 128; the waves of the block share the whole steps between them and the
  // last wave also takes the partial step at the end, if there is one
  const int steps_full = K / kStepK;
  const int steps_per_wave = (steps_full + WAVES - 1) / WAVES;
  const int step_lo = min(wave * steps_per_wave, steps_full);
  const int step_hi = min(step_lo + steps_per_wave, steps_full);

  // rows of W past N are clamped, rows of A past M read row 0: neither result is stored
  const bf16_t* wsrc[4 * NW];
#pragma unroll
  for (int t = 0; t < NW; ++t)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // half: tile rows 0..7 are gate rows n0.., rows 8..15 the up rows of the same columns
      const size_t row = HALF ? (size_t)(j / 2) * N + min(n0 + 4 * (j % 2) + q, N - 1) : (size_t)t * N + min(n0 + 4 * j + q, N - 1);
      wsrc[4 * t + j] = W + row * ldw + 8 * piece;
    }
  const bf16_t* asrc[MR];
#pragma unroll
  for (int j = 0; j < MR; ++j) {
    const int m = 4 * j + q;
    asrc[j] = A + (size_t)(m < M ? m : 0) * lda + 8 * piece;
  }

  float4_t acc[NW];
#pragma unroll
  for (int t = 0; t < NW; ++t) acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};

  // what the query/key/value epilogue reads from memory is asked for now and has long arrived when
  // the walk along K ends (asked for at the end, it would be one more round trip to memory)
  QkvOperands qkv_operands = {};
  if constexpr (EPI == kQkv) qkv_operands = qkv_fetch(min(n16, M - 1), n0 + 4 * g4, qa);

  // so are the pieces of the rows' sums of squares and the residual variant's four elements of the
  // rows it adds to.  The pieces of the 4 MR rows that the block may have are shared out over all its
  // lanes: lane l of a wave takes row l % (4 MR), and the lanes of a row take its pieces in turn (eight
  // each cover 256 pieces with eight rows and four waves, or sixteen rows and eight).  The loads stand
  // under no branch, so that nothing of theirs is waited for before the walk: without sums they
  // read the start of A, which nobody uses.
  constexpr bool NORMED = EPI == kGated || EPI == kGatedHalf || EPI == kQkv;
  constexpr int kHeldSums = held_sums(MR);
  constexpr int kSumSide = 4 * MR;                       // rows side by side in the lanes of a wave
  constexpr int kSumLanes = (kWave / kSumSide) * WAVES;  // lanes of the block that share a row's pieces
  const int sum_first = lane / kSumSide + (kWave / kSumSide) * wave;
  const bool normed = NORMED && na.row_sums != nullptr;
  const float* sum_base = normed ? na.row_sums : reinterpret_cast<const float*>(A);
  const uint32_t sum_row = normed && lane % kSumSide < M ? lane % kSumSide : 0;
  const int sum_last = normed ? na.n_row_sums - 1 : 0;
  float held[kHeldSums];
  if constexpr (NORMED) {
#pragma unroll
    for (int j = 0; j < kHeldSums; ++j) held[j] = sum_base[(uint32_t)min(sum_first + j * kSumLanes, sum_last) * kSumRows + sum_row];
  }
  u32x2_t residual = {0u, 0u}, gain = {0u, 0u};
  if constexpr (EPI == kResidual) {
    residual = *reinterpret_cast<const u32x2_t*>(na.residual + (size_t)min(n16, M - 1) * na.ldr + min(n0 + 4 * g4, N - 4));
    gain = *reinterpret_cast<const u32x2_t*>(na.gain + min(n0 + 4 * g4, N - 4));
  }

  auto fetch = [&](int st, u32x4_t* w, u32x4_t* a) {
    const int k0 = st * kStepK;
#pragma unroll
    for (int j = 0; j < 4 * NW; ++j) w[j] = *reinterpret_cast<const u32x4_t*>(wsrc[j] + k0);
#pragma unroll
    for (int j = 0; j < MR; ++j) a[j] = *reinterpret_cast<const u32x4_t*>(asrc[j] + k0);
  };
  // registers in fetch layout -> LDS -> registers in operand layout -> MFMA; the second W tile of
  // the gated variant passes through the same piece of LDS after the first (LDS runs in order)
  auto consume = [&](const u32x4_t* w, const u32x4_t* a) {
    u32x4_t wop[4], aop[4];
#pragma unroll
    for (int t = 0; t < NW; ++t) {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
#pragma unroll
      for (int j = 0; j < 4; ++j) *reinterpret_cast<u32x4_t*>(w_lds + (4 * j + q) * kPitch + 8 * piece) = w[4 * t + j];
      if (t == 0) {
#pragma unroll
        for (int j = 0; j < MR; ++j) *reinterpret_cast<u32x4_t*>(a_lds + (4 * j + q) * kPitch + 8 * piece) = a[j];
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        wop[u] = *reinterpret_cast<const u32x4_t*>(w_lds + n16 * kPitch + 8 * (g4 + 4 * u));
        if (t == 0) aop[u] = *reinterpret_cast<const u32x4_t*>(a_lds + n16 * kPitch + 8 * (g4 + 4 * u));
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(lo_half(wop[u]), lo_half(aop[u]), acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(hi_half(wop[u]), hi_half(aop[u]), acc[t], 0, 0, 0);
      }
    }
  };

  u32x4_t w0[4 * NW], w1[4 * NW], a0[MR], a1[MR];
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
  // Inside the loop the prefetches are unconditional: a load under a branch would make the wait
  // before its use cover both paths, that is, wait for the prefetch itself.  The last one or two
  // steps stand behind the loop, so that nothing is fetched that nobody uses (with two to four
  // steps a wave, as in the products with few columns, one spare fetch was a fifth of all).
  // This lane's share of its row's sum of squares.  The pieces asked for at the start are added up as
  // soon as the first tile of W has come (loads return in the order they were asked for, so the pieces
  // are there too and nothing new is waited for), so that they hold no registers through the rest of
  // the walk: registers decide between one block a CU and two.
  float squares = 0.f;
  auto add_held = [&]() {
    if constexpr (NORMED) {
#pragma unroll
      for (int j = 0; j < kHeldSums; ++j) squares += normed && sum_first + j * kSumLanes <= sum_last ? held[j] : 0.f;
      asm volatile("" : "+v"(squares));  // here, not wherever the result is used
    }
  };
  if (nst > 0) {
    fetch(step_of(0), w0, a0);
    int i = 0;
    if (nst > 2) {  // the loop's first trip, with the pieces added in its middle
      fetch(step_of(1), w1, a1);
      consume(w0, a0);
      add_held();
      fetch(step_of(2), w0, a0);
      consume(w1, a1);
      i = 2;
    }
    for (; i + 2 < nst; i += 2) {
      fetch(step_of(i + 1), w1, a1);
      consume(w0, a0);
      fetch(step_of(i + 2), w0, a0);
      consume(w1, a1);
    }
    if (i + 1 < nst) {
      fetch(step_of(i + 1), w1, a1);
      consume(w0, a0);
      consume(w1, a1);
    } else {
      consume(w0, a0);
    }
  }
  // the partial step: pieces past K are read from a clamped address and the A side is zeroed, so the
  // out-of-range products vanish
  if (wave == WAVES - 1 && steps_full * kStepK < K) {
    const int k = steps_full * kStepK + 8 * piece;
    const int kc = min(k, K - 8) - 8 * piece;
    const uint32_t keep = k < K ? 0xFFFFFFFFu : 0u;
#pragma unroll
    for (int j = 0; j < 4 * NW; ++j) w0[j] = *reinterpret_cast<const u32x4_t*>(wsrc[j] + kc);
#pragma unroll
    for (int j = 0; j < MR; ++j) {
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(asrc[j] + kc);
      a0[j] = u32x4_t{v[0] & keep, v[1] & keep, v[2] & keep, v[3] & keep};
    }
    consume(w0, a0);
  }

  if (nst <= 2) add_held();
  if constexpr (NORMED) {  // pieces beyond those asked for at the start (more than eight or sixteen for each of a row's lanes)
    if (normed)
      for (int p = sum_first + kHeldSums * kSumLanes; p <= sum_last; p += kSumLanes) squares += sum_base[(uint32_t)p * kSumRows + sum_row];
  }

  // acc[t][i] = C^T[n0 + 4 g4 + i][n16]; add the waves' shares in wave order (the wave's own W tile
  // in LDS serves as its slot, the lanes' shares of the sums of squares behind the products')
  if (WAVES > 1) {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    float* slot = reinterpret_cast<float*>(w_lds);
#pragma unroll
    for (int t = 0; t < NW; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) slot[(t * kWave + lane) * 4 + i] = acc[t][i];
    if constexpr (NORMED) slot[NW * kWave * 4 + lane] = squares;
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int t = 0; t < NW; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float sum = 0.f;
#pragma unroll
        for (int w2 = 0; w2 < WAVES; ++w2)
          sum += reinterpret_cast<const float*>(lds + (size_t)w2 * kWaveElems)[(t * kWave + lane) * 4 + i];
        acc[t][i] = sum;
      }
    if constexpr (NORMED) {
      squares = 0.f;
#pragma unroll
      for (int w2 = 0; w2 < WAVES; ++w2) squares += reinterpret_cast<const float*>(lds + (size_t)w2 * kWaveElems)[NW * kWave * 4 + lane];
    }
  }
  if constexpr (NORMED) {
    // the lanes of a row lie 4 MR apart (every lane of the wave is here); lane n16 < 4 MR then holds row n16's sum
#pragma unroll
    for (int apart = kSumSide; apart < kWave; apart *= 2) squares += __shfl_xor(squares, apart, kWave);
    if (normed) {
      const float scale = 1.0f / sqrtf(squares / na.width + na.eps);
#pragma unroll
      for (int t = 0; t < NW; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[t][i] *= scale;
    }
  }
  if constexpr (EPI == kQkv) {
    // the lane's four columns are channels of one head (N % 4 == 0)
    const int n = n0 + 4 * g4;
    if (n16 < M && n < N) {
      const float sums[4] = {acc[0][0], acc[0][1], acc[0][2], acc[0][3]};
      qkv_finish(sums, n16, n, qa, reinterpret_cast<bf16_t*>(C), ldc, qkv_operands);
    }
  } else if constexpr (HALF) {
    // lanes with g4 < 2 hold the gate sums of columns n0 + 4 g4 + i, the lanes 32 further on the up
    // sums of the same columns (every lane takes part in the exchange)
    float up[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) up[i] = __shfl(acc[0][i], (lane + 32) % kWave, kWave);
    if (n16 < M && g4 < 2) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + 4 * g4 + i;
        if (n >= N) continue;
        const float g = to_f32(from_f32<OutT>(acc[0][i]));
        const float u = to_f32(from_f32<OutT>(up[i]));
        const float act = to_f32(from_f32<OutT>(g / (1.0f + expf(-g))));
        C[(size_t)n16 * ldc + n] = from_f32<OutT>(act * u);
      }
    }
  } else if constexpr (EPI == kResidual) {
    // the lane's four columns n0 + 4 g4 .. + 3 of row n16 (N % 4 == 0): new row = residual + product
    const int n = n0 + 4 * g4;
    const bool mine = n16 < M && n < N;
    float sq = 0.f;
    uint32_t packed[2], packed_gained[2];
    auto wide = [](uint32_t word, int i) { return __builtin_bit_cast(float, i % 2 ? word & 0xFFFF0000u : word << 16); };
    auto bits = [](bf16_t v) { return (uint32_t)__builtin_bit_cast(uint16_t, v); };
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bf16_t sum = from_f32<bf16_t>(wide(residual[i / 2], i) + to_f32(from_f32<bf16_t>(acc[0][i])));
      const float f = to_f32(sum);
      sq += f * f;
      const bf16_t with_gain = from_f32<bf16_t>(f * wide(gain[i / 2], i));
      packed[i / 2] = i % 2 ? packed[i / 2] | (bits(sum) << 16) : bits(sum);
      packed_gained[i / 2] = i % 2 ? packed_gained[i / 2] | (bits(with_gain) << 16) : bits(with_gain);
    }
    if (mine) {
      *reinterpret_cast<u32x2_t*>(C + (size_t)n16 * ldc + n) = u32x2_t{packed[0], packed[1]};
      *reinterpret_cast<u32x2_t*>(na.gained + (size_t)n16 * ldc + n) = u32x2_t{packed_gained[0], packed_gained[1]};
    }
    sq = mine ? sq : 0.f;
    sq += __shfl_xor(sq, 16, kWave);
    sq += __shfl_xor(sq, 32, kWave);
    if (g4 == 0 && n16 < M) na.sums_out[(size_t)blockIdx.x * kSumRows + n16] = sq;
  } else if (n16 < M) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + 4 * g4 + i;
      if (n >= N) continue;
      if constexpr (GLU) {
        const float g = to_f32(from_f32<OutT>(acc[0][i]));
        const float u = to_f32(from_f32<OutT>(acc[1][i]));
        const float act = to_f32(from_f32<OutT>(g / (1.0f + expf(-g))));
        C[(size_t)n16 * ldc + n] = from_f32<OutT>(act * u);
      } else {
        C[(size_t)n16 * ldc + n] = from_f32<OutT>(acc[0][i]);
      }
    }
  }
}

template <int MR, int WAVES, typename OutT, int EPI>
int launch_typed(const bf16_t* A, int lda, const bf16_t* W, int ldw, OutT* C, int ldc, int M, int N, int K,
                 const QkvArgs& qa, const NormArgs& na, hipStream_t stream) {
  const size_t lds = (size_t)WAVES * 2 * kTileElems * sizeof(bf16_t);
  static bool raised = false;  // blocks past 64 KB of LDS have to be allowed once per kernel
  if (lds > 64 * 1024 && !raised) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_stream_kernel<MR, WAVES, OutT, EPI>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return tl_fail(TL_ERR_HIP, "gemm_stream: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    raised = true;
  }
  constexpr int kCols = EPI == kGatedHalf ? kStrip / 2 : kStrip;  // columns of C per block
  const dim3 grid((N + kCols - 1) / kCols);
  gemm_stream_kernel<MR, WAVES, OutT, EPI><<<grid, WAVES * kWave, lds, stream>>>(A, lda, W, ldw, C, ldc, M, N, K, qa, na);
  return tl_check_launch("gemm_stream");
}

template <int MR, int WAVES>
int launch(const bf16_t* A, int lda, const bf16_t* W, int ldw, void* C, int ldc, int M, int N, int K,
           int out_dtype, int epi, const QkvArgs& qa, const NormArgs& na, hipStream_t stream) {
  if (epi == kResidual) return launch_typed<MR, WAVES, bf16_t, kResidual>(A, lda, W, ldw, (bf16_t*)C, ldc, M, N, K, qa, na, stream);
  if (epi == kGated) return launch_typed<MR, WAVES, bf16_t, kGated>(A, lda, W, ldw, (bf16_t*)C, ldc, M, N, K, qa, na, stream);
  if (epi == kGatedHalf) return launch_typed<MR, WAVES, bf16_t, kGatedHalf>(A, lda, W, ldw, (bf16_t*)C, ldc, M, N, K, qa, na, stream);
  if (epi == kQkv) return launch_typed<MR, WAVES, bf16_t, kQkv>(A, lda, W, ldw, (bf16_t*)C, ldc, M, N, K, qa, na, stream);
  if (out_dtype == TL_BF16) return launch_typed<MR, WAVES, bf16_t, kPlain>(A, lda, W, ldw, (bf16_t*)C, ldc, M, N, K, qa, na, stream);
  return launch_typed<MR, WAVES, float, kPlain>(A, lda, W, ldw, (float*)C, ldc, M, N, K, qa, na, stream);
}

template <int MR>
int launch_waves(int waves, const bf16_t* A, int lda, const bf16_t* W, int ldw, void* C, int ldc, int M, int N,
                 int K, int out_dtype, int epi, const QkvArgs& qa, const NormArgs& na, hipStream_t stream) {
  switch (waves) {
    case 1: return launch<MR, 1>(A, lda, W, ldw, C, ldc, M, N, K, out_dtype, epi, qa, na, stream);
    case 2: return launch<MR, 2>(A, lda, W, ldw, C, ldc, M, N, K, out_dtype, epi, qa, na, stream);
    case 4: return launch<MR, 4>(A, lda, W, ldw, C, ldc, M, N, K, out_dtype, epi, qa, na, stream);
    default: return launch<MR, 8>(A, lda, W, ldw, C, ldc, M, N, K, out_dtype, epi, qa, na, stream);
  }
}

int run(const void* A, int lda, const void* W, int ldw, void* C, int ldc, int M, int N, int K, int out_dtype,
        int waves, int epi, const QkvArgs& qa, const NormArgs& na, hipStream_t stream) {
  TL_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_stream: bad sizes M=%d N=%d K=%d", M, N, K);
  if (M > 16) return tl_fail(TL_ERR_UNSUPPORTED, "gemm_stream: M=%d exceeds 16", M);
  if (K % 8) return tl_fail(TL_ERR_UNSUPPORTED, "gemm_stream: K=%d is not a multiple of 8", K);
  TL_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_stream: leading dimensions too small");
  TL_REQUIRE(lda % 8 == 0 && ldw % 8 == 0 && ((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0,
             "gemm_stream: rows must start on 16-byte boundaries");
  TL_REQUIRE(out_dtype == TL_BF16 || out_dtype == TL_F32, "gemm_stream: out_dtype must be 0 or 1");
  if (na.row_sums != nullptr) {
    TL_REQUIRE(epi != kPlain && epi != kResidual, "gemm_stream: only the gated and the query/key/value variants scale their rows");
    TL_REQUIRE(na.n_row_sums > 0 && na.width > 0.f && ((uintptr_t)na.row_sums % 4) == 0, "gemm_stream: bad sums of squares");
  }
  if (epi == kResidual) {
    TL_REQUIRE(na.residual != nullptr && na.sums_out != nullptr && na.gain != nullptr && na.gained != nullptr,
               "gemm_stream_residual: rows to add to, a gain and places for the results are needed");
    if (N % 4) return tl_fail(TL_ERR_UNSUPPORTED, "gemm_stream_residual: N=%d is not a multiple of 4", N);
    TL_REQUIRE(na.ldr >= N && na.ldr % 4 == 0 && ldc % 4 == 0 && ((uintptr_t)na.residual % 8) == 0 && ((uintptr_t)C % 8) == 0 &&
                   ((uintptr_t)na.gain % 8) == 0 && ((uintptr_t)na.gained % 8) == 0,
               "gemm_stream_residual: rows must start on 8-byte boundaries");
  }
  if (M == 0) return TL_OK;
  if (waves == 0) {
    // enough waves to keep loads in flight on every CU: about 16 a CU (4,096 on 256 CUs), at least two steps each
    const int enough = 16 * tl_device_facts().compute_units;
    const int cols = epi == kGatedHalf ? kStrip / 2 : kStrip;
    const int strips = (N + cols - 1) / cols;
    const int steps = (K + kStepK - 1) / kStepK;
    waves = 1;
    while (waves < 8 && strips * waves < enough && steps >= 2 * waves * 2) waves *= 2;
  }
  TL_REQUIRE(waves == 1 || waves == 2 || waves == 4 || waves == 8, "gemm_stream: waves must be 1, 2, 4 or 8");
  if (na.row_sums != nullptr) {
    // as many waves as take in all pieces of the sums of squares ahead (rows of 8,192 elements come in 512
    // pieces): a wave that fetches its share at the end waits a trip to memory for every few of them
    const int mr = M <= 4 ? 1 : M <= 8 ? 2 : 4;
    while (waves < 8 && sums_taken_ahead(mr, waves) < na.n_row_sums && K / kStepK >= 2 * waves) waves *= 2;
  }
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  if (M <= 4) return launch_waves<1>(waves, a, lda, w, ldw, C, ldc, M, N, K, out_dtype, epi, qa, na, stream);
  if (M <= 8) return launch_waves<2>(waves, a, lda, w, ldw, C, ldc, M, N, K, out_dtype, epi, qa, na, stream);
  return launch_waves<4>(waves, a, lda, w, ldw, C, ldc, M, N, K, out_dtype, epi, qa, na, stream);
}

}  // namespace

// A [M, K] and W [N, K] bfloat16, row-major with leading dimensions lda / ldw (multiples of 8, bases
// 16-byte aligned); C [M, N] bfloat16 (out_dtype 1) or 32-bit (out_dtype 0).  M <= 16, K a multiple of 8.
// waves = 0 picks the number of K splits from the sizes.
TL_EXPORT int tl_gemm_stream(const void* A, int lda, const void* W, int ldw, void* C, int ldc, int M, int N,
                             int K, int out_dtype, int waves, hipStream_t stream) {
  return run(A, lda, W, ldw, C, ldc, M, N, K, out_dtype, waves, kPlain, QkvArgs{}, NormArgs{}, stream);
}

// The gated pair of products: W [2 N, K] = gate rows | up rows; C [M, N] bfloat16 =
// silu(A gate^T) * (A up^T), rounded as the two products, the activation and the final product
// would be if each were stored in bfloat16.  cols: 16 or 8 columns of C per block.
// row_sums [n_row_sums][16] 32-bit or null: pieces of a sum of squares per row, as tl_gemm_stream_residual
// leaves them; then row m of both products is scaled by 1 / sqrt(sum / K + eps) before the roundings.
TL_EXPORT int tl_gemm_stream_glu(const void* A, int lda, const void* W, int ldw, void* C, int ldc, int M, int N,
                                 int K, int waves, int cols, const float* row_sums, int n_row_sums, float eps,
                                 hipStream_t stream) {
  TL_REQUIRE(cols == 8 || cols == 16, "gemm_stream_glu: cols must be 8 or 16");
  NormArgs na = {};
  na.row_sums = row_sums; na.n_row_sums = n_row_sums; na.width = (float)K; na.eps = eps;
  return run(A, lda, W, ldw, C, ldc, M, N, K, TL_BF16, waves, cols == 8 ? kGatedHalf : kGated, QkvArgs{}, na, stream);
}

// C [M, N] bfloat16 = residual [M, N] + A W^T (the product rounded to bfloat16, then the sum in
// 32-bit, rounded); gained [M, N] (leading dimension ldc) = C * gain [N], rounded; and sums_out
// [ceil(N / 16)][16] 32-bit = the sums of squares of the rows of C by blocks of 16 columns, the rows
// side by side (only the first M of each 16 are written): what a root-mean-square norm of those
// rows needs, for the product that reads `gained` next.  N a multiple of 4.
TL_EXPORT int tl_gemm_stream_residual(const void* A, int lda, const void* W, int ldw, const void* residual, int ldr,
                                      const void* gain, void* C, void* gained, int ldc, float* sums_out, int M,
                                      int N, int K, int waves, hipStream_t stream) {
  NormArgs na = {};
  na.residual = (const bf16_t*)residual; na.ldr = ldr; na.gain = (const bf16_t*)gain; na.gained = (bf16_t*)gained;
  na.sums_out = sums_out;
  return run(A, lda, W, ldw, C, ldc, M, N, K, TL_BF16, waves, kResidual, QkvArgs{}, na, stream);
}

// The query/key/value projection with the rotary kernel's work in its epilogue.  W [(Hq + 2 Hkv) *
// head_dim, K]; C [M, that width] receives the rotated queries (and keys and values when no pages are
// given).  cos_sin [M][rotary_dim / 2][2]: cosine and sine of each row's position (interleaved pairs
// only).  k_pages / v_pages [page][Hkv][page_size][head_dim]; slot_mapping [M].  head_dim % 4 == 0.
// row_sums, n_row_sums, eps: as for tl_gemm_stream_glu.
TL_EXPORT int tl_gemm_stream_qkv(const void* A, int lda, const void* W, int ldw, void* C, int ldc, int M, int K,
                                 int n_q_heads, int n_kv_heads, int head_dim, int rotary_dim,
                                 const float* cos_sin, void* k_pages, void* v_pages,
                                 const int32_t* slot_mapping, int page_size, int waves, const float* row_sums,
                                 int n_row_sums, float eps, hipStream_t stream) {
  QkvArgs qa;
  const int rc = qkv_args("gemm_stream_qkv", n_q_heads, n_kv_heads, head_dim, rotary_dim, cos_sin, k_pages, v_pages,
                          slot_mapping, page_size, C, ldc, &qa);
  if (rc != TL_OK) return rc;
  const int N = (n_q_heads + 2 * n_kv_heads) * head_dim;
  NormArgs na = {};
  na.row_sums = row_sums; na.n_row_sums = n_row_sums; na.width = (float)K; na.eps = eps;
  return run(A, lda, W, ldw, C, ldc, M, N, K, TL_BF16, waves, kQkv, qa, na, stream);
}
