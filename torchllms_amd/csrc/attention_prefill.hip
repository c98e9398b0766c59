// Causal attention of prompt portions over paged bfloat16 keys and values (the cached prefix and
// the portion itself, which the step has already written into the pages): the prefill kernel.
//
//   * a block takes a tile of consecutive queries of one request and one kv head, with all query
//     heads that share it: the 128 MFMA columns of its 4 waves are (query, head) pairs, so a key or
//     value is fetched once for the whole group.  A launch whose blocks all fit the GPU at once is as
//     long as its longest block; there a block has a second set of 4 waves for the same columns, each
//     set takes every second tile of keys, and they add up what they have through LDS at the end.
//   * keys and values stream through LDS in tiles of 64 keys, both as they lie in the page, and get
//     there without passing through registers: `global_load_lds_dwordx4` puts a wave's 64 x 16 bytes
//     at consecutive LDS addresses.  Rows are therefore not padded; instead the 16-byte pieces of a
//     row are stored in an order that depends on the row (piece ^ f(row)), so that the 16 lanes that
//     read the same piece of 16 rows still meet 16 different banks.  Two buffers per set of waves:
//     the next tile lands while the current one is worked off, with one barrier a tile.
//   * scores are computed transposed, S^T[key][column] = K Q^T, by MFMA 16x16x32 bf16 (a lane's 16
//     bytes of a key row are one operand); their output layout, taken over two blocks of 16 keys, is
//     exactly the B-operand layout of P^T in O^T[channel][column] = V^T P^T, so the probabilities
//     never leave their registers.  Softmax statistics are 32-bit, per column.
//   * the A operand of the second product wants, per lane, one channel of eight keys, while the
//     values lie in LDS key by key.  gfx950's transposing LDS load (ds_read_b64_tr_b16) hands every
//     lane one channel of four key rows: two of them are an operand, no permutes.
//   * every column has its own causal limit (its query's position) and window start.
//
// Compiled once per head size (-DTL_HEAD_DIM=32|64|128|256).
#include <stdarg.h>
#include <stdio.h>

#include <type_traits>

#include "common.h"

#ifndef TL_HEAD_DIM
#error "compile with -DTL_HEAD_DIM=<head size>"
#endif

static thread_local char g_variant_error[512] = "";
static int variant_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_variant_error, sizeof(g_variant_error), fmt, ap);
  va_end(ap);
  return code;
}
TL_EXPORT const char* tl_variant_last_error() { return g_variant_error; }

namespace {

constexpr int DH = TL_HEAD_DIM;
static_assert(DH == 32 || DH == 64 || DH == 128 || DH == 256, "prefill kernel: head size 32, 64, 128 or 256");

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kWaves = 4;                   // waves that share the columns of a block
constexpr int NC = DH <= 128 ? 2 : 1;        // MFMA column blocks per wave
constexpr int kCols = kWaves * NC * 16;      // columns per block
constexpr int KT = DH <= 128 ? 64 : 32;       // keys per LDS tile
constexpr int KL = DH / 32;                  // 16-byte pieces of a key row per lane
constexpr int DT = DH / 16;                  // channel tiles of the output
constexpr int kPieces = DH / 8;              // 16-byte pieces in a key/value row
constexpr int kRowsPerLoad = kWave / kPieces;  // rows that one wave load (64 lanes x 16 bytes) covers
constexpr int kLoadsPerWave = KT / kRowsPerLoad / kWaves;  // wave loads per tile and operand
static_assert(kRowsPerLoad >= 1 && KT % (kRowsPerLoad * kWaves) == 0, "tile does not divide over the block");
constexpr int kTileElems = KT * DH;          // one operand's tile in LDS, rows unpadded
// The piece s of row r lies at slot s ^ swizzle(r).  Banks repeat every 256 bytes, that is every
// kRowsPerSweep rows; rows that start on the same bank get different slots for the same piece.
constexpr int kRowsPerSweep = DH >= 128 ? 1 : 128 / DH;
constexpr int kSwizzle = kPieces < 16 ? kPieces : 16;
__device__ __forceinline__ int swizzle(int row) { return (row / kRowsPerSweep) % kSwizzle; }
// element offset of piece `piece` of row `row` within a tile of keys
__device__ __forceinline__ int tile_at(int row, int piece) { return row * DH + 8 * (piece ^ swizzle(row)); }
// Values are read by transposing loads (see below): 16 lanes fetch 32 bytes at the same place of four
// consecutive rows, and these four have to meet different banks.  Rows of 256 bytes and more start on
// the same bank, rows of 128 bytes on every second: the pair of pieces moves with the row.
__device__ __forceinline__ int swizzle_v(int row) { return DH >= 128 ? 2 * (row % 8) : DH == 64 ? 2 * ((row / 2) % 4) : 0; }
__device__ __forceinline__ int tile_at_v(int row, int piece) { return row * DH + 8 * (piece ^ swizzle_v(row)); }

struct PrefillArgs {
  const bf16_t* q;
  int q_stride;
  bf16_t* out;
  int out_stride;
  const bf16_t* k_pages;
  const bf16_t* v_pages;
  const int32_t* qo_indptr;   // [rows + 1] first token of each row in this launch's token numbering
  const int32_t* kv_lens;     // [rows] tokens of the request after this step
  const int32_t* block_table;
  int bt_stride;
  const int32_t* tile_row;    // [tiles] row of each query tile
  const int32_t* tile_q0;     // [tiles] first query of the tile, counted from the row's first new token
  int n_kv_heads;
  int group;
  int page_size;
  int page_shift;
  int window;
  float scale_log2e;
};

typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

// 16 bytes as they come from memory = eight bfloat16 = one operand of the 16x16x32 MFMA
struct Pack16 {
  u32x4_t u;
  __device__ __forceinline__ bf16x8_t op() const { return __builtin_bit_cast(bf16x8_t, u); }
};

// two floats -> two bfloat16 in one 32-bit word (first in the low half), round to nearest even
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2_t{a, b}, bf16x2_t));
}

// Target builtins that the kernel's own body uses stand in device functions: the host pass, which
// only needs the kernel's stub, does not know them.
__device__ __forceinline__ int wave_uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ void wait_for_loads() { __builtin_amdgcn_s_waitcnt(0); }
__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// The block's LDS: [group][buffer][keys | values][kTileElems].  It is declared here and not in the
// kernel: a __shared__ array whose size depends on a template parameter of the kernel itself keeps
// this compiler from emitting the kernel's host stub.
template <int GROUPS>
__device__ __forceinline__ bf16_t* tile_memory() {
  __shared__ __attribute__((aligned(16))) bf16_t tiles[GROUPS * 2 * 2 * kTileElems];
  return tiles;
}

// The transposing LDS load of gfx950 (ds_read_b64_tr_b16).  Each lane names 8 bytes (four 16-bit
// elements); within every 16 lanes, lane 4a + b receives element b of the lanes a, 4 + a, 8 + a and
// 12 + a, in this order.  With lane 4j + a pointing at four consecutive channels 4a .. 4a + 3 of key
// row j, lane m = 4a + b ends up with channel m of four key rows: half an MFMA operand of V^T,
// straight from values that lie in LDS as they lie in the page.
typedef short short4v_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x2_t lds_transposed(const bf16_t* src) {
  typedef short4v_t __attribute__((address_space(3))) * lds_ptr_t;
  return __builtin_bit_cast(u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)src));
}

// RP: query heads per kv head, rounded up to a power of two.  WINDOWED: whether queries have a lower
// bound on the keys they see; without one the test against it is compiled out.  GROUPS: 1, or 2 sets
// of kWaves waves that take the same columns and every second tile of keys each, and add up what
// they have at the end through LDS: a block's chain of tiles is half as long, which is what a launch
// needs whose blocks all fit the GPU at once and whose time is therefore that of its longest block.
template <int RP, bool WINDOWED, int GROUPS>
__global__ void __launch_bounds__(GROUPS * kWaves * kWave, GROUPS == 1 ? 2 : 1) attn_prefill_kernel(PrefillArgs a) {
  constexpr int QB = kCols / RP;  // queries per block

  const int tile = blockIdx.y;  // the host lists the tiles in the order that balances the launch
  const int kvh = blockIdx.x;
  const int grp = GROUPS == 1 ? 0 : wave_uniform(threadIdx.x / (kWaves * kWave));
  bf16_t* const tiles = tile_memory<GROUPS>() + grp * 4 * kTileElems;  // this group's [buffer][keys | values]
  const int wave = (threadIdx.x / kWave) % kWaves;  // within the group
  const int lane = threadIdx.x % kWave;
  const int n16 = lane % 16;
  const int g4 = lane / 16;
  const int R = a.group;

  const int row = a.tile_row[tile];
  const int q0 = a.tile_q0[tile];
  const int tok0 = a.qo_indptr[row];
  const int q_len = a.qo_indptr[row + 1] - tok0;
  const int kv_len = a.kv_lens[row];
  const int pos0 = kv_len - q_len;  // position of the row's first new token
  const int32_t* bt = a.block_table + (size_t)row * a.bt_stride;
  const size_t head_elems = (size_t)a.page_size * DH;

  auto window_lo = [&](int pos) { return (a.window > 0 && pos - a.window + 1 > 0) ? pos - a.window + 1 : 0; };
  const int q_last = min(q0 + QB, q_len) - 1;       // last query of the tile
  const int key_lo = window_lo(pos0 + q0);          // first key any column sees
  const int key_hi = pos0 + q_last;                 // last key any column sees
  const int tile_begin = key_lo & ~(KT - 1);

  // this lane's columns: col -> (query, head)
  int col_pos[NC], col_lo[NC], col_tok[NC], col_head[NC];
  bool col_ok[NC];
  Pack16 qreg[NC][KL];
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int col = 16 * (wave * NC + i) + n16;
    const int ql = q0 + col / RP;
    const int hh = col % RP;
    col_ok[i] = ql < q_len && hh < R;
    col_tok[i] = tok0 + (col_ok[i] ? ql : q0);
    col_head[i] = kvh * R + (col_ok[i] ? hh : 0);
    // a column that stands for nothing sees every key with a zero query: finite, never stored
    col_pos[i] = col_ok[i] ? pos0 + ql : 0x3fffffff;
    col_lo[i] = col_ok[i] ? window_lo(pos0 + ql) : 0;
    const bf16_t* qrow = a.q + (size_t)col_tok[i] * a.q_stride + (size_t)col_head[i] * DH;
#pragma unroll
    for (int u = 0; u < KL; ++u) {
      qreg[i][u].u = *reinterpret_cast<const u32x4_t*>(qrow + 32 * u + 8 * g4);
      if (!col_ok[i]) qreg[i][u].u = u32x4_t{0u, 0u, 0u, 0u};
    }
  }
  // range of keys this wave's columns can see at all (tiles outside it are skipped)
  int wave_hi = -1, wave_lo = 0x3fffffff;
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int p_ok = col_ok[i] ? col_pos[i] : -1;
    const int l_ok = col_ok[i] ? col_lo[i] : 0x3fffffff;
    wave_hi = max(wave_hi, p_ok);
    wave_lo = min(wave_lo, l_ok);
  }
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    wave_hi = max(wave_hi, __shfl_xor(wave_hi, off, kWave));
    wave_lo = min(wave_lo, __shfl_xor(wave_lo, off, kWave));
  }

  float m_run[NC], l_part[NC];
  float4_t acc[NC][DT];
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    m_run[i] = -INFINITY;
    l_part[i] = 0.f;
#pragma unroll
    for (int t = 0; t < DT; ++t) acc[i][t] = float4_t{0.f, 0.f, 0.f, 0.f};
  }

  // global -> LDS for one tile of keys and values, asynchronously.  Wave load j of wave w covers rows
  // (j * kWaves + w) * kRowsPerLoad ... of the tile: lane -> (row, slot), and fetches the piece that
  // belongs in that slot.  Keys outside the visible range are clamped into it (their scores are
  // masked), so no load touches a page the request does not hold.
  auto dma = [&](int base, int buffer) {
#pragma unroll
    for (int j = 0; j < kLoadsPerWave; ++j) {
      const int first = (j * kWaves + wave) * kRowsPerLoad;
      const int r = first + lane / kPieces;
      const int piece_k = (lane % kPieces) ^ swizzle(r);
      const int piece_v = (lane % kPieces) ^ swizzle_v(r);
      int key = base + r;
      key = key < key_lo ? key_lo : (key > key_hi ? key_hi : key);
      const int blk = a.page_shift >= 0 ? key >> a.page_shift : key / a.page_size;
      const int off = a.page_shift >= 0 ? key & (a.page_size - 1) : key % a.page_size;
      const size_t at = ((size_t)bt[blk] * a.n_kv_heads + kvh) * head_elems + (size_t)off * DH;
      __builtin_amdgcn_global_load_lds(a.k_pages + at + 8 * piece_k, &tiles[(2 * buffer) * kTileElems + first * DH], 16, 0, 0);
      __builtin_amdgcn_global_load_lds(a.v_pages + at + 8 * piece_v, &tiles[(2 * buffer + 1) * kTileElems + first * DH], 16, 0, 0);
    }
  };

  dma(tile_begin + grp * KT, 0);
  int buffer = 0;
  // One tile of keys: wait for it, start the next one's loads, work it off.  `masked`: whether some
  // column may not see some key of the tile; where every column sees every key the tests are
  // compiled out.
  auto work_tile = [&](int base, auto masked) {
    // this wave's loads of the tile have landed; after the barrier everybody's have, and everybody
    // has finished with the tile before, whose buffer the next tile's loads may now overwrite
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    dma(base + GROUPS * KT, buffer ^ 1);  // unconditional (keys are clamped): no wait has to cover a path without it
    const bf16_t* k_lds = tiles + (2 * buffer) * kTileElems;
    const bf16_t* v_lds = tiles + (2 * buffer + 1) * kTileElems;

    if (base > wave_hi || base + KT - 1 < wave_lo) return;  // nothing here for this wave's columns

    // the whole tile at once: scores, softmax bookkeeping (one running maximum and one rescaling of
    // the sums per tile), then P.V in groups of 32 keys
    constexpr int NS = KT / 16;  // blocks of 16 keys
    {
    // phase 1: scores S^T[key][column], one MFMA chain per (16 keys, column block).  No branch from
    // here to the end of the tile, so that the compiler can interleave the chains and the column
    // blocks' softmax arithmetic; a block of 16 keys that the wave does not see at all is computed
    // and masked like any other.
    float4_t c[NC][NS];
#pragma unroll
    for (int sub = 0; sub < NS; ++sub)
#pragma unroll
      for (int i = 0; i < NC; ++i) c[i][sub] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < KL; ++u) {
      Pack16 ka[NS];
#pragma unroll
      for (int sub = 0; sub < NS; ++sub)
        ka[sub].u = *reinterpret_cast<const u32x4_t*>(&k_lds[tile_at(16 * sub + n16, g4 + 4 * u)]);
#pragma unroll
      for (int sub = 0; sub < NS; ++sub)
#pragma unroll
        for (int i = 0; i < NC; ++i)
          c[i][sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[sub].op(), qreg[i][u].op(), c[i][sub], 0, 0, 0);
    }
    // softmax bookkeeping once per tile and column: mask, maximum, rescale, probabilities.
    // Scores stay unscaled; the scale enters through one fused multiply-add per element:
    // exp2(s * scale - m), with m the running maximum of s * scale.
    bf16x8_t pb[NC][NS / 2];  // per 32 keys; slot e < 4: key 4 g4 + e of the first 16 keys; e >= 4: of the second 16
    float alpha[NC];
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      float tmax = -INFINITY;
#pragma unroll
      for (int sub = 0; sub < NS; ++sub)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          // plain bit operations, no short-circuit: a branch here, right behind the MFMAs, is what
          // this compiler has been seen to get wrong (the masked value overwrote live scores)
          float sc = c[i][sub][r];
          if constexpr (decltype(masked)::value) {
            const int key = base + 16 * sub + 4 * g4 + r;
            const bool valid = WINDOWED ? (key >= col_lo[i]) & (key <= col_pos[i]) : key <= col_pos[i];
            sc = valid ? sc : -INFINITY;
            c[i][sub][r] = sc;
          }
          tmax = fmaxf(tmax, sc);
        }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
      const float m_new = fmaxf(m_run[i], tmax * a.scale_log2e);  // the scale is positive
      // a column may not have met a visible key yet: then nothing is rescaled and nothing added
      const bool none = m_new == -INFINITY;
      alpha[i] = none ? 1.f : __builtin_amdgcn_exp2f(m_run[i] - m_new);
      const float neg_m = none ? 0.f : -m_new;
      float psum = 0.f;
      uint32_t pw[2 * NS];
#pragma unroll
      for (int sub = 0; sub < NS; ++sub) {
        float pr[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          pr[r] = __builtin_amdgcn_exp2f(fmaf(c[i][sub][r], a.scale_log2e, neg_m));  // exp2(-inf) = 0
          psum += pr[r];
        }
        pw[2 * sub] = pack_bf16x2(pr[0], pr[1]);
        pw[2 * sub + 1] = pack_bf16x2(pr[2], pr[3]);
      }
#pragma unroll
      for (int g = 0; g < NS / 2; ++g)
        pb[i][g] = __builtin_bit_cast(bf16x8_t, u32x4_t{pw[4 * g], pw[4 * g + 1], pw[4 * g + 2], pw[4 * g + 3]});
      l_part[i] = l_part[i] * alpha[i] + psum;
      m_run[i] = m_new;
    }
    // the sums so far follow the maxima (no test whether any moved: a branch here keeps the compiler
    // from overlapping this arithmetic with the MFMAs around it, which costs more than it saves)
#pragma unroll
    for (int i = 0; i < NC; ++i)
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][t][r] *= alpha[i];
    // phase 2: O^T[channel][column] += V^T[channel][key] P^T[key][column], 32 keys at a time, 16
    // channels an MFMA.  Its A operand (lane (m, g4): channel 16 t + m of the keys 4 g4 .. + 3 and
    // 16 + 4 g4 .. + 3, the order in which the probabilities lie in pb) comes from two transposing
    // loads.  A block of 16 keys that no column of the wave sees has zero probabilities: its rows are
    // read all the same (they lie in the tile) and add nothing.
    const int tr_row = 4 * g4 + n16 / 4;  // the key row this lane points at, within 16 keys
    const int tr_ch = 4 * (n16 % 4);      // the first of its four channels, within 16 channels
#pragma unroll
    for (int g = 0; g < NS / 2; ++g) {
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        const int r0 = 32 * g + tr_row, r1 = r0 + 16;
        const int ch = 16 * t + tr_ch;
        const u32x2_t lo = lds_transposed(&v_lds[tile_at_v(r0, ch / 8) + ch % 8]);
        const u32x2_t hi = lds_transposed(&v_lds[tile_at_v(r1, ch / 8) + ch % 8]);
        const bf16x8_t va = __builtin_bit_cast(bf16x8_t, u32x4_t{lo[0], lo[1], hi[0], hi[1]});
#pragma unroll
        for (int i = 0; i < NC; ++i) acc[i][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb[i][g], acc[i][t], 0, 0, 0);
      }
    }
    }
  };
  // Tiles that lie wholly before the tile's first query (and after no window's edge) are seen by all
  // columns of the block: they run in a loop of their own, without masks.  The two loops are code
  // one after the other, not two arms of a branch inside one loop, which is what keeps the register
  // count where it was.
  // Every wave of the block passes the same number of barriers: with two groups both make as many
  // steps, and the second one's last tile may lie past the last key (then it only waits and loads).
  const int n_steps = ((key_hi - tile_begin) / KT + GROUPS) / GROUPS;
  int base = tile_begin + grp * KT;
  int step = 0;
  if (!WINDOWED) {
    for (; step < n_steps && base + KT - 1 <= pos0 + q0; ++step, base += GROUPS * KT, buffer ^= 1)
      work_tile(base, std::false_type{});
  }
  for (; step < n_steps; ++step, base += GROUPS * KT, buffer ^= 1) work_tile(base, std::true_type{});

  if constexpr (GROUPS == 2) {
    // The second group hands its maxima, sums and outputs to the first through the memory of the
    // tiles (nobody reads a tile any more, and the last, unused load has landed).  Value i of thread
    // t lies at i * 256 + t: consecutive lanes, consecutive words.
    constexpr int kPerLane = NC * (2 + 4 * DT);
    static_assert(kPerLane * kWaves * kWave * sizeof(float) <= GROUPS * 4 * kTileElems * sizeof(bf16_t),
                  "the tiles' memory is too small for the exchange");
    float* xch = reinterpret_cast<float*>(tile_memory<GROUPS>()) + (wave * kWave + lane);
    constexpr int kStride = kWaves * kWave;
    wait_for_loads();
    __syncthreads();
    if (grp == 1) {
#pragma unroll
      for (int i = 0; i < NC; ++i) {
        float* x = xch + i * (2 + 4 * DT) * kStride;
        x[0] = m_run[i];
        x[kStride] = l_part[i];
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
          for (int r = 0; r < 4; ++r) x[(2 + 4 * t + r) * kStride] = acc[i][t][r];
      }
    }
    __syncthreads();
    if (grp == 1) return;
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const float* x = xch + i * (2 + 4 * DT) * kStride;
      const float m_other = x[0];
      const float m_new = fmaxf(m_run[i], m_other);
      // a group that has met no visible key of a column has maximum -inf and nothing to add
      const float mine = m_run[i] == -INFINITY ? 0.f : exp2_fast(m_run[i] - m_new);
      const float other = m_other == -INFINITY ? 0.f : exp2_fast(m_other - m_new);
      l_part[i] = l_part[i] * mine + x[kStride] * other;
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][t][r] = acc[i][t][r] * mine + x[(2 + 4 * t + r) * kStride] * other;
    }
  }

#pragma unroll
  for (int i = 0; i < NC; ++i) {
    float l = l_part[i];
    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    if (!col_ok[i]) continue;
    const float inv = 1.0f / l;
    bf16_t* orow = a.out + (size_t)col_tok[i] * a.out_stride + (size_t)col_head[i] * DH;
    // acc[i][t][r] is channel 16 t + 4 g4 + r: four consecutive channels per output block
#pragma unroll
    for (int t = 0; t < DT; ++t)
      *reinterpret_cast<u32x2_t*>(orow + 16 * t + 4 * g4) =
          u32x2_t{pack_bf16x2(acc[i][t][0] * inv, acc[i][t][1] * inv), pack_bf16x2(acc[i][t][2] * inv, acc[i][t][3] * inv)};
  }
}

}  // namespace

TL_EXPORT int tl_attn_prefill_head_dim() { return DH; }

// Columns of one block: a tile holds tl_attn_prefill_block_cols() / RP queries, RP = the number of
// query heads per kv head rounded up to a power of two.
TL_EXPORT int tl_attn_prefill_block_cols() { return kCols; }

// q: element (t, h, d) at q + t*q_stride + h*DH + d, token t counted as in qo_indptr; out likewise.
// Pages [page][Hkv][page_size][DH].  Row r holds tokens qo_indptr[r]..qo_indptr[r+1]-1, which are the
// last positions of a request of kv_lens[r] tokens.  tile_row / tile_q0 list the query tiles (see above).
TL_EXPORT int tl_attn_prefill(const void* q, int q_stride, void* out, int out_stride, const void* k_pages,
                              const void* v_pages, const int32_t* qo_indptr, const int32_t* kv_lens,
                              const int32_t* block_table, int bt_stride, const int32_t* tile_row,
                              const int32_t* tile_q0, int n_tiles, int n_q_heads, int n_kv_heads, int head_dim,
                              int page_size, int window, float scale, int key_groups, hipStream_t stream) {
  if (head_dim != DH) return variant_fail(TL_ERR_ARG, "attn_prefill: built for head_dim %d, called with %d", DH, head_dim);
  if (n_tiles < 0 || n_q_heads <= 0 || n_kv_heads <= 0 || page_size <= 0 || bt_stride <= 0 || window < 0)
    return variant_fail(TL_ERR_ARG, "attn_prefill: bad sizes");
  if (n_q_heads % n_kv_heads) return variant_fail(TL_ERR_ARG, "attn_prefill: %d query heads are not a multiple of %d kv heads", n_q_heads, n_kv_heads);
  const int R = n_q_heads / n_kv_heads;
  if (R > 16) return variant_fail(TL_ERR_UNSUPPORTED, "attn_prefill: %d query heads per kv head exceed 16", R);
  if (n_tiles > 65535) return variant_fail(TL_ERR_UNSUPPORTED, "attn_prefill: %d query tiles exceed a launch's 65535", n_tiles);
  // the running maximum is taken over raw scores and scaled afterwards
  if (!(scale > 0.f)) return variant_fail(TL_ERR_UNSUPPORTED, "attn_prefill: softmax scale %g must be positive", (double)scale);
  if (q_stride % 8 || ((uintptr_t)q % 16) || out_stride % 8 || ((uintptr_t)out % 16))
    return variant_fail(TL_ERR_ARG, "attn_prefill: queries and outputs need 16-byte aligned rows");
  if (key_groups != 1 && key_groups != 2) return variant_fail(TL_ERR_ARG, "attn_prefill: key_groups must be 1 or 2, got %d", key_groups);
  if (n_tiles == 0) return TL_OK;
  PrefillArgs a;
  a.q = (const bf16_t*)q; a.q_stride = q_stride; a.out = (bf16_t*)out; a.out_stride = out_stride;
  a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages;
  a.qo_indptr = qo_indptr; a.kv_lens = kv_lens; a.block_table = block_table; a.bt_stride = bt_stride;
  a.tile_row = tile_row; a.tile_q0 = tile_q0;
  a.n_kv_heads = n_kv_heads; a.group = R; a.page_size = page_size; a.window = window;
  a.page_shift = -1;
  for (int sh = 0; sh < 31; ++sh)
    if ((1 << sh) == page_size) a.page_shift = sh;
  a.scale_log2e = scale * 1.4426950408889634f;
  dim3 grid(n_kv_heads, n_tiles);  // consecutive blocks share a query tile: their loads of q overlap
  const bool windowed = window > 0;
  const int threads = kWaves * kWave;
#define TL_PREFILL_LAUNCH(rp)                                                                      \
  do {                                                                                             \
    if (key_groups == 2) {                                                                         \
      if (windowed) attn_prefill_kernel<rp, true, 2><<<grid, 2 * threads, 0, stream>>>(a);         \
      else attn_prefill_kernel<rp, false, 2><<<grid, 2 * threads, 0, stream>>>(a);                 \
    } else {                                                                                       \
      if (windowed) attn_prefill_kernel<rp, true, 1><<<grid, threads, 0, stream>>>(a);             \
      else attn_prefill_kernel<rp, false, 1><<<grid, threads, 0, stream>>>(a);                     \
    }                                                                                              \
  } while (0)
  if (R == 1) TL_PREFILL_LAUNCH(1);
  else if (R == 2) TL_PREFILL_LAUNCH(2);
  else if (R <= 4) TL_PREFILL_LAUNCH(4);
  else if (R <= 8) TL_PREFILL_LAUNCH(8);
  else TL_PREFILL_LAUNCH(16);
#undef TL_PREFILL_LAUNCH
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return variant_fail(TL_ERR_HIP, "attn_prefill: %s", hipGetErrorString(e));
  return TL_OK;
}
