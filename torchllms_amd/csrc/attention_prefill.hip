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
//     read the same piece of 16 rows still meet 16 different banks.  Two buffers of keys and two of
//     values per set of waves, one barrier a tile: a tile lands one pass before it is read.
//   * within a wave the tiles run through a pipeline of three stages (scores of the next tile, softmax
//     of this one, output product of the last), so matrix cores and vector units have independent work
//     at the same time; sums of probabilities are one more MFMA row, a column's reference maximum
//     moves only when a score passes it by a margin, and masks are applied only on tiles that hold a
//     causal limit, a window's edge or the end of the keys.  Page sizes are powers of two.
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
  int page_shift;  // log2(page_size)
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
// With two groups the second one hands its results over through the same memory at the end: per
// lane and column block a maximum, a sum and the output's 4 * DT sums, as 32-bit floats.
constexpr int kExchangeBytes = NC * (2 + 4 * DT) * kWaves * kWave * 4;
template <int GROUPS>
__device__ __forceinline__ bf16_t* tile_memory() {
  constexpr int kTileBytes = GROUPS * 2 * 2 * kTileElems * 2;
  constexpr int kBytes = GROUPS == 2 && kExchangeBytes > kTileBytes ? kExchangeBytes : kTileBytes;
  __shared__ __attribute__((aligned(16))) bf16_t tiles[kBytes / 2];
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
  const int wave = wave_uniform((threadIdx.x / kWave) % kWaves);  // within the group
  const int lane = threadIdx.x % kWave;
  const int n16 = lane % 16;
  const int g4 = lane / 16;
  const int R = a.group;

  const int row = wave_uniform(a.tile_row[tile]);
  const int q0 = wave_uniform(a.tile_q0[tile]);
  const int tok0 = wave_uniform(a.qo_indptr[row]);
  const int q_len = wave_uniform(a.qo_indptr[row + 1]) - tok0;
  const int kv_len = wave_uniform(a.kv_lens[row]);
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
  float m_run[NC];
  float4_t acc[NC][DT];
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    m_run[i] = -INFINITY;
#pragma unroll
    for (int t = 0; t < DT; ++t) acc[i][t] = float4_t{0.f, 0.f, 0.f, 0.f};
  }

  // global -> LDS for one tile of keys or of values, asynchronously.  Wave load j of wave w covers rows
  // (j * kWaves + w) * kRowsPerLoad ... of the tile: lane -> (row, slot), and fetches the piece that
  // belongs in that slot.  Keys outside the visible range are clamped into it (their scores are
  // masked), so no load touches a page the request does not hold.
  // The pages of a tile's rows are looked up one pass before the loads that need them are issued
  // (`lookup`, then `dma` with what it found), so that no pass begins by waiting for its block table.
  // Rows outside the visible range (before a window's edge, behind the last key) are fetched from the
  // nearest page the request holds, at their own offset in the page: any row of a held page is memory
  // that may be read, and their scores are masked.  Addresses are a page's offset (one 64-bit
  // multiply-add per load) plus what does not depend on the page.
  const int blk_lo = key_lo >> a.page_shift, blk_hi = key_hi >> a.page_shift;
  const unsigned page_bytes = (unsigned)a.n_kv_heads * (unsigned)a.page_size * DH * 2;  // all kv heads of a page
  const char* const k_head = reinterpret_cast<const char*>(a.k_pages) + (size_t)kvh * head_elems * 2;  // this kv head's rows in page 0
  const char* const v_head = reinterpret_cast<const char*>(a.v_pages) + (size_t)kvh * head_elems * 2;
  // The rows of one wave load (64 lanes x 16 bytes: kRowsPerLoad rows) lie in one page (the host sees to
  // it that a page holds at least as many rows, and tiles start at multiples of the tile's size), so a
  // load's page is one number for the wave: it is looked up by a scalar load and the page's address is
  // scalar arithmetic; a lane adds what does not change from tile to tile (its row within the load and
  // its piece's slot).
  typedef const int32_t __attribute__((address_space(4))) * table_ptr_t;  // read-only for the kernel's life
  const table_ptr_t table = (table_ptr_t)(uintptr_t)bt;
  struct Rows {
    int page[kLoadsPerWave];
  };
  auto lookup = [&](int base, Rows& rows) {
#pragma unroll
    for (int j = 0; j < kLoadsPerWave; ++j) {
      int blk = (base + (j * kWaves + wave) * kRowsPerLoad) >> a.page_shift;
      blk = blk < blk_lo ? blk_lo : (blk > blk_hi ? blk_hi : blk);
      rows.page[j] = table[blk];
    }
  };
  auto dma = [&](int base, const Rows& rows, int buffer, bool values) {
#pragma unroll
    for (int j = 0; j < kLoadsPerWave; ++j) {
      const int first = (j * kWaves + wave) * kRowsPerLoad;
      const int r = first + lane / kPieces;
      const int piece = (lane % kPieces) ^ (values ? swizzle_v(r) : swizzle(r));
      const unsigned of_lane = (unsigned)(lane / kPieces) * (DH * 2) + 16 * piece;  // the same for every tile
      const unsigned in_page = (unsigned)((base + first) & (a.page_size - 1)) * (DH * 2);
      const char* src = (values ? v_head : k_head) + ((size_t)(unsigned)rows.page[j] * page_bytes + in_page);
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const bf16_t*>(src + of_lane),
                                       &tiles[(2 * buffer + (values ? 1 : 0)) * kTileElems + first * DH], 16, 0, 0);
    }
  };

  constexpr int NS = KT / 16;  // blocks of 16 keys in a tile
  // The tiles of keys are worked off in a pipeline of three stages, so that the matrix cores and the
  // vector units have independent work at the same time within one wave:
  //   scores of tile t+1 (MFMA)  |  softmax of tile t (vector)  |  output of tile t-1 (MFMA)
  // One pass of the loop does the softmax of tile t beside the output product of tile t-1, then the
  // rescaling of the sums beside the scores of tile t+1.  Keys are fetched two tiles ahead and values
  // as their tile's scores are computed; each lands one pass before it is read.
  float4_t c[NC][NS];                  // scores S^T of the current tile
  bf16x8_t pb_prev[NC][NS / 2];        // probabilities of the tile before, as the B operand of the output product
  float4_t acc_l[NC];                  // sums of probabilities: the output product with a row of ones as its values
#pragma unroll
  for (int i = 0; i < NC; ++i) acc_l[i] = float4_t{0.f, 0.f, 0.f, 0.f};
  const bf16x8_t ones = __builtin_bit_cast(bf16x8_t, u32x4_t{0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u});

  // scores S^T[key][column] of one tile, one MFMA chain per (16 keys, column block)
  auto scores = [&](const bf16_t* k_lds) {
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
  };

  // O^T[channel][column] += V^T[channel][key] P^T[key][column], 32 keys at a time, 16 channels an MFMA.
  // Its A operand (lane (m, g4): channel 16 t + m of the keys 4 g4 .. + 3 and 16 + 4 g4 .. + 3, the
  // order in which the probabilities lie in pb) comes from two transposing loads.  The sum of the
  // probabilities is the same product with ones for values: a few MFMAs instead of an addition per
  // score, and exactly the sum of what the output was weighted with.
  const int tr_row = 4 * g4 + n16 / 4;  // the key row this lane points at, within 16 keys
  const int tr_ch = 4 * (n16 % 4);      // the first of its four channels, within 16 channels
  auto output = [&](const bf16_t* v_lds, const bf16x8_t (&pb)[NC][NS / 2]) {
#pragma unroll
    for (int g = 0; g < NS / 2; ++g) {
#pragma unroll
      for (int i = 0; i < NC; ++i) acc_l[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pb[i][g], acc_l[i], 0, 0, 0);
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
  };

  // Softmax bookkeeping of the tile whose scores are in c, once per tile and column: mask, maximum,
  // probabilities (into pb), and alpha, the factor by which everything summed so far shrinks.
  // Scores stay unscaled; the scale enters through one fused multiply-add per element:
  // exp2(s * scale - m), with m the running maximum of s * scale.  `masked`: whether some column may
  // not see some key of the tile; where every column sees every key the tests are compiled out.
  constexpr float kSlack = 8.f;
  // scores of keys that a column does not see become -inf (plain selects, no short-circuit)
  auto mask = [&](int base) {
#pragma unroll
    for (int i = 0; i < NC; ++i)
#pragma unroll
      for (int sub = 0; sub < NS; ++sub)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key = base + 16 * sub + 4 * g4 + r;
          const bool valid = WINDOWED ? (key >= col_lo[i]) & (key <= col_pos[i]) : key <= col_pos[i];
          c[i][sub][r] = valid ? c[i][sub][r] : -INFINITY;
        }
  };
  auto softmax = [&](bf16x8_t (&pb)[NC][NS / 2], float (&alpha)[NC], bool& moved) {
    moved = false;
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      float tmax = -INFINITY;
#pragma unroll
      for (int sub = 0; sub < NS; ++sub)
#pragma unroll
        for (int r = 0; r < 4; ++r) tmax = fmaxf(tmax, c[i][sub][r]);
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
      // The reference maximum of a column only moves when a score exceeds it by more than kSlack
      // powers of two.  Until then the tile's probabilities may exceed 1, by at most 2^kSlack, which
      // costs nothing (32-bit sums, and bfloat16 keeps its relative precision), and everything summed
      // so far keeps its scale: most tiles need no rescaling at all.
      const float t_max = tmax * a.scale_log2e;  // the scale is positive
      const bool move = t_max > m_run[i] + kSlack;  // also the first visible key of a column (from -inf)
      moved |= move;
      const float m_new = move ? t_max : m_run[i];
      alpha[i] = move ? __builtin_amdgcn_exp2f(m_run[i] - m_new) : 1.f;
      // a column may not have met a visible key yet: then its scores are all -inf and nothing is added
      const float neg_m = m_new == -INFINITY ? 0.f : -m_new;
      uint32_t pw[2 * NS];
#pragma unroll
      for (int sub = 0; sub < NS; ++sub) {
        float pr[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) pr[r] = __builtin_amdgcn_exp2f(fmaf(c[i][sub][r], a.scale_log2e, neg_m));  // exp2(-inf) = 0
        pw[2 * sub] = pack_bf16x2(pr[0], pr[1]);
        pw[2 * sub + 1] = pack_bf16x2(pr[2], pr[3]);
      }
#pragma unroll
      for (int g = 0; g < NS / 2; ++g)
        pb[i][g] = __builtin_bit_cast(bf16x8_t, u32x4_t{pw[4 * g], pw[4 * g + 1], pw[4 * g + 2], pw[4 * g + 3]});
      m_run[i] = m_new;
    }
  };

  // everything summed so far follows the maxima that moved
  auto rescale = [&](const float (&alpha)[NC]) {
#pragma unroll
    for (int i = 0; i < NC; ++i) {
#pragma unroll
      for (int r = 0; r < 4; ++r) acc_l[i][r] *= alpha[i];
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][t][r] *= alpha[i];
    }
  };

  // Every wave of the block passes the same number of barriers: with two groups both make as many
  // steps, and the second one's last tile may lie past the last key (its keys are clamped and masked).
  const int n_steps = ((key_hi - tile_begin) / KT + GROUPS) / GROUPS;
  auto base_of = [&](int step) { return tile_begin + (step * GROUPS + grp) * KT; };
  auto k_tile = [&](int step) { return tiles + (2 * (step & 1)) * kTileElems; };
  auto v_tile = [&](int step) { return tiles + (2 * (step & 1) + 1) * kTileElems; };

  Rows rows_k, rows_v;  // the rows of the next pass's loads: keys of tile step + 2, values of tile step
  lookup(base_of(0), rows_v);
  lookup(base_of(1), rows_k);
  dma(base_of(0), rows_v, 0, false);  // (tile 0's keys lie where its values do)
  dma(base_of(1), rows_k, 1, false);
  lookup(base_of(2), rows_k);
  // the first pass has no tile before it: its output product runs all the same (no branch in a pass),
  // on probabilities of zero and values of zero
#pragma unroll
  for (int i = 0; i < NC; ++i)
#pragma unroll
    for (int g = 0; g < NS / 2; ++g) pb_prev[i][g] = __builtin_bit_cast(bf16x8_t, u32x4_t{0u, 0u, 0u, 0u});
  for (int e = (wave * kWave + lane) * 8; e < kTileElems; e += kWaves * kWave * 8)
    *reinterpret_cast<u32x4_t*>(&tiles[3 * kTileElems + e]) = u32x4_t{0u, 0u, 0u, 0u};  // the values' second buffer
  wait_for_loads();
  __syncthreads();
  scores(k_tile(0));

  // one pass: tile `step`'s softmax beside tile `step - 1`'s output, then the rescaling beside tile
  // `step + 1`'s scores
  auto pass = [&](int step) {
    // this wave's loads of the pass before have landed (keys of tile step + 1, values of tile step - 1);
    // after the barrier everybody's have, and everybody has finished with the buffers that this
    // pass's loads overwrite (keys of tile step, values of tile step - 2)
    wait_for_loads();
    __syncthreads();
    dma(base_of(step + 2), rows_k, step & 1, false);  // unconditional (pages are clamped): no wait has to cover a path without it
    dma(base_of(step), rows_v, step & 1, true);
    lookup(base_of(step + 3), rows_k);  // for the next pass
    lookup(base_of(step + 1), rows_v);
    bf16x8_t pb[NC][NS / 2];
    float alpha[NC];
    bool moved;
    // a tile that lies wholly before the block's first query (and behind every window's edge) is seen
    // whole by every column: no masks (the same decision for all waves of the block)
    const int base = base_of(step);
    if (base + KT - 1 > pos0 + q0 || (WINDOWED && base < window_lo(pos0 + q_last))) mask(base);
    softmax(pb, alpha, moved);
    output(v_tile(step - 1), pb_prev);
    if (__any(moved)) rescale(alpha);  // (the same for the whole wave)
    scores(k_tile(step + 1));
#pragma unroll
    for (int i = 0; i < NC; ++i)
#pragma unroll
      for (int g = 0; g < NS / 2; ++g) pb_prev[i][g] = pb[i][g];
  };
  // (One loop for all tiles.  Two loops, the first without masks for the tiles that every column sees
  // whole, cost this compiler more registers than it has: everything the pipeline carries from pass to
  // pass is then alive across both.)
  for (int step = 0; step < n_steps; ++step) pass(step);
  // the last tile's output
  wait_for_loads();
  __syncthreads();
  output(v_tile(n_steps - 1), pb_prev);
  // the sum of the probabilities of this lane's columns (every channel row of acc_l holds it)
  float l_part[NC];
#pragma unroll
  for (int i = 0; i < NC; ++i) l_part[i] = acc_l[i][0];

  if constexpr (GROUPS == 2) {
    // The second group hands its maxima, sums and outputs to the first through the memory of the
    // tiles (nobody reads a tile any more, and the last, unused load has landed).  Value i of thread
    // t lies at i * 256 + t: consecutive lanes, consecutive words.
    constexpr int kPerLane = NC * (2 + 4 * DT);
    static_assert(kPerLane * kWaves * kWave * sizeof(float) == kExchangeBytes, "the exchange is as large as tile_memory says");
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
    const float l = l_part[i];
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
  a.page_shift = 0;
  while ((1 << a.page_shift) < page_size) ++a.page_shift;
  if ((1 << a.page_shift) != page_size)
    return variant_fail(TL_ERR_UNSUPPORTED, "attn_prefill: page_size %d is no power of two", page_size);
  // (a wave fetches kRowsPerLoad rows with one instruction and looks up one page for them)
  if (page_size < kRowsPerLoad)
    return variant_fail(TL_ERR_UNSUPPORTED, "attn_prefill: pages of %d tokens are shorter than the %d rows a wave fetches at once at head size %d",
                        page_size, kRowsPerLoad, DH);
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
