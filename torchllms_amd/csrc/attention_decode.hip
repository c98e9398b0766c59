// Attention of single new tokens over their requests' paged bfloat16 keys and values: the decode
// kernel.  The work is reading the cache, so the design goal is to keep many wide loads in flight
// with few registers per wave (more resident waves = more bytes in flight):
//
//   * grid (split, kv head, token): the keys of one (token, kv head) are cut into splits of
//     `split_size` keys so that a small batch still fills 256 CUs; a second kernel merges the
//     splits' partial results with their running maxima and sums (all 32-bit).
//   * a block has 4 waves; wave w takes the 16-key tiles w, w+4, ... of the split.  All query heads
//     that share the kv head are handled together, so keys and values are read once for the group.
//   * scores: S^T[16 keys x 16 heads] by MFMA 16x16x16 bf16, A = the key rows exactly as they lie
//     in the page (each lane loads 16-byte pieces of one row), B = the queries, kept in registers.
//   * softmax statistics in 32-bit on the MFMA's output layout.  That layout (lane = head, four
//     consecutive keys) is also the B operand layout of P^T, so the probabilities go to the second
//     product without leaving their lane.
//   * values: O^T[channels x heads] = V^T . P^T by MFMA.  A lane loads, from each of its four key
//     rows, the DH/16 consecutive channels  (DH/16) * n16 ...; the A operand of output block b is
//     channel b of the four rows (two byte permutes).  Output block b, row m is therefore channel
//     (DH/16) * m + b: a fixed renaming that the final store undoes.
//
// Compiled once per head size (-DTL_HEAD_DIM=32|64|128|256); any number 1..16 of query heads per kv
// head runs through the same kernel (unused MFMA columns compute on zero queries).
#include <stdarg.h>
#include <stdio.h>

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
static_assert(DH == 32 || DH == 64 || DH == 128 || DH == 256, "decode kernel: head size 32, 64, 128 or 256");

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kTile = 16;             // keys per tile = MFMA M
#ifndef TL_DECODE_WAVES
#define TL_DECODE_WAVES 4
#endif
#ifndef TL_DECODE_MIN_WAVES
#define TL_DECODE_MIN_WAVES (TL_HEAD_DIM <= 128 ? 4 : 2)  // blocks per CU the register budget is cut for
#endif
constexpr int kWaves = TL_DECODE_WAVES;
constexpr int kKLoads = DH / 32;      // 16-byte loads a lane makes of its key row
constexpr int kE = DH / 16;           // channels of a value row that one lane owns = output blocks
constexpr int kVDwords = kE / 2;      // 32-bit words a lane loads from one value row

struct DecodeArgs {
  const bf16_t* q;
  int q_stride;
  bf16_t* out;
  int out_stride;
  const bf16_t* k_pages;
  const bf16_t* v_pages;
  const int32_t* token_seq;
  const int32_t* positions;
  const int32_t* block_table;
  int bt_stride;
  int n_kv_heads;
  int group;  // query heads per kv head
  int page_size;
  int page_shift;  // log2(page_size) when that is a power of two, else -1
  int window;
  float scale_log2e;  // softmax scale * log2(e): probabilities are exp2 of scaled differences
  int split_size;     // keys per split, a multiple of 64
  int n_splits;
  float* ws_o;   // [token][q head][split][DH]
  float* ws_ml;  // [token][q head][split][2] = running maximum (log2 domain), sum
};

struct Pack16 {
  u32x4_t u;
  __device__ __forceinline__ short4_t half(int e) const {
    return __builtin_bit_cast(short4_t, e == 0 ? u32x2_t{u[0], u[1]} : u32x2_t{u[2], u[3]});
  }
};

__device__ __forceinline__ uint32_t bf16_bits(float x) {
  return (uint32_t)__builtin_bit_cast(uint16_t, from_f32<bf16_t>(x));
}
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) { return bf16_bits(a) | (bf16_bits(b) << 16); }

// kVDwords consecutive 32-bit words from a pointer aligned to their total size
__device__ __forceinline__ void load_value_words(const bf16_t* src, uint32_t* dst) {
  if constexpr (kVDwords == 1) {
    dst[0] = *reinterpret_cast<const uint32_t*>(src);
  } else if constexpr (kVDwords == 2) {
    const u32x2_t v = *reinterpret_cast<const u32x2_t*>(src);
    dst[0] = v[0];
    dst[1] = v[1];
  } else {
#pragma unroll
    for (int i = 0; i < kVDwords / 4; ++i) {
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(src + 8 * i);
#pragma unroll
      for (int e = 0; e < 4; ++e) dst[4 * i + e] = v[e];
    }
  }
}

// kPow2Pages: the page size is a power of two, so a key's page and offset are a shift and a mask;
// the general kernel divides, inlined at each of the 25 places that look a page up (6.6 KB of code
// against 4.7).  Both run at the same speed; they are two kernels so that neither carries the
// other's code and branches.
template <bool kPow2Pages>
__global__ void __launch_bounds__(kWaves* kWave, TL_DECODE_MIN_WAVES) attn_decode_kernel(DecodeArgs a) {
  extern __shared__ float red_o[];  // [kWaves][group][DH]: per-wave partial outputs for the block merge
  __shared__ float red_m[kWaves][16], red_l[kWaves][16];

  const int kvh = blockIdx.y;
  const int t = blockIdx.z;
  // Blocks go to the eight XCDs in turn by their linear index, and a request's later splits are
  // short or empty when requests differ in length.  Taken as blockIdx.x alone, split s of every
  // (token, head) would land on the same XCDs (all of them, when the number of splits divides 8):
  // some XCDs would get the full splits and others the empty ones.  Rotating by head and token
  // spreads each split index over all XCDs.
  const int split = (blockIdx.x + blockIdx.y + blockIdx.z) % a.n_splits;
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int n16 = lane % 16;  // MFMA column: head within the group; also the key row this lane loads
  const int g4 = lane / 16;   // MFMA row group

  const int b = a.token_seq[t];
  const int p = a.positions[t];
  const int lo = (a.window > 0 && p - a.window + 1 > 0) ? p - a.window + 1 : 0;
  const int lo_al = lo & ~(kTile - 1);
  const int split_begin = lo_al + split * a.split_size;
  if (split_begin > p) return;  // whole block: nothing in this split
  const int split_end = min(split_begin + a.split_size - 1, p);  // last key, inclusive
  const int32_t* bt = a.block_table + (size_t)b * a.bt_stride;
  const int R = a.group;
  const size_t head_elems = (size_t)a.page_size * DH;

  // queries of the group as B operands: lane (n16, g4), slice s = 2u + e holds q[n16][32u + 8 g4 + 4e + j]
  Pack16 qreg[kKLoads];
  {
    const bf16_t* qrow = a.q + (size_t)t * a.q_stride + ((size_t)kvh * R + (n16 < R ? n16 : 0)) * DH;
#pragma unroll
    for (int u = 0; u < kKLoads; ++u) {
      qreg[u].u = *reinterpret_cast<const u32x4_t*>(qrow + 32 * u + 8 * g4);
      if (n16 >= R) qreg[u].u = u32x4_t{0, 0, 0, 0};
    }
  }

  float m_run = -INFINITY;  // running maximum of head n16 (same in the four g4 lanes)
  float l_part = 0.f;       // sum of this lane's own probabilities
  float4_t acc[kE];         // acc[b][i]: head n16, channel kE * (4 g4 + i) + b
#pragma unroll
  for (int e = 0; e < kE; ++e) acc[e] = float4_t{0.f, 0.f, 0.f, 0.f};

  // Keys are clamped to the split's own range: the prefetch that runs past the split's end then
  // reads one row that the block has read already, not rows of the next split, which another block
  // reads (a quarter more traffic at splits of 256 keys).
  auto clamp_key = [&](int key) { return key < lo ? lo : (key > split_end ? split_end : key); };
  auto block_of = [&](int key) { return kPow2Pages ? key >> a.page_shift : key / a.page_size; };
  auto offset_of = [&](int key) { return kPow2Pages ? key & (a.page_size - 1) : key % a.page_size; };
  auto row_ptr = [&](const bf16_t* pages, int page, int key) {
    return pages + ((size_t)page * a.n_kv_heads + kvh) * head_elems + (size_t)offset_of(key) * DH;
  };

  // The page ids of a tile's rows: one for the lane's key row, four for its value rows.  They are
  // fetched from the block table a tile before the rows themselves, so that a row's load waits for
  // one trip to memory, not for two in a row (at small batches a tile is worked off faster than that).
  struct TilePages {
    int32_t k;
    int32_t v[4];
  };
  auto fetch_pages = [&](int base) {
    TilePages tp;
    tp.k = bt[block_of(clamp_key(base + n16))];
#pragma unroll
    for (int j = 0; j < 4; ++j) tp.v[j] = bt[block_of(clamp_key(base + 4 * g4 + j))];
    return tp;
  };

  // The compiler may not move a load across this: without it, it sinks the prefetches of the next
  // tile down to their first use, at the top of the next pass, and every tile waits a whole trip
  // to memory.
  auto keep_loads_here = [] { asm volatile("" ::: "memory"); };

  // Rolling prefetch: the keys of tile t+1 are requested as soon as the MFMAs of tile t have read
  // their registers, the values of tile t+1 as soon as the value operands of tile t are packed, so
  // one set of registers per operand keeps a load in flight at all times.  The prefetches are not
  // put under a branch (a conditional load makes the compiler's wait before the next use cover both
  // paths and so wait for the prefetch itself); past the end of the split they read the split's
  // last key again, which nobody uses.
  Pack16 kreg[kKLoads];
  uint32_t vreg[4][kVDwords];
  auto load_k = [&](int base, const TilePages& tp) {
    const bf16_t* kr = row_ptr(a.k_pages, tp.k, clamp_key(base + n16));
#pragma unroll
    for (int u = 0; u < kKLoads; ++u) kreg[u].u = *reinterpret_cast<const u32x4_t*>(kr + 32 * u + 8 * g4);
  };
  auto load_v = [&](int base, const TilePages& tp) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      load_value_words(row_ptr(a.v_pages, tp.v[j], clamp_key(base + 4 * g4 + j)) + kE * n16, vreg[j]);
  };

  int base = split_begin + wave * kTile;
  TilePages pages_next = fetch_pages(base + kWaves * kTile);
  if (base <= split_end) {
    const TilePages pages_now = fetch_pages(base);
    load_k(base, pages_now);
    load_v(base, pages_now);
    keep_loads_here();
  }
  for (; base <= split_end; base += kWaves * kTile) {
    const int next = base + kWaves * kTile;

    // scores S^T[key][head]
    float4_t c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < kKLoads; ++u) {
      c = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kreg[u].half(0), qreg[u].half(0), c, 0, 0, 0);
      c = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kreg[u].half(1), qreg[u].half(1), c, 0, 0, 0);
    }
    load_k(next, pages_next);  // unconditional: past the split's end the keys are clamped and unused
    keep_loads_here();
    float s[4];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = base + 4 * g4 + i;
      const bool valid = (key >= lo) & (key <= p);  // bit operation: no branch behind the MFMAs
      s[i] = valid ? c[i] * a.scale_log2e : -INFINITY;
      tmax = fmaxf(tmax, s[i]);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
    const float m_new = fmaxf(m_run, tmax);  // finite: every tile holds at least one valid key
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    float pr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pr[i] = __builtin_amdgcn_exp2f(s[i] - m_new);  // exp2(-inf) = 0 for masked keys
      l_part = (i == 0 ? l_part * alpha : l_part) + pr[i];
    }
    m_run = m_new;
    const short4_t pop = __builtin_bit_cast(short4_t, u32x2_t{pack_bf16x2(pr[0], pr[1]), pack_bf16x2(pr[2], pr[3])});

    // O^T += V^T . P^T, block by block of 16 channels
#pragma unroll
    for (int e = 0; e < kE; ++e) {
      const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;  // the odd or the even halves of two words
      const uint32_t lo2 = __builtin_amdgcn_perm(vreg[1][e / 2], vreg[0][e / 2], sel);
      const uint32_t hi2 = __builtin_amdgcn_perm(vreg[3][e / 2], vreg[2][e / 2], sel);
      const short4_t vop = __builtin_bit_cast(short4_t, u32x2_t{lo2, hi2});
      acc[e] = acc[e] * alpha;
      acc[e] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vop, pop, acc[e], 0, 0, 0);
    }
    load_v(next, pages_next);
    keep_loads_here();
    pages_next = fetch_pages(next + kWaves * kTile);  // for the tile after the next
    keep_loads_here();
  }

  // the lane's own sums join over the four row groups
  l_part += __shfl_xor(l_part, 16, kWave);
  l_part += __shfl_xor(l_part, 32, kWave);
  if (lane < 16) {
    red_m[wave][n16] = m_run;
    red_l[wave][n16] = l_part;
  }
  if (n16 < R) {
#pragma unroll
    for (int e = 0; e < kE; ++e)
#pragma unroll
      for (int i = 0; i < 4; ++i) red_o[((size_t)wave * R + n16) * DH + kE * (4 * g4 + i) + e] = acc[e][i];
  }
  __syncthreads();

  // block merge: thread -> (head, channel)
  for (int idx = threadIdx.x; idx < R * DH; idx += kWaves * kWave) {
    const int h = idx / DH;
    const int d = idx % DH;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) M = fmaxf(M, red_m[w][h]);
    float L = 0.f, O = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float f = red_m[w][h] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(red_m[w][h] - M);
      L += red_l[w][h] * f;
      O += red_o[((size_t)w * R + h) * DH + d] * f;
    }
    const int qh = kvh * R + h;
    if (a.n_splits == 1) {
      a.out[(size_t)t * a.out_stride + (size_t)qh * DH + d] = from_f32<bf16_t>(O / L);
    } else {
      const size_t slot = ((size_t)t * a.n_kv_heads * R + qh) * a.n_splits + split;
      a.ws_o[slot * DH + d] = O;
      if (d == 0) {
        a.ws_ml[slot * 2] = M;
        a.ws_ml[slot * 2 + 1] = L;
      }
    }
  }
}

// Merge of the splits: one wave per (token, query head); lane -> channels.  The kernel runs between
// two large ones, where every load misses all caches, and is as long as its chain of dependent loads:
// so the token's position, the statistics of the first 64 splits (lane s: split s) and the outputs of
// the first eight are all asked for at the top, before anything is known about how many splits are
// valid (every slot of the workspace exists; what an invalid one holds is not used).  Each output
// still adds its splits in ascending order.
__global__ void __launch_bounds__(kWave) attn_decode_merge_kernel(DecodeArgs a, int n_q_heads) {
  constexpr int NC = (DH + kWave - 1) / kWave;
  constexpr int kAhead = 8;  // splits whose outputs are in flight together
  const int t = blockIdx.x;
  const int qh = blockIdx.y;
  const int lane = threadIdx.x;
  const size_t slot0 = ((size_t)t * n_q_heads + qh) * a.n_splits;
  const int p = a.positions[t];
  const int mine = min(lane, a.n_splits - 1);
  const float m_mine = a.ws_ml[(slot0 + mine) * 2];
  const float l_mine = a.ws_ml[(slot0 + mine) * 2 + 1];
  float v[kAhead][NC];
  auto fetch = [&](int first) {
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const size_t at = (slot0 + min(first + u, a.n_splits - 1)) * DH;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int d = lane + c * kWave;
        v[u][c] = a.ws_o[at + (d < DH ? d : 0)];
      }
    }
  };
  fetch(0);
  const int lo = (a.window > 0 && p - a.window + 1 > 0) ? p - a.window + 1 : 0;
  const int lo_al = lo & ~(kTile - 1);
  const int n_valid = min((p - lo_al) / a.split_size + 1, a.n_splits);
  float M = lane < n_valid ? m_mine : -INFINITY;
  for (int s = lane + kWave; s < n_valid; s += kWave) M = fmaxf(M, a.ws_ml[(slot0 + s) * 2]);
  M = wave_max(M);
  float L = lane < n_valid ? l_mine * __builtin_amdgcn_exp2f(m_mine - M) : 0.f;
  for (int s = lane + kWave; s < n_valid; s += kWave)
    L += a.ws_ml[(slot0 + s) * 2 + 1] * __builtin_amdgcn_exp2f(a.ws_ml[(slot0 + s) * 2] - M);
  L = wave_sum(L);
  float o[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) o[c] = 0.f;
  for (int s = 0; s < n_valid; s += kAhead) {
    if (s > 0) fetch(s);
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const int split = s + u;
      // the split's maximum: from the lane that holds it, or from memory past the first 64
      const float m_u = split < kWave ? __shfl(m_mine, split, kWave) : a.ws_ml[(slot0 + min(split, a.n_splits - 1)) * 2];
      const float w = split < n_valid ? __builtin_amdgcn_exp2f(m_u - M) : 0.f;
#pragma unroll
      for (int c = 0; c < NC; ++c) o[c] += split < n_valid ? v[u][c] * w : 0.f;
    }
  }
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int d = lane + c * kWave;
    if (d < DH) a.out[(size_t)t * a.out_stride + (size_t)qh * DH + d] = from_f32<bf16_t>(o[c] / L);
  }
}

}  // namespace

TL_EXPORT int tl_attn_decode_head_dim() { return DH; }

// q: element (t, h, d) at q + t*q_stride + h*DH + d; out likewise.  Pages [page][Hkv][page_size][DH].
// Every token is one query at positions[t] of request row token_seq[t].  split_size: keys per
// split (a multiple of 64); n_splits >= ceil(longest visible range / split_size), counted from the
// 16-aligned first visible key.  ws_o / ws_ml: workspaces (unused when n_splits == 1).
TL_EXPORT int tl_attn_decode(const void* q, int q_stride, void* out, int out_stride, const void* k_pages,
                             const void* v_pages, const int32_t* token_seq, const int32_t* positions,
                             const int32_t* block_table, int bt_stride, int n_tokens, int n_q_heads,
                             int n_kv_heads, int head_dim, int page_size, int window, float scale,
                             int split_size, int n_splits, float* ws_o, float* ws_ml, hipStream_t stream) {
  if (head_dim != DH) return variant_fail(TL_ERR_ARG, "attn_decode: built for head_dim %d, called with %d", DH, head_dim);
  if (n_tokens < 0 || n_q_heads <= 0 || n_kv_heads <= 0 || page_size <= 0 || bt_stride <= 0 || window < 0)
    return variant_fail(TL_ERR_ARG, "attn_decode: bad sizes");
  if (n_q_heads % n_kv_heads) return variant_fail(TL_ERR_ARG, "attn_decode: %d query heads are not a multiple of %d kv heads", n_q_heads, n_kv_heads);
  const int R = n_q_heads / n_kv_heads;
  constexpr int kMaxGroup = DH <= 128 ? 16 : 8;  // bounded by the block's LDS (64 KB of partial outputs)
  if (R > kMaxGroup) return variant_fail(TL_ERR_UNSUPPORTED, "attn_decode: %d query heads per kv head exceed %d at head_dim %d", R, kMaxGroup, DH);
  if (split_size <= 0 || split_size % (kWaves * kTile)) return variant_fail(TL_ERR_ARG, "attn_decode: split_size=%d must be a positive multiple of %d", split_size, kWaves * kTile);
  if (n_splits <= 0 || n_splits > 65535 || n_kv_heads > 65535 || n_tokens > 65535) return variant_fail(TL_ERR_ARG, "attn_decode: grid out of range");
  if (n_splits > 1 && (!ws_o || !ws_ml)) return variant_fail(TL_ERR_ARG, "attn_decode: workspaces missing");
  if (q_stride % 8 || ((uintptr_t)q % 16)) return variant_fail(TL_ERR_ARG, "attn_decode: queries must be 16-byte aligned with a row stride that is a multiple of 8");
  if (n_tokens == 0) return TL_OK;
  DecodeArgs a;
  a.q = (const bf16_t*)q; a.q_stride = q_stride; a.out = (bf16_t*)out; a.out_stride = out_stride;
  a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages;
  a.token_seq = token_seq; a.positions = positions; a.block_table = block_table; a.bt_stride = bt_stride;
  a.n_kv_heads = n_kv_heads; a.group = R; a.page_size = page_size; a.window = window;
  a.page_shift = -1;
  for (int sh = 0; sh < 31; ++sh)
    if ((1 << sh) == page_size) a.page_shift = sh;
  a.scale_log2e = scale * 1.4426950408889634f;
  a.split_size = split_size; a.n_splits = n_splits; a.ws_o = ws_o; a.ws_ml = ws_ml;
  dim3 grid(n_splits, n_kv_heads, n_tokens);
  const int threads = kWaves * kWave;
  const size_t lds = (size_t)kWaves * R * DH * sizeof(float);
  if (a.page_shift >= 0)
    attn_decode_kernel<true><<<grid, threads, lds, stream>>>(a);
  else
    attn_decode_kernel<false><<<grid, threads, lds, stream>>>(a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return variant_fail(TL_ERR_HIP, "attn_decode: %s", hipGetErrorString(e));
  if (n_splits > 1) {
    attn_decode_merge_kernel<<<dim3(n_tokens, n_q_heads), kWave, 0, stream>>>(a, n_q_heads);
    e = hipGetLastError();
    if (e != hipSuccess) return variant_fail(TL_ERR_HIP, "attn_decode merge: %s", hipGetErrorString(e));
  }
  return TL_OK;
}
