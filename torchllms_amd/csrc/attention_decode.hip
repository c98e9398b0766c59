// Attention of single new tokens over their requests' paged bfloat16 keys and values: the decode
// kernel.  The work is reading the cache, so the design goal is to keep many wide loads in flight:
//
//   * grid (split, kv head, token): the keys of one (token, kv head) are cut into splits of
//     `split_size` keys so that a small batch still fills 256 CUs; a second kernel merges the
//     splits' partial results with their running maxima and sums (all 32-bit).
//   * a block has 4 waves; wave w takes the 16-key tiles w, w+4, ... of the split.  All query heads
//     that share the kv head are handled together, so keys and values are read once for the group.
//   * scores: S^T[16 keys x 16 heads] by MFMA 16x16x16 bf16, A = the key rows exactly as they lie
//     in the page (each lane loads 16-byte pieces of one row), B = the queries, kept in registers.
//   * softmax statistics in 32-bit on the MFMA's output layout; the probabilities cross to the
//     value layout through a small per-wave LDS buffer.
//   * values: each lane loads 16 bytes (8 channels) of a value row; P.V accumulates in 32-bit
//     registers on the vector ALU, which has time to spare while the loads stream.
//
// Compiled once per head size (-DTL_HEAD_DIM=32|64|128|256); the number of query heads per kv head
// (1..16) is a template parameter rounded up to a power of two.
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

constexpr int kTile = 16;             // keys per tile = MFMA M
#ifndef TL_DECODE_WAVES
#define TL_DECODE_WAVES 4
#endif
constexpr int kWaves = TL_DECODE_WAVES;
constexpr int kKLoads = DH / 32;      // 16-byte loads a lane makes of its key row
constexpr int kLPR = DH / 8;          // lanes that cover one value row with 16-byte loads
constexpr int kRPI = kWave / kLPR;    // value rows one load instruction covers
constexpr int kVLoads = kTile / kRPI; // load instructions per tile of values
static_assert(kRPI <= kTile, "head size too small for this layout");

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

union Pack16 {
  uint4 u;
  short4_t s[2];
  uint16_t h[8];
};

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }

template <int RP>
__global__ void __launch_bounds__(kWaves* kWave) attn_decode_kernel(DecodeArgs a) {
  __shared__ float p_lds[kWaves][kTile][RP];            // probabilities of the wave's current tile
  __shared__ float red_o[kWaves][RP][DH];               // per-wave partial outputs for the block merge
  __shared__ float red_m[kWaves][RP], red_l[kWaves][RP];

  const int split = blockIdx.x;
  const int kvh = blockIdx.y;
  const int t = blockIdx.z;
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
      qreg[u].u = *reinterpret_cast<const uint4*>(qrow + 32 * u + 8 * g4);
      if (n16 >= R) qreg[u].u = make_uint4(0, 0, 0, 0);
    }
  }

  float m_run = -INFINITY;  // running maximum of head n16 (same in the four g4 lanes)
  float l_part = 0.f;       // sum of this lane's own probabilities
  float acc[RP][8];
#pragma unroll
  for (int h = 0; h < RP; ++h)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[h][e] = 0.f;

  const int vrow = lane / kLPR;
  const int dchunk = lane % kLPR;

  auto clamp_key = [&](int key) { return key < lo ? lo : (key > p ? p : key); };
  auto row_ptr = [&](const bf16_t* pages, int key) {
    const int blk = a.page_shift >= 0 ? key >> a.page_shift : key / a.page_size;
    const int off = a.page_shift >= 0 ? key & (a.page_size - 1) : key % a.page_size;
    return pages + ((size_t)bt[blk] * a.n_kv_heads + kvh) * head_elems + (size_t)off * DH;
  };

  // Rolling prefetch: the keys of tile t+1 are requested as soon as the MFMAs of tile t have read
  // their registers, the values of tile t+1 as soon as P.V of tile t is done, so one set of
  // registers per operand keeps a load in flight at all times.
  Pack16 kreg[kKLoads];
  Pack16 vreg[kVLoads];
  auto load_k = [&](int base, Pack16* kd) {
    const bf16_t* kr = row_ptr(a.k_pages, clamp_key(base + n16));
#pragma unroll
    for (int u = 0; u < kKLoads; ++u) kd[u].u = *reinterpret_cast<const uint4*>(kr + 32 * u + 8 * g4);
  };
  auto load_v = [&](int base, Pack16* vd) {
#pragma unroll
    for (int j = 0; j < kVLoads; ++j) {
      const bf16_t* vr = row_ptr(a.v_pages, clamp_key(base + j * kRPI + vrow));
      vd[j].u = *reinterpret_cast<const uint4*>(vr + 8 * dchunk);
    }
  };

  int base = split_begin + wave * kTile;
  if (base <= split_end) {
    load_k(base, kreg);
    load_v(base, vreg);
  }
  for (; base <= split_end; base += kWaves * kTile) {
    const int next = base + kWaves * kTile;

    // scores S^T[key][head]
    float4_t c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < kKLoads; ++u) {
      c = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kreg[u].s[0], qreg[u].s[0], c, 0, 0, 0);
      c = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kreg[u].s[1], qreg[u].s[1], c, 0, 0, 0);
    }
    if (next <= split_end) load_k(next, kreg);
    float s[4];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = base + 4 * g4 + i;
      const bool valid = key >= lo && key <= p;
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

    // probabilities and the rescale factor go to the value layout through LDS (per wave)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    if (n16 < RP) {
#pragma unroll
      for (int i = 0; i < 4; ++i) p_lds[wave][4 * g4 + i][n16] = pr[i];
    }
    // alpha of head h sits in lanes n16 == h; every lane needs all of them
    float alpha_h[RP];
#pragma unroll
    for (int h = 0; h < RP; ++h) alpha_h[h] = __shfl(alpha, h, kWave);
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();

#pragma unroll
    for (int h = 0; h < RP; ++h)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[h][e] *= alpha_h[h];
#pragma unroll
    for (int j = 0; j < kVLoads; ++j) {
      const int kt = j * kRPI + vrow;  // key within the tile
      float vf[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) vf[e] = bf16_bits_to_f32(vreg[j].h[e]);
#pragma unroll
      for (int h = 0; h < RP; ++h) {
        const float ph = p_lds[wave][kt][h];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[h][e] = fmaf(ph, vf[e], acc[h][e]);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();

    if (next <= split_end) load_v(next, vreg);
  }

  // wave-level reductions: sums over the four row groups; outputs over the value-row lanes
  l_part += __shfl_xor(l_part, 16, kWave);
  l_part += __shfl_xor(l_part, 32, kWave);
#pragma unroll
  for (int off = kLPR; off < kWave; off <<= 1)
#pragma unroll
    for (int h = 0; h < RP; ++h)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[h][e] += __shfl_xor(acc[h][e], off, kWave);

  if (lane < 16 && n16 < RP) {
    red_m[wave][n16] = m_run;
    red_l[wave][n16] = l_part;
  }
  if (vrow == 0) {
#pragma unroll
    for (int h = 0; h < RP; ++h)
#pragma unroll
      for (int e = 0; e < 8; ++e) red_o[wave][h][8 * dchunk + e] = acc[h][e];
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
      O += red_o[w][h][d] * f;
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

// Merge of the splits: one wave per (token, query head); lane -> channels.
__global__ void __launch_bounds__(kWave) attn_decode_merge_kernel(DecodeArgs a, int n_q_heads) {
  const int t = blockIdx.x;
  const int qh = blockIdx.y;
  const int lane = threadIdx.x;
  const int p = a.positions[t];
  const int lo = (a.window > 0 && p - a.window + 1 > 0) ? p - a.window + 1 : 0;
  const int lo_al = lo & ~(kTile - 1);
  const int n_valid = min((p - lo_al) / a.split_size + 1, a.n_splits);
  const size_t slot0 = ((size_t)t * n_q_heads + qh) * a.n_splits;
  // lane s (and s + 64, ...) reads the statistics of split s; the maximum is reduced over the wave
  float M = -INFINITY;
  for (int s = lane; s < n_valid; s += kWave) M = fmaxf(M, a.ws_ml[(slot0 + s) * 2]);
  M = wave_max(M);
  float L = 0.f;
  for (int s = lane; s < n_valid; s += kWave)
    L += a.ws_ml[(slot0 + s) * 2 + 1] * __builtin_amdgcn_exp2f(a.ws_ml[(slot0 + s) * 2] - M);
  L = wave_sum(L);
  constexpr int NC = (DH + kWave - 1) / kWave;
  float o[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) o[c] = 0.f;
  int s = 0;
  for (; s + 4 <= n_valid; s += 4) {  // four splits' loads in flight at a time
    float f[4], v[4][NC];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      f[u] = a.ws_ml[(slot0 + s + u) * 2];
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int d = lane + c * kWave;
        v[u][c] = d < DH ? a.ws_o[(slot0 + s + u) * DH + d] : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float w = __builtin_amdgcn_exp2f(f[u] - M);
#pragma unroll
      for (int c = 0; c < NC; ++c) o[c] += v[u][c] * w;
    }
  }
  for (; s < n_valid; ++s) {
    const float w = __builtin_amdgcn_exp2f(a.ws_ml[(slot0 + s) * 2] - M);
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d = lane + c * kWave;
      if (d < DH) o[c] += a.ws_o[(slot0 + s) * DH + d] * w;
    }
  }
#pragma unroll
  for (int c = 0; c < (DH + kWave - 1) / kWave; ++c) {
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
  constexpr int kMaxGroup = DH <= 128 ? 16 : 8;  // bounded by the block's LDS
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
  if (R == 1) attn_decode_kernel<1><<<grid, threads, 0, stream>>>(a);
  else if (R == 2) attn_decode_kernel<2><<<grid, threads, 0, stream>>>(a);
  else if (R <= 4) attn_decode_kernel<4><<<grid, threads, 0, stream>>>(a);
  else if (R <= 8) attn_decode_kernel<8><<<grid, threads, 0, stream>>>(a);
  else if constexpr (kMaxGroup >= 16) attn_decode_kernel<16><<<grid, threads, 0, stream>>>(a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return variant_fail(TL_ERR_HIP, "attn_decode: %s", hipGetErrorString(e));
  if (n_splits > 1) {
    attn_decode_merge_kernel<<<dim3(n_tokens, n_q_heads), kWave, 0, stream>>>(a, n_q_heads);
    e = hipGetLastError();
    if (e != hipSuccess) return variant_fail(TL_ERR_HIP, "attn_decode merge: %s", hipGetErrorString(e));
  }
  return TL_OK;
}
