// Attention over paged keys and values, plain edition: any head size up to 256, any number of
// heads and groups, 32-bit or bfloat16 storage, all arithmetic in 32-bit.  One wave per
// (token, query head).  Keys are visited in ascending position in blocks of 64 aligned to
// absolute position, so a result depends only on the query's position and the cache contents,
// never on how the step was batched.  This is the kernel of the 32-bit path and the fallback of
// the bfloat16 path for sizes the MFMA kernels refuse.
#include <limits.h>

#include "common.h"

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kMaxHeadDim = 256;
constexpr int kChanPerLane = kMaxHeadDim / kWave;
constexpr int kTileMinTokens = 32;  // steps with at least this many tokens share keys and values through LDS

// Four consecutive elements of a row as floats (the row is 16-byte aligned for float, 8-byte for bfloat16).
__device__ __forceinline__ void load4(const float* p, float (&v)[4]) {
  const float4 x = *reinterpret_cast<const float4*>(p);
  v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float (&v)[4]) {
  const uint2 x = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(x.x << 16); v[1] = __uint_as_float(x.x & 0xffff0000u);
  v[2] = __uint_as_float(x.y << 16); v[3] = __uint_as_float(x.y & 0xffff0000u);
}

// The same in two steps: the load as it comes from memory, and its elements as floats later.
template <typename T> struct Raw4;
template <> struct Raw4<float> { float4 x; };
template <> struct Raw4<bf16_t> { uint2 x; };
__device__ __forceinline__ Raw4<float> load_raw4(const float* p) { return {*reinterpret_cast<const float4*>(p)}; }
__device__ __forceinline__ Raw4<bf16_t> load_raw4(const bf16_t* p) { return {*reinterpret_cast<const uint2*>(p)}; }
__device__ __forceinline__ void unpack4(const Raw4<float>& r, float (&v)[4]) {
  v[0] = r.x.x; v[1] = r.x.y; v[2] = r.x.z; v[3] = r.x.w;
}
__device__ __forceinline__ void unpack4(const Raw4<bf16_t>& r, float (&v)[4]) {
  v[0] = __uint_as_float(r.x.x << 16); v[1] = __uint_as_float(r.x.x & 0xffff0000u);
  v[2] = __uint_as_float(r.x.y << 16); v[3] = __uint_as_float(r.x.y & 0xffff0000u);
}

// What a wave needs to know about its (token, query head).
template <typename T>
struct Query {
  const float* qs;          // the query in LDS, 32-bit
  const T* k_pages;
  const T* v_pages;
  const int32_t* bt;        // the request's block table
  int n_kv_heads, g, head_dim, page_size;
  size_t head_elems;
  int lo, p;                // the keys it sees: positions lo .. p
  float scale;
};

// One block of 64 keys (positions j0 .. j0 + 63, j0 a multiple of 64), by one wave, all in 32-bit:
//   s_j = scale * (q . k_j), products chained from channel 0 up;  m = max_j s_j;  p_j = exp(s_j - m);
//   l = sum_j p_j (butterfly order);  o[d] = sum_j p_j v_j[d], chained from the lowest visible key up.
// Lane j takes key j0 + j for the scores (its row read 4 elements at a time); then the probabilities and
// the addresses of the value rows travel from lane to lane, and every lane adds up its channels, eight
// value rows requested at a time.  VEC: head_dim is a multiple of 4 and all rows are aligned for load4.
// The block's result depends on the query, the keys and values at these positions and nothing else.
template <typename T, bool VEC>
__device__ __forceinline__ void block_partial(const Query<T>& a, int j0, int lane, float& m_b, float& l_b,
                                              float (&o_b)[kChanPerLane]) {
#pragma clang fp contract(off)  // only the fused multiply-adds written out below: the same operations wherever this is inlined
  const int j = j0 + lane;
  const bool valid = j >= a.lo && j <= a.p;
  float s = -INFINITY;
  long long row_at = 0;  // element offset of this lane's key (and value) row in the pages
  if (valid) {
    const int page = a.bt[j / a.page_size];
    row_at = (long long)(((size_t)page * a.n_kv_heads + a.g) * a.head_elems + (size_t)(j % a.page_size) * a.head_dim);
    const T* kr = a.k_pages + row_at;
    float dot = 0.f;
    if (VEC) {
      // eight pieces of the row are asked for before the first is multiplied (a piece past the row's end is
      // the row's first once more, and not used): left to itself the compiler waited for every load of a
      // bfloat16 row in turn
      constexpr int kAhead = 8;
      for (int d0 = 0; d0 < a.head_dim; d0 += 4 * kAhead) {
        Raw4<T> raw[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) raw[u] = load_raw4(kr + (d0 + 4 * u < a.head_dim ? d0 + 4 * u : 0));
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
          const int d = d0 + 4 * u;
          if (d < a.head_dim) {
            float kv[4];
            unpack4(raw[u], kv);
#pragma unroll
            for (int e = 0; e < 4; ++e) dot = fmaf(a.qs[d + e], kv[e], dot);
          }
        }
      }
    } else {
      for (int d = 0; d < a.head_dim; ++d) dot = fmaf(a.qs[d], to_f32(kr[d]), dot);
    }
    s = dot * a.scale;
  }
  m_b = wave_max(s);
  const float pj = valid ? expf(s - m_b) : 0.f;
  l_b = wave_sum(pj);
#pragma unroll
  for (int c = 0; c < kChanPerLane; ++c) o_b[c] = 0.f;
  const int jj_lo = a.lo > j0 ? a.lo - j0 : 0;
  const int jj_hi = a.p - j0 < kWave - 1 ? a.p - j0 : kWave - 1;
  constexpr int U = 8;  // value rows in flight
  for (int jj = jj_lo; jj <= jj_hi; jj += U) {
    // the rows' elements as they come from memory (a channel past the head's size reads channel 0 and
    // counts as zero below): nothing looks at a loaded value before all U rows are asked for
    T vv[U][kChanPerLane];
    float pw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int src = jj + u <= jj_hi ? jj + u : jj_hi;  // rows past the end: fetched again, never added
      const T* vr = a.v_pages + __shfl(row_at, src, kWave);
      pw[u] = __shfl(pj, src, kWave);
#pragma unroll
      for (int c = 0; c < kChanPerLane; ++c) {
        const int d = lane + c * kWave;
        if (c * kWave < a.head_dim) vv[u][c] = vr[d < a.head_dim ? d : 0];
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (jj + u <= jj_hi) {
#pragma unroll
        for (int c = 0; c < kChanPerLane; ++c) {
          const int d = lane + c * kWave;
          if (c * kWave < a.head_dim) o_b[c] = fmaf(pw[u], d < a.head_dim ? to_f32(vv[u][c]) : 0.f, o_b[c]);
        }
      }
  }
}

// The running result takes one more block in: blocks join in ascending order of their positions, each
// by exactly these operations, whoever computed the block.
__device__ __forceinline__ void merge_block(float& m, float& l, float (&acc)[kChanPerLane], float m_b, float l_b,
                                            const float (&o_b)[kChanPerLane]) {
#pragma clang fp contract(off)
  const float m_new = fmaxf(m, m_b);
  const float keep = expf(m - m_new);  // 0 for the first block (m = -inf)
  const float take = expf(m_b - m_new);
  l = fmaf(l, keep, l_b * take);
#pragma unroll
  for (int c = 0; c < kChanPerLane; ++c) acc[c] = fmaf(acc[c], keep, o_b[c] * take);
  m = m_new;
}

template <typename T>
__device__ __forceinline__ Query<T> make_query(const float* qs, const T* k_pages, const T* v_pages,
                                               const int32_t* token_seq, const int32_t* positions,
                                               const int32_t* block_table, int bt_stride, int t, int h, int n_q_heads,
                                               int n_kv_heads, int head_dim, int page_size, int window, float scale) {
  Query<T> a;
  a.qs = qs; a.k_pages = k_pages; a.v_pages = v_pages;
  a.bt = block_table + (size_t)token_seq[t] * bt_stride;
  a.n_kv_heads = n_kv_heads; a.g = h / (n_q_heads / n_kv_heads); a.head_dim = head_dim; a.page_size = page_size;
  a.head_elems = (size_t)page_size * head_dim;
  a.p = positions[t];
  a.lo = (window > 0 && a.p - window + 1 > 0) ? a.p - window + 1 : 0;
  a.scale = scale;
  return a;
}

// One wave per (token, query head) walks all blocks of 64 keys in ascending order.  It works alone:
// no barrier inside the loop.
template <typename T, bool VEC>
__global__ void __launch_bounds__(kWavesPerBlock* kWave)
attention_generic_kernel(const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
                         const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                         const int32_t* __restrict__ token_seq, const int32_t* __restrict__ positions,
                         const int32_t* __restrict__ block_table, int bt_stride, int n_q_heads,
                         int n_kv_heads, int head_dim, int page_size, int window, float scale) {
  __shared__ float q_lds[kWavesPerBlock][kMaxHeadDim];
  const int t = blockIdx.x;
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int h_raw = blockIdx.y * kWavesPerBlock + wave;
  const bool active = h_raw < n_q_heads;
  const int h = active ? h_raw : n_q_heads - 1;  // idle waves shadow the last head, store nothing
  const T* qv = q + (size_t)t * q_stride + (size_t)h * head_dim;
  for (int d = lane; d < head_dim; d += kWave) q_lds[wave][d] = to_f32(qv[d]);
  __syncthreads();
  const Query<T> a = make_query<T>(q_lds[wave], k_pages, v_pages, token_seq, positions, block_table, bt_stride, t, h,
                                   n_q_heads, n_kv_heads, head_dim, page_size, window, scale);
  float acc[kChanPerLane];
#pragma unroll
  for (int c = 0; c < kChanPerLane; ++c) acc[c] = 0.f;
  float m = -INFINITY, l = 0.f;
  for (int j0 = a.lo - a.lo % kWave; j0 <= a.p; j0 += kWave) {
    float m_b, l_b, o_b[kChanPerLane];
    block_partial<T, VEC>(a, j0, lane, m_b, l_b, o_b);
    merge_block(m, l, acc, m_b, l_b, o_b);
  }
  if (active) {
    T* o = out + (size_t)t * out_stride + (size_t)h * head_dim;
    const float inv_l = 1.0f / l;
#pragma unroll
    for (int c = 0; c < kChanPerLane; ++c) {
      const int d = lane + c * kWave;
      if (d < head_dim) o[d] = from_f32<T>(acc[c] * inv_l);
    }
  }
}

// The same result for prompt portions, with the keys and values shared: a block of 16 waves takes
// kTileWaves / HB consecutive tokens and HB query heads that read the same kv head, and every block of 64
// keys is brought into LDS once for all of them (as 32-bit floats, rows padded so that 64 lanes that read
// 64 different rows meet different banks).  Each wave then computes its block exactly as block_partial
// does, operation for operation, from LDS instead of from the pages, and lets it join its running result:
// the same bits as one wave walking alone, at a sixteenth of the traffic.  Tokens of different requests
// (a block that straddles two rows of the step) have different keys: such a block walks alone as above.
constexpr int kTileWaves = 16;
constexpr int kTilePad = 4;  // floats between LDS rows beyond head_dim: rows start four banks apart

template <bool VEC, int CH>
__device__ __forceinline__ void block_partial_lds(const float* qs, const float* k_t, const float* v_t, int pitch,
                                                  int head_dim, int lo, int p, float scale, int j0, int lane,
                                                  float& m_b, float& l_b, float (&o_b)[kChanPerLane]) {
#pragma clang fp contract(off)
  const int j = j0 + lane;
  const bool valid = j >= lo && j <= p;
  float s = -INFINITY;
  if (valid) {
    const float* kr = k_t + lane * pitch;
    float dot = 0.f;
    if (VEC) {
      for (int d = 0; d < head_dim; d += 4) {
        float kv[4];
        load4(kr + d, kv);
#pragma unroll
        for (int u = 0; u < 4; ++u) dot = fmaf(qs[d + u], kv[u], dot);
      }
    } else {
      for (int d = 0; d < head_dim; ++d) dot = fmaf(qs[d], kr[d], dot);
    }
    s = dot * scale;
  }
  m_b = wave_max(s);
  const float pj = valid ? expf(s - m_b) : 0.f;
  l_b = wave_sum(pj);
#pragma unroll
  for (int c = 0; c < kChanPerLane; ++c) o_b[c] = 0.f;
  const int jj_lo = lo > j0 ? lo - j0 : 0;
  const int jj_hi = p - j0 < kWave - 1 ? p - j0 : kWave - 1;
  // jj is the same in every lane: the probability of key jj comes out of its lane as a scalar.  Only the
  // CH channel slots that the head size fills are touched (the others stay zero, as in the walk alone, where
  // they add zeros).
  auto value = [&](int jj, int c) {
    const int d = lane + c * kWave;
    return (c + 1 < CH || d < head_dim) ? v_t[jj * pitch + d] : 0.f;
  };
  constexpr int U = 4;  // value rows asked for together; they are still added one after the other
  int jj = jj_lo;
  for (; jj + U - 1 <= jj_hi; jj += U) {
    float pw[U], vv[U][CH];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      pw[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(pj), jj + u));
#pragma unroll
      for (int c = 0; c < CH; ++c) vv[u][c] = value(jj + u, c);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int c = 0; c < CH; ++c) o_b[c] = fmaf(pw[u], vv[u][c], o_b[c]);
  }
  for (; jj <= jj_hi; ++jj) {
    const float pw = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(pj), jj));
#pragma unroll
    for (int c = 0; c < CH; ++c) o_b[c] = fmaf(pw, value(jj, c), o_b[c]);
  }
}

template <typename T, bool VEC, int CH>
__global__ void __launch_bounds__(kTileWaves* kWave)
attention_tile_kernel(const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
                      const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                      const int32_t* __restrict__ token_seq, const int32_t* __restrict__ positions,
                      const int32_t* __restrict__ block_table, int bt_stride, int n_tokens, int n_q_heads,
                      int n_kv_heads, int head_dim, int page_size, int window, float scale, int heads_per_block) {
  extern __shared__ __attribute__((aligned(16))) float tile_lds[];
  const int pitch = head_dim + kTilePad;
  float* q_lds = tile_lds;                          // [kTileWaves][head_dim]
  float* k_t = tile_lds + kTileWaves * head_dim;    // [64][pitch]
  float* v_t = k_t + kWave * pitch;                 // [64][pitch]
  const int HB = heads_per_block;
  const int QT = kTileWaves / HB;
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int t0 = blockIdx.x * QT;
  const int t_raw = t0 + wave / HB;
  const int h_raw = blockIdx.y * HB + wave % HB;
  const bool active = t_raw < n_tokens && h_raw < n_q_heads;
  const int t = t_raw < n_tokens ? t_raw : n_tokens - 1;  // idle waves shadow a real token, store nothing
  const int h = h_raw < n_q_heads ? h_raw : n_q_heads - 1;
  const T* qv = q + (size_t)t * q_stride + (size_t)h * head_dim;
  for (int d = lane; d < head_dim; d += kWave) q_lds[wave * head_dim + d] = to_f32(qv[d]);
  const Query<T> a = make_query<T>(q_lds + wave * head_dim, k_pages, v_pages, token_seq, positions, block_table,
                                   bt_stride, t, h, n_q_heads, n_kv_heads, head_dim, page_size, window, scale);
  // what the whole block sees: the same for every thread, from the tokens' own entries
  const int last = min(t0 + QT, n_tokens) - 1;
  const int seq0 = token_seq[t0];
  bool together = true;
  int blk_lo = INT_MAX, blk_hi = -1, key_lo = INT_MAX;
  for (int i = t0; i <= last; ++i) {
    together = together && token_seq[i] == seq0;
    const int pi = positions[i];
    const int li = (window > 0 && pi - window + 1 > 0) ? pi - window + 1 : 0;
    blk_lo = min(blk_lo, li - li % kWave);
    key_lo = min(key_lo, li);
    blk_hi = max(blk_hi, pi);
  }
  __syncthreads();  // the queries are in LDS
  // the wave's own bounds, as scalars (they are the same in all its lanes)
  const int lo_u = __builtin_amdgcn_readfirstlane(a.lo), p_u = __builtin_amdgcn_readfirstlane(a.p);
  float acc[kChanPerLane];
#pragma unroll
  for (int c = 0; c < kChanPerLane; ++c) acc[c] = 0.f;
  float m = -INFINITY, l = 0.f;
  if (!together) {
    for (int j0 = a.lo - a.lo % kWave; j0 <= a.p; j0 += kWave) {
      float m_b, l_b, o_b[kChanPerLane];
      block_partial<T, VEC>(a, j0, lane, m_b, l_b, o_b);
      merge_block(m, l, acc, m_b, l_b, o_b);
    }
  } else {
    const int g = (blockIdx.y * HB) / (n_q_heads / n_kv_heads);  // the kv head of all the block's heads
    const int32_t* bt = block_table + (size_t)seq0 * bt_stride;
    const size_t head_elems = (size_t)page_size * head_dim;
    const int per_row = VEC ? head_dim / 4 : head_dim;  // pieces of a row: four elements, or one
    for (int j0 = blk_lo; j0 <= blk_hi; j0 += kWave) {
      if (j0 > blk_lo) __syncthreads();  // everybody has finished with the tiles of the block before
      for (int idx = threadIdx.x; idx < kWave * per_row; idx += kTileWaves * kWave) {
        const int r = idx / per_row, piece = idx % per_row;
        const int j = j0 + r;
        if (j < key_lo || j > blk_hi) continue;  // nobody in the block sees this key
        const int page = bt[j / page_size];
        if (page < 0) continue;  // a page that a window gave back: no token of the step sees its keys
        const size_t row_at = ((size_t)page * n_kv_heads + g) * head_elems + (size_t)(j % page_size) * head_dim;
        if (VEC) {
          float kv[4], vv[4];
          load4(k_pages + row_at + 4 * piece, kv);
          load4(v_pages + row_at + 4 * piece, vv);
          *reinterpret_cast<float4*>(k_t + r * pitch + 4 * piece) = float4{kv[0], kv[1], kv[2], kv[3]};
          *reinterpret_cast<float4*>(v_t + r * pitch + 4 * piece) = float4{vv[0], vv[1], vv[2], vv[3]};
        } else {
          k_t[r * pitch + piece] = to_f32(k_pages[row_at + piece]);
          v_t[r * pitch + piece] = to_f32(v_pages[row_at + piece]);
        }
      }
      __syncthreads();
      if (j0 >= lo_u - lo_u % kWave && j0 <= p_u) {  // (uniform per wave)
        float m_b, l_b, o_b[kChanPerLane];
        block_partial_lds<VEC, CH>(a.qs, k_t, v_t, pitch, head_dim, lo_u, p_u, scale, j0, lane, m_b, l_b, o_b);
        merge_block(m, l, acc, m_b, l_b, o_b);
      }
    }
  }
  if (active) {
    T* o = out + (size_t)t * out_stride + (size_t)h * head_dim;
    const float inv_l = 1.0f / l;
#pragma unroll
    for (int c = 0; c < kChanPerLane; ++c) {
      const int d = lane + c * kWave;
      if (d < head_dim) o[d] = from_f32<T>(acc[c] * inv_l);
    }
  }
}

// The same result from many waves, for steps with few tokens and long contexts (decode): wave
// (token, head, r) computes block r of the token's key range alone and leaves it in `partials`
// ([token][head][r][head_dim + 2]: the sums, then maximum and sum of probabilities); a second kernel
// lets them join in ascending order.  Same blocks, same operations, same order: same bits.
constexpr int kPartialExtra = 2;

template <typename T, bool VEC>
__global__ void __launch_bounds__(kWavesPerBlock* kWave)
attention_blocks_kernel(const T* __restrict__ q, int q_stride, const T* __restrict__ k_pages,
                        const T* __restrict__ v_pages, const int32_t* __restrict__ token_seq,
                        const int32_t* __restrict__ positions, const int32_t* __restrict__ block_table, int bt_stride,
                        int n_q_heads, int n_kv_heads, int head_dim, int page_size, int window, float scale,
                        float* __restrict__ partials, int max_blocks) {
  __shared__ float q_lds[kWavesPerBlock][kMaxHeadDim];
  const int t = blockIdx.x;
  const int r = blockIdx.z;
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int h_raw = blockIdx.y * kWavesPerBlock + wave;
  const bool active = h_raw < n_q_heads;
  const int h = active ? h_raw : n_q_heads - 1;
  const T* qv = q + (size_t)t * q_stride + (size_t)h * head_dim;
  for (int d = lane; d < head_dim; d += kWave) q_lds[wave][d] = to_f32(qv[d]);
  __syncthreads();
  const Query<T> a = make_query<T>(q_lds[wave], k_pages, v_pages, token_seq, positions, block_table, bt_stride, t, h,
                                   n_q_heads, n_kv_heads, head_dim, page_size, window, scale);
  const int j0 = a.lo - a.lo % kWave + r * kWave;
  if (j0 > a.p || !active) return;  // (uniform per wave)
  float m_b, l_b, o_b[kChanPerLane];
  block_partial<T, VEC>(a, j0, lane, m_b, l_b, o_b);
  float* dst = partials + (((size_t)t * n_q_heads + h) * max_blocks + r) * (head_dim + kPartialExtra);
#pragma unroll
  for (int c = 0; c < kChanPerLane; ++c) {
    const int d = lane + c * kWave;
    if (d < head_dim) dst[d] = o_b[c];
  }
  if (lane == 0) {
    dst[head_dim] = m_b;
    dst[head_dim + 1] = l_b;
  }
}

template <typename T>
__global__ void __launch_bounds__(kWavesPerBlock* kWave)
attention_join_kernel(T* __restrict__ out, int out_stride, const int32_t* __restrict__ positions, int n_q_heads,
                      int head_dim, int window, const float* __restrict__ partials, int max_blocks) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int h = blockIdx.y * kWavesPerBlock + wave;
  if (h >= n_q_heads) return;
  const int p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int n_blocks = (p - (lo - lo % kWave)) / kWave + 1;
  const int stride = head_dim + kPartialExtra;
  const float* src = partials + ((size_t)t * n_q_heads + h) * max_blocks * stride;
  float acc[kChanPerLane];
#pragma unroll
  for (int c = 0; c < kChanPerLane; ++c) acc[c] = 0.f;
  float m = -INFINITY, l = 0.f;
  constexpr int U = 4;  // blocks in flight
  for (int r0 = 0; r0 < n_blocks; r0 += U) {
    float m_b[U], l_b[U], o_b[U][kChanPerLane];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float* blk = src + (size_t)(r0 + u < n_blocks ? r0 + u : n_blocks - 1) * stride;
      m_b[u] = blk[head_dim];
      l_b[u] = blk[head_dim + 1];
#pragma unroll
      for (int c = 0; c < kChanPerLane; ++c) {
        const int d = lane + c * kWave;
        o_b[u][c] = d < head_dim ? blk[d] : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (r0 + u < n_blocks) merge_block(m, l, acc, m_b[u], l_b[u], o_b[u]);
  }
  T* o = out + (size_t)t * out_stride + (size_t)h * head_dim;
  const float inv_l = 1.0f / l;
#pragma unroll
  for (int c = 0; c < kChanPerLane; ++c) {
    const int d = lane + c * kWave;
    if (d < head_dim) o[d] = from_f32<T>(acc[c] * inv_l);
  }
}

}  // namespace

// q: element (t, h, d) at q + t*q_stride + h*head_dim + d.  out likewise with out_stride.
// pages: [page][n_kv_heads][page_size][head_dim].  token_seq[t]: row of block_table;
// positions[t]: absolute position; the token sees positions max(0, p-window+1)..p (window 0: all).
TL_EXPORT int tl_attention_generic(const void* q, int q_stride, void* out, int out_stride,
                                   const void* k_pages, const void* v_pages, const int32_t* token_seq,
                                   const int32_t* positions, const int32_t* block_table, int bt_stride,
                                   int n_tokens, int n_q_heads, int n_kv_heads, int head_dim,
                                   int page_size, int window, float scale, int dtype,
                                   hipStream_t stream) {
  TL_REQUIRE(n_tokens >= 0 && n_q_heads > 0 && n_kv_heads > 0 && page_size > 0 && bt_stride > 0,
             "attention: bad sizes");
  TL_REQUIRE(n_q_heads % n_kv_heads == 0, "attention: %d query heads are not a multiple of %d kv heads",
             n_q_heads, n_kv_heads);
  if (head_dim <= 0 || head_dim > kMaxHeadDim)
    return tl_fail(TL_ERR_UNSUPPORTED, "attention: head_dim=%d outside 1..%d", head_dim, kMaxHeadDim);
  TL_REQUIRE(window >= 0, "attention: window=%d must be >= 0", window);
  if (n_tokens == 0) return TL_OK;
  dim3 grid(n_tokens, (n_q_heads + kWavesPerBlock - 1) / kWavesPerBlock);
  // rows of the pages start at multiples of head_dim elements from an allocation's start
  const bool vec = head_dim % 4 == 0 && ((uintptr_t)k_pages % 16) == 0;
  // prompt portions: tokens and heads that read the same keys share them through LDS (same bits)
  if (n_tokens >= kTileMinTokens) {
    const int group = n_q_heads / n_kv_heads;
    const int hb = group % 4 == 0 ? 4 : (group % 2 == 0 ? 2 : 1);
    const int qt = kTileWaves / hb;
    const size_t lds = ((size_t)kTileWaves * head_dim + 2 * (size_t)kWave * (head_dim + kTilePad)) * sizeof(float);
    dim3 tgrid((n_tokens + qt - 1) / qt, (n_q_heads + hb - 1) / hb);
#define TL_TILE_LAUNCH_CH(T, VEC, CH)                                                                            \
  do {                                                                                                           \
    if (lds > 48 * 1024) {                                                                                       \
      hipError_t e = hipFuncSetAttribute((const void*)attention_tile_kernel<T, VEC, CH>,                         \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                  \
      if (e != hipSuccess) return tl_fail(TL_ERR_HIP, "attention: %s", hipGetErrorString(e));                    \
    }                                                                                                            \
    attention_tile_kernel<T, VEC, CH><<<tgrid, kTileWaves * kWave, lds, stream>>>(                               \
        (const T*)q, q_stride, (T*)out, out_stride, (const T*)k_pages, (const T*)v_pages, token_seq, positions,  \
        block_table, bt_stride, n_tokens, n_q_heads, n_kv_heads, head_dim, page_size, window, scale, hb);        \
  } while (0)
#define TL_TILE_LAUNCH(T, VEC)                                                                                   \
  do {                                                                                                           \
    if (head_dim <= 64) TL_TILE_LAUNCH_CH(T, VEC, 1);                                                            \
    else if (head_dim <= 128) TL_TILE_LAUNCH_CH(T, VEC, 2);                                                      \
    else if (head_dim <= 192) TL_TILE_LAUNCH_CH(T, VEC, 3);                                                      \
    else TL_TILE_LAUNCH_CH(T, VEC, 4);                                                                           \
  } while (0)
    if (dtype == TL_F32) {
      if (vec) TL_TILE_LAUNCH(float, true);
      else TL_TILE_LAUNCH(float, false);
    } else if (dtype == TL_BF16) {
      if (vec) TL_TILE_LAUNCH(bf16_t, true);
      else TL_TILE_LAUNCH(bf16_t, false);
    } else {
      return tl_fail(TL_ERR_ARG, "attention: unknown dtype %d", dtype);
    }
#undef TL_TILE_LAUNCH_CH
#undef TL_TILE_LAUNCH
    return tl_check_launch("attention_tile");
  }
#define TL_ATTN_LAUNCH(T, VEC)                                                                              \
  attention_generic_kernel<T, VEC><<<grid, kWavesPerBlock * kWave, 0, stream>>>(                            \
      (const T*)q, q_stride, (T*)out, out_stride, (const T*)k_pages, (const T*)v_pages, token_seq, positions, \
      block_table, bt_stride, n_q_heads, n_kv_heads, head_dim, page_size, window, scale)
  if (dtype == TL_F32) {
    if (vec) TL_ATTN_LAUNCH(float, true);
    else TL_ATTN_LAUNCH(float, false);
  } else if (dtype == TL_BF16) {
    if (vec) TL_ATTN_LAUNCH(bf16_t, true);
    else TL_ATTN_LAUNCH(bf16_t, false);
  } else {
    return tl_fail(TL_ERR_ARG, "attention: unknown dtype %d", dtype);
  }
#undef TL_ATTN_LAUNCH
  return tl_check_launch("attention_generic");
}

// The same attention for steps with few tokens (decode): the blocks of 64 keys are computed by waves of
// their own and joined in order by a second kernel; the result has the bits of tl_attention_generic.
// max_blocks: at least the largest number of 64-key blocks (aligned to absolute positions) any token
// sees; partials: workspace of n_tokens * n_q_heads * max_blocks * (head_dim + 2) floats.
TL_EXPORT int tl_attention_generic_split(const void* q, int q_stride, void* out, int out_stride,
                                         const void* k_pages, const void* v_pages, const int32_t* token_seq,
                                         const int32_t* positions, const int32_t* block_table, int bt_stride,
                                         int n_tokens, int n_q_heads, int n_kv_heads, int head_dim,
                                         int page_size, int window, float scale, int dtype, int max_blocks,
                                         float* partials, hipStream_t stream) {
  TL_REQUIRE(n_tokens >= 0 && n_q_heads > 0 && n_kv_heads > 0 && page_size > 0 && bt_stride > 0,
             "attention: bad sizes");
  TL_REQUIRE(n_q_heads % n_kv_heads == 0, "attention: %d query heads are not a multiple of %d kv heads",
             n_q_heads, n_kv_heads);
  if (head_dim <= 0 || head_dim > kMaxHeadDim)
    return tl_fail(TL_ERR_UNSUPPORTED, "attention: head_dim=%d outside 1..%d", head_dim, kMaxHeadDim);
  TL_REQUIRE(window >= 0, "attention: window=%d must be >= 0", window);
  TL_REQUIRE(max_blocks >= 1 && max_blocks <= 65535 && partials != nullptr, "attention: max_blocks=%d outside 1..65535, or no workspace", max_blocks);
  TL_REQUIRE(n_tokens <= 65535, "attention: the split form takes at most 65535 tokens");
  if (n_tokens == 0) return TL_OK;
  const int head_blocks = (n_q_heads + kWavesPerBlock - 1) / kWavesPerBlock;
  dim3 grid(n_tokens, head_blocks, max_blocks);
  dim3 grid_join(n_tokens, head_blocks);
  const bool vec = head_dim % 4 == 0 && ((uintptr_t)k_pages % 16) == 0;
#define TL_ATTN_LAUNCH(T, VEC)                                                                                  \
  do {                                                                                                          \
    attention_blocks_kernel<T, VEC><<<grid, kWavesPerBlock * kWave, 0, stream>>>(                               \
        (const T*)q, q_stride, (const T*)k_pages, (const T*)v_pages, token_seq, positions, block_table, bt_stride, \
        n_q_heads, n_kv_heads, head_dim, page_size, window, scale, partials, max_blocks);                       \
    int rc = tl_check_launch("attention_blocks");                                                               \
    if (rc != TL_OK) return rc;                                                                                 \
    attention_join_kernel<T><<<grid_join, kWavesPerBlock * kWave, 0, stream>>>(                                 \
        (T*)out, out_stride, positions, n_q_heads, head_dim, window, partials, max_blocks);                     \
  } while (0)
  if (dtype == TL_F32) {
    if (vec) TL_ATTN_LAUNCH(float, true);
    else TL_ATTN_LAUNCH(float, false);
  } else if (dtype == TL_BF16) {
    if (vec) TL_ATTN_LAUNCH(bf16_t, true);
    else TL_ATTN_LAUNCH(bf16_t, false);
  } else {
    return tl_fail(TL_ERR_ARG, "attention: unknown dtype %d", dtype);
  }
#undef TL_ATTN_LAUNCH
  return tl_check_launch("attention_join");
}
