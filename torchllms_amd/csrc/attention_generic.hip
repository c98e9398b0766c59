// Attention over paged keys and values, plain edition: any head size up to 256, any number of
// heads and groups, 32-bit or bfloat16 storage, all arithmetic in 32-bit.  One wave per
// (token, query head).  Keys are visited in ascending position in blocks of 64 aligned to
// absolute position, so a result depends only on the query's position and the cache contents,
// never on how the step was batched.  This is the kernel of the 32-bit path and the fallback of
// the bfloat16 path for sizes the MFMA kernels refuse.
#include "common.h"

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kMaxHeadDim = 256;
constexpr int kChanPerLane = kMaxHeadDim / kWave;

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
      for (int d = 0; d < a.head_dim; d += 4) {
        float kv[4];
        load4(kr + d, kv);
#pragma unroll
        for (int u = 0; u < 4; ++u) dot = fmaf(a.qs[d + u], kv[u], dot);
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
    float vv[U][kChanPerLane];
    float pw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int src = jj + u <= jj_hi ? jj + u : jj_hi;  // rows past the end: fetched again, never added
      const T* vr = a.v_pages + __shfl(row_at, src, kWave);
      pw[u] = __shfl(pj, src, kWave);
#pragma unroll
      for (int c = 0; c < kChanPerLane; ++c) {
        const int d = lane + c * kWave;
        vv[u][c] = d < a.head_dim ? to_f32(vr[d]) : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (jj + u <= jj_hi) {
#pragma unroll
        for (int c = 0; c < kChanPerLane; ++c) o_b[c] = fmaf(pw[u], vv[u][c], o_b[c]);
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
