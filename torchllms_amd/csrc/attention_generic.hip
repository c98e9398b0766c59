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

template <typename T>
__global__ void __launch_bounds__(kWavesPerBlock* kWave)
attention_generic_kernel(const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
                         const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                         const int32_t* __restrict__ token_seq, const int32_t* __restrict__ positions,
                         const int32_t* __restrict__ block_table, int bt_stride, int n_q_heads,
                         int n_kv_heads, int head_dim, int page_size, int window, float scale) {
  __shared__ float q_lds[kWavesPerBlock][kMaxHeadDim];
  __shared__ float p_lds[kWavesPerBlock][kWave];

  const int t = blockIdx.x;
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int h_raw = blockIdx.y * kWavesPerBlock + wave;
  const bool active = h_raw < n_q_heads;
  const int h = active ? h_raw : n_q_heads - 1;  // idle waves shadow the last head, store nothing
  const int g = h / (n_q_heads / n_kv_heads);
  const int b = token_seq[t];
  const int p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int32_t* bt = block_table + (size_t)b * bt_stride;

  const T* qv = q + (size_t)t * q_stride + (size_t)h * head_dim;
  for (int d = lane; d < head_dim; d += kWave) q_lds[wave][d] = to_f32(qv[d]);
  __syncthreads();

  float acc[kChanPerLane];
#pragma unroll
  for (int c = 0; c < kChanPerLane; ++c) acc[c] = 0.f;
  float m = -INFINITY;
  float l = 0.f;
  const size_t head_elems = (size_t)page_size * head_dim;

  for (int j0 = lo - lo % kWave; j0 <= p; j0 += kWave) {
    const int j = j0 + lane;
    const bool valid = j >= lo && j <= p;
    float s = -INFINITY;
    if (valid) {
      const int page = bt[j / page_size];
      const T* kr = k_pages + ((size_t)page * n_kv_heads + g) * head_elems + (size_t)(j % page_size) * head_dim;
      float dot = 0.f;
      for (int d = 0; d < head_dim; ++d) dot += q_lds[wave][d] * to_f32(kr[d]);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float pj = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);  // 0 on the first block (m = -inf)
    l = l * alpha + wave_sum(pj);
    m = m_new;
    p_lds[wave][lane] = pj;
    __syncthreads();
    const int jj_lo = lo > j0 ? lo - j0 : 0;
    const int jj_hi = p - j0 < kWave - 1 ? p - j0 : kWave - 1;
#pragma unroll
    for (int c = 0; c < kChanPerLane; ++c) acc[c] *= alpha;
    for (int jj = jj_lo; jj <= jj_hi; ++jj) {
      const int jv = j0 + jj;
      const int page = bt[jv / page_size];
      const T* vr = v_pages + ((size_t)page * n_kv_heads + g) * head_elems + (size_t)(jv % page_size) * head_dim;
      const float pw = p_lds[wave][jj];
#pragma unroll
      for (int c = 0; c < kChanPerLane; ++c) {
        const int d = lane + c * kWave;
        if (d < head_dim) acc[c] += pw * to_f32(vr[d]);
      }
    }
    __syncthreads();
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
  if (dtype == TL_F32)
    attention_generic_kernel<float><<<grid, kWavesPerBlock * kWave, 0, stream>>>(
        (const float*)q, q_stride, (float*)out, out_stride, (const float*)k_pages, (const float*)v_pages,
        token_seq, positions, block_table, bt_stride, n_q_heads, n_kv_heads, head_dim, page_size, window, scale);
  else if (dtype == TL_BF16)
    attention_generic_kernel<bf16_t><<<grid, kWavesPerBlock * kWave, 0, stream>>>(
        (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages,
        token_seq, positions, block_table, bt_stride, n_q_heads, n_kv_heads, head_dim, page_size, window, scale);
  else
    return tl_fail(TL_ERR_ARG, "attention: unknown dtype %d", dtype);
  return tl_check_launch("attention_generic");
}
