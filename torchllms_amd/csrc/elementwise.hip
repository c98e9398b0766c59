// Row-wise kernels: embedding gather, RMS norm fused with the residual sum, rotary position
// encoding fused with the write of keys and values into cache pages, SwiGLU gate, bias.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

// ----------------------------------------------------------------------------- errors
static thread_local char g_last_error[512] = "";

int tl_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

int tl_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return tl_fail(TL_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
  return TL_OK;
}

const TlDeviceFacts& tl_device_facts() {
  constexpr int kMaxDevices = 64;
  static TlDeviceFacts facts[kMaxDevices];  // zero until read; a race reads the same values twice
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = 0;
  if (facts[dev].compute_units == 0) {
    hipDeviceProp_t prop;
    TlDeviceFacts f = {256, 160 * 1024};  // MI355X, should the device refuse to answer
    if (hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0) {
      f.compute_units = prop.multiProcessorCount;
      f.lds_bytes = (int)prop.sharedMemPerBlock;
    }
    facts[dev] = f;
  }
  return facts[dev];
}

TL_EXPORT const char* tl_last_error() { return g_last_error; }
// The same figures for the host side's launch plans.
TL_EXPORT int tl_device_compute_units() { return tl_device_facts().compute_units; }
TL_EXPORT int tl_device_lds_bytes() { return tl_device_facts().lds_bytes; }
TL_EXPORT int tl_abi_version() { return 1; }

// ----------------------------------------------------------------------------- embedding
// out[t, :] = table[tokens[t], :].  One block per token; 16-byte copies when the row allows.
template <typename T>
__global__ void embed_kernel(const int32_t* __restrict__ tokens, const T* __restrict__ table,
                             T* __restrict__ out, int hidden) {
  const int t = blockIdx.x;
  const T* src = table + (size_t)tokens[t] * hidden;
  T* dst = out + (size_t)t * hidden;
  constexpr int VEC = 16 / sizeof(T);
  if (hidden % VEC == 0) {
    const uint4* s4 = reinterpret_cast<const uint4*>(src);
    uint4* d4 = reinterpret_cast<uint4*>(dst);
    for (int i = threadIdx.x; i < hidden / VEC; i += blockDim.x) d4[i] = s4[i];
  } else {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = src[i];
  }
}

TL_EXPORT int tl_embed(const int32_t* tokens, const void* table, void* out, int n_tokens, int hidden,
                       int dtype, hipStream_t stream) {
  TL_REQUIRE(n_tokens >= 0 && hidden > 0, "embed: bad sizes n_tokens=%d hidden=%d", n_tokens, hidden);
  if (n_tokens == 0) return TL_OK;
  if (dtype == TL_F32)
    embed_kernel<float><<<n_tokens, 256, 0, stream>>>(tokens, (const float*)table, (float*)out, hidden);
  else if (dtype == TL_BF16)
    embed_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>(tokens, (const bf16_t*)table, (bf16_t*)out, hidden);
  else
    return tl_fail(TL_ERR_ARG, "embed: unknown dtype %d", dtype);
  return tl_check_launch("embed");
}

// ----------------------------------------------------------------------------- RMS norm
// For output row r (source row s = rows ? rows[r] : r):
//   h   = T(float(x[s]) + float(delta[s]))            (delta optional; sum in 32-bit, one rounding)
//   n   = T(float(h) * 1/sqrt(mean(float(h)^2) + eps))
//   y   = T(float(n) * float(weight))
// h is written to h_out when given.  Statistics are 32-bit with a fixed reduction order.
constexpr int kNormThreads = 256;

template <typename T, typename WT>
__global__ void __launch_bounds__(kNormThreads)
rmsnorm_kernel(const T* __restrict__ x, const T* __restrict__ delta, const int32_t* __restrict__ rows,
               const WT* __restrict__ weight, T* __restrict__ h_out, T* __restrict__ y, int hidden,
               float eps) {
  __shared__ float scratch[kNormThreads / kWave];
  extern __shared__ float row_cache[];  // hidden floats: the summed row, kept between the passes
  const int r = blockIdx.x;
  const size_t s = rows ? (size_t)rows[r] : (size_t)r;
  const T* xr = x + s * hidden;
  const T* dr = delta ? delta + s * hidden : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += kNormThreads) {
    float v = to_f32(xr[i]);
    if (dr) v = to_f32(from_f32<T>(v + to_f32(dr[i])));
    row_cache[i] = v;
    ss += v * v;
  }
  ss = block_sum<kNormThreads / kWave>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
  T* yr = y + (size_t)r * hidden;
  T* hr = h_out ? h_out + (size_t)r * hidden : nullptr;
  for (int i = threadIdx.x; i < hidden; i += kNormThreads) {
    const float v = row_cache[i];
    if (hr) hr[i] = from_f32<T>(v);
    const float n = to_f32(from_f32<T>(v * inv));
    yr[i] = from_f32<T>(n * to_f32(weight[i]));
  }
}

// Fast path: rows whose length is a multiple of the 16-byte vector and at most kNormThreads * 4 vectors
// long are read with 16-byte loads and kept in registers between the two passes.  NV = vectors per
// thread.  Between two large kernels every load here misses all caches, so the kernel's time is its
// chain of dependent loads: everything it will need (row, delta and the weight) is asked for at the
// top, without a branch in between, and waited for once.
template <typename T, int VEC>
struct alignas(16) NormVec {
  T e[VEC];
};

template <typename T, typename WT, int NV>
__global__ void __launch_bounds__(kNormThreads)
rmsnorm_vec_kernel(const T* __restrict__ x, const T* __restrict__ delta, const int32_t* __restrict__ rows,
                   const WT* __restrict__ weight, T* __restrict__ h_out, T* __restrict__ y, int hidden,
                   float eps) {
  constexpr int VEC = 16 / sizeof(T);
  typedef NormVec<T, VEC> V;
  typedef NormVec<WT, VEC> W;
  __shared__ float scratch[kNormThreads / kWave];
  const int r = blockIdx.x;
  const size_t s = rows ? (size_t)rows[r] : (size_t)r;
  const int n_vec = hidden / VEC;
  const V* xr = reinterpret_cast<const V*>(x + s * hidden);
  const V* dr = reinterpret_cast<const V*>(delta ? delta + s * hidden : x + s * hidden);
  const W* wr = reinterpret_cast<const W*>(weight);
  int at[NV];   // a thread past the row's end reads the last vector again and uses nothing of it
#pragma unroll
  for (int it = 0; it < NV; ++it) at[it] = min(threadIdx.x + it * kNormThreads, n_vec - 1);
  V xin[NV], din[NV];
  W win[NV];
#pragma unroll
  for (int it = 0; it < NV; ++it) xin[it] = xr[at[it]];
#pragma unroll
  for (int it = 0; it < NV; ++it) din[it] = dr[at[it]];
#pragma unroll
  for (int it = 0; it < NV; ++it) win[it] = wr[at[it]];
  const bool add = delta != nullptr;
  float v[NV][VEC];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < NV; ++it) {
    const bool live = threadIdx.x + it * kNormThreads < n_vec;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      float f = to_f32(xin[it].e[e]);
      const float sum = to_f32(from_f32<T>(f + to_f32(din[it].e[e])));
      f = add ? sum : f;
      f = live ? f : 0.f;
      v[it][e] = f;
      ss += f * f;
    }
  }
  ss = block_sum<kNormThreads / kWave>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
  V* yr = reinterpret_cast<V*>(y + (size_t)r * hidden);
  V* hr = h_out ? reinterpret_cast<V*>(h_out + (size_t)r * hidden) : nullptr;
#pragma unroll
  for (int it = 0; it < NV; ++it) {
    const int c = threadIdx.x + it * kNormThreads;
    if (c < n_vec) {
      V out, hs;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        hs.e[e] = from_f32<T>(v[it][e]);
        const float n = to_f32(from_f32<T>(v[it][e] * inv));
        out.e[e] = from_f32<T>(n * to_f32(win[it].e[e]));
      }
      yr[c] = out;
      if (hr) hr[c] = hs;
    }
  }
}

template <typename T, typename WT>
static void launch_rmsnorm_vec(const void* x, const void* delta, const int32_t* rows, const void* weight, void* h_out, void* y,
                               int n_rows, int hidden, float eps, hipStream_t stream) {
  const int per_thread = (hidden / (16 / (int)sizeof(T)) + kNormThreads - 1) / kNormThreads;
#define TL_NORM_VEC(NV)                                                                                          \
  rmsnorm_vec_kernel<T, WT, NV><<<n_rows, kNormThreads, 0, stream>>>((const T*)x, (const T*)delta, rows, (const WT*)weight, \
                                                                     (T*)h_out, (T*)y, hidden, eps)
  if (per_thread <= 1) TL_NORM_VEC(1);
  else if (per_thread == 2) TL_NORM_VEC(2);
  else if (per_thread == 3) TL_NORM_VEC(3);
  else TL_NORM_VEC(4);
#undef TL_NORM_VEC
}

TL_EXPORT int tl_rmsnorm(const void* x, const void* delta, const int32_t* rows, const void* weight,
                         int weight_dtype, void* h_out, void* y, int n_rows, int hidden, float eps,
                         int dtype, hipStream_t stream) {
  TL_REQUIRE(n_rows >= 0 && hidden > 0, "rmsnorm: bad sizes n_rows=%d hidden=%d", n_rows, hidden);
  TL_REQUIRE(!(rows && h_out), "rmsnorm: h_out cannot be combined with a row gather");
  TL_REQUIRE((size_t)hidden * sizeof(float) <= (size_t)tl_device_facts().lds_bytes - 1024, "rmsnorm: hidden=%d does not fit LDS", hidden);
  if (n_rows == 0) return TL_OK;
  const size_t lds = (size_t)hidden * sizeof(float);
  const int vec = dtype == TL_F32 ? 4 : 8;
  const bool aligned = ((uintptr_t)x % 16 == 0) && ((uintptr_t)y % 16 == 0) && (!delta || (uintptr_t)delta % 16 == 0) &&
                       (!h_out || (uintptr_t)h_out % 16 == 0) && ((uintptr_t)weight % 16 == 0);
  if (hidden % vec == 0 && hidden / vec <= kNormThreads * 4 && aligned) {
    if (dtype == TL_F32 && weight_dtype == TL_F32)
      launch_rmsnorm_vec<float, float>(x, delta, rows, weight, h_out, y, n_rows, hidden, eps, stream);
    else if (dtype == TL_BF16 && weight_dtype == TL_BF16)
      launch_rmsnorm_vec<bf16_t, bf16_t>(x, delta, rows, weight, h_out, y, n_rows, hidden, eps, stream);
    else if (dtype == TL_BF16 && weight_dtype == TL_F32)
      launch_rmsnorm_vec<bf16_t, float>(x, delta, rows, weight, h_out, y, n_rows, hidden, eps, stream);
    else
      return tl_fail(TL_ERR_ARG, "rmsnorm: unsupported dtypes x=%d weight=%d", dtype, weight_dtype);
    return tl_check_launch("rmsnorm");
  }
#define TL_NORM_LAUNCH(T, WT)                                                                       \
  do {                                                                                              \
    if (lds > 48 * 1024) {                                                                          \
      hipError_t e = hipFuncSetAttribute((const void*)rmsnorm_kernel<T, WT>,                        \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);     \
      if (e != hipSuccess) return tl_fail(TL_ERR_HIP, "rmsnorm: %s", hipGetErrorString(e));         \
    }                                                                                               \
    rmsnorm_kernel<T, WT><<<n_rows, kNormThreads, lds, stream>>>(                                   \
        (const T*)x, (const T*)delta, rows, (const WT*)weight, (T*)h_out, (T*)y, hidden, eps);      \
  } while (0)
  if (dtype == TL_F32 && weight_dtype == TL_F32)
    TL_NORM_LAUNCH(float, float);
  else if (dtype == TL_BF16 && weight_dtype == TL_BF16)
    TL_NORM_LAUNCH(bf16_t, bf16_t);
  else if (dtype == TL_BF16 && weight_dtype == TL_F32)
    TL_NORM_LAUNCH(bf16_t, float);
  else
    return tl_fail(TL_ERR_ARG, "rmsnorm: unsupported dtypes x=%d weight=%d", dtype, weight_dtype);
#undef TL_NORM_LAUNCH
  return tl_check_launch("rmsnorm");
}

// The same for a delta that arrives as the 32-bit partial sums of a matrix product split along K
// (partial[s][row][i], s = 0 .. splits - 1): they are added in the order of the splits and rounded
// to bfloat16, as the kernel that would otherwise finish the product does, and then the row goes the
// way of rmsnorm_vec_kernel.  One launch instead of two.
template <typename WT, int NV>
__global__ void __launch_bounds__(kNormThreads)
rmsnorm_split_kernel(const bf16_t* __restrict__ x, const float* __restrict__ partial, int splits, size_t split_stride,
                     const int32_t* __restrict__ rows, const WT* __restrict__ weight, bf16_t* __restrict__ h_out,
                     bf16_t* __restrict__ y, int hidden, float eps) {
  constexpr int VEC = 8;
  typedef NormVec<bf16_t, VEC> V;
  typedef NormVec<WT, VEC> W;
  typedef NormVec<float, VEC> P;
  __shared__ float scratch[kNormThreads / kWave];
  const int r = blockIdx.x;
  const size_t s = rows ? (size_t)rows[r] : (size_t)r;
  const int n_vec = hidden / VEC;
  const V* xr = reinterpret_cast<const V*>(x + s * hidden);
  const P* pr = reinterpret_cast<const P*>(partial + s * hidden);
  const W* wr = reinterpret_cast<const W*>(weight);
  const size_t step = split_stride / VEC;
  int at[NV];
#pragma unroll
  for (int it = 0; it < NV; ++it) at[it] = min(threadIdx.x + it * kNormThreads, n_vec - 1);
  // row, weight and the first two splits are asked for together; further splits two at a time.  Each
  // element still adds its splits in their order.
  V xin[NV];
  W win[NV];
  P first[NV], second[NV];
#pragma unroll
  for (int it = 0; it < NV; ++it) xin[it] = xr[at[it]];
#pragma unroll
  for (int it = 0; it < NV; ++it) first[it] = pr[at[it]];
  const size_t one = splits > 1 ? step : 0;
#pragma unroll
  for (int it = 0; it < NV; ++it) second[it] = pr[one + at[it]];
#pragma unroll
  for (int it = 0; it < NV; ++it) win[it] = wr[at[it]];
  float d[NV][VEC];
#pragma unroll
  for (int it = 0; it < NV; ++it)
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      d[it][e] = 0.f + first[it].e[e];
      if (splits > 1) d[it][e] += second[it].e[e];
    }
  for (int k = 2; k < splits; k += 2) {
    const size_t next = k + 1 < splits ? step : 0;
#pragma unroll
    for (int it = 0; it < NV; ++it) first[it] = pr[k * step + at[it]];
#pragma unroll
    for (int it = 0; it < NV; ++it) second[it] = pr[k * step + next + at[it]];
#pragma unroll
    for (int it = 0; it < NV; ++it)
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        d[it][e] += first[it].e[e];
        if (k + 1 < splits) d[it][e] += second[it].e[e];
      }
  }
  float v[NV][VEC];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < NV; ++it) {
    const bool live = threadIdx.x + it * kNormThreads < n_vec;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      float f = to_f32(from_f32<bf16_t>(to_f32(xin[it].e[e]) + to_f32(from_f32<bf16_t>(d[it][e]))));
      f = live ? f : 0.f;
      v[it][e] = f;
      ss += f * f;
    }
  }
  ss = block_sum<kNormThreads / kWave>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
  V* yr = reinterpret_cast<V*>(y + (size_t)r * hidden);
  V* hr = h_out ? reinterpret_cast<V*>(h_out + (size_t)r * hidden) : nullptr;
#pragma unroll
  for (int it = 0; it < NV; ++it) {
    const int c = threadIdx.x + it * kNormThreads;
    if (c < n_vec) {
      V out, hs;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        hs.e[e] = from_f32<bf16_t>(v[it][e]);
        const float n = to_f32(from_f32<bf16_t>(v[it][e] * inv));
        out.e[e] = from_f32<bf16_t>(n * to_f32(win[it].e[e]));
      }
      yr[c] = out;
      if (hr) hr[c] = hs;
    }
  }
}

template <typename WT>
static void launch_rmsnorm_split(const void* x, const float* partial, int splits, size_t split_stride, const int32_t* rows,
                                 const void* weight, void* h_out, void* y, int n_rows, int hidden, float eps, hipStream_t stream) {
  const int per_thread = (hidden / 8 + kNormThreads - 1) / kNormThreads;
#define TL_NORM_SPLIT(NV)                                                                                                \
  rmsnorm_split_kernel<WT, NV><<<n_rows, kNormThreads, 0, stream>>>((const bf16_t*)x, partial, splits, split_stride, rows, \
                                                                    (const WT*)weight, (bf16_t*)h_out, (bf16_t*)y, hidden, eps)
  if (per_thread <= 1) TL_NORM_SPLIT(1);
  else if (per_thread == 2) TL_NORM_SPLIT(2);
  else if (per_thread == 3) TL_NORM_SPLIT(3);
  else TL_NORM_SPLIT(4);
#undef TL_NORM_SPLIT
}

// RMS norm of x + sum of the splits, bfloat16 x / h_out / y [.., hidden]; partial: 32-bit, split s of
// row r at partial + s * split_stride + r * hidden (split_stride in elements, a multiple of 8).
// hidden must be a multiple of 8 and at most 8 * 4 * 256.
TL_EXPORT int tl_rmsnorm_split(const void* x, const float* partial, int splits, int64_t split_stride, const int32_t* rows,
                               const void* weight, int weight_dtype, void* h_out, void* y, int n_rows, int hidden,
                               float eps, hipStream_t stream) {
  TL_REQUIRE(n_rows >= 0 && hidden > 0 && splits >= 1, "rmsnorm_split: bad sizes n_rows=%d hidden=%d splits=%d", n_rows, hidden, splits);
  TL_REQUIRE(!(rows && h_out), "rmsnorm_split: h_out cannot be combined with a row gather");
  if (hidden % 8 != 0 || hidden / 8 > kNormThreads * 4)
    return tl_fail(TL_ERR_UNSUPPORTED, "rmsnorm_split: hidden=%d must be a multiple of 8 and at most %d", hidden, 8 * 4 * kNormThreads);
  TL_REQUIRE(split_stride % 8 == 0 && ((uintptr_t)partial % 16) == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)y % 16) == 0 &&
                 (!h_out || (uintptr_t)h_out % 16 == 0) && ((uintptr_t)weight % 16) == 0,
             "rmsnorm_split: tensors must start on 16-byte boundaries and splits lie a multiple of 8 elements apart");
  if (n_rows == 0) return TL_OK;
  if (weight_dtype == TL_BF16)
    launch_rmsnorm_split<bf16_t>(x, partial, splits, (size_t)split_stride, rows, weight, h_out, y, n_rows, hidden, eps, stream);
  else if (weight_dtype == TL_F32)
    launch_rmsnorm_split<float>(x, partial, splits, (size_t)split_stride, rows, weight, h_out, y, n_rows, hidden, eps, stream);
  else
    return tl_fail(TL_ERR_ARG, "rmsnorm_split: unsupported weight dtype %d", weight_dtype);
  return tl_check_launch("rmsnorm_split");
}

// ----------------------------------------------------------------------------- rotary + KV write
// qkv: [n_tokens, (Hq + 2 Hkv) * dh], each row = q heads | k heads | v heads.
// For token t at position p: angle_i = float(p) * inv_freq[i], i < rotary_dim/2 (32-bit), and
//   pairing 0 (interleaved): (x[2i], x[2i+1])     pairing 1 (half split): (x[i], x[i + rotary_dim/2])
//   x0' = x0 cos - x1 sin ;  x1' = x1 cos + x0 sin        (32-bit, then one rounding)
// q is rotated in place.  k is rotated and, with v, stored at slot_mapping[t] = page * P + offset
// of pages laid out [page][Hkv][P][dh]; slot < 0 skips the store.  Without pages k is rotated in place.
// The cosines and sines may come from a table [token][rotary_dim/2] of (cos, sin) made by
// rope_table_kernel from the same positions (one table serves all layers of a step).
__global__ void rope_table_kernel(const int32_t* __restrict__ positions, const float* __restrict__ inv_freq,
                                  int n_tokens, int rot_half, float2* __restrict__ table) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n_tokens * rot_half) return;
  const int t = idx / rot_half;
  const int i = idx % rot_half;
  const float ang = (float)positions[t] * inv_freq[i];
  table[idx] = make_float2(cosf(ang), sinf(ang));
}

TL_EXPORT int tl_rope_table(const int32_t* positions, const float* inv_freq, int n_tokens, int rot_half,
                            float* table, hipStream_t stream) {
  TL_REQUIRE(n_tokens >= 0 && rot_half > 0, "rope_table: bad sizes");
  TL_REQUIRE((long long)n_tokens * rot_half < (1ll << 31), "rope_table: too many entries");
  if (n_tokens == 0) return TL_OK;
  const int total = n_tokens * rot_half;
  rope_table_kernel<<<(total + 255) / 256, 256, 0, stream>>>(positions, inv_freq, n_tokens, rot_half, (float2*)table);
  return tl_check_launch("rope_table");
}

template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, int n_q_heads, int n_kv_heads, int head_dim,
                                     const int32_t* __restrict__ positions,
                                     const float* __restrict__ inv_freq, const float2* __restrict__ cos_sin,
                                     int rotary_dim, int pairing,
                                     T* __restrict__ k_pages, T* __restrict__ v_pages,
                                     const int32_t* __restrict__ slot_mapping, int page_size) {
  const int t = blockIdx.x;
  const int half = head_dim / 2;
  const int rot_half = rotary_dim / 2;
  const float pos = (float)positions[t];
  const int row = (n_q_heads + 2 * n_kv_heads) * head_dim;
  T* base = qkv + (size_t)t * row;
  const int slot = slot_mapping ? slot_mapping[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? slot % page_size : 0;
  const bool store = k_pages != nullptr && slot >= 0;

  // queries and keys: a thread owns one pair index and walks over heads, so the angle's cosine and
  // sine are formed once per (token, pair) and block; with few tokens the heads are spread over
  // gridDim.y blocks so that the launch still fills the GPU
  const int n_rot_heads = n_q_heads + n_kv_heads;
  const int lanes_per_head = half;                       // threads that cover the pairs of one head
  const int head_groups = blockDim.x / lanes_per_head > 0 ? blockDim.x / lanes_per_head : 1;
  for (int i = threadIdx.x % lanes_per_head; i < half; i += blockDim.x) {
    const int hgrp = threadIdx.x / lanes_per_head;
    if (hgrp >= head_groups) continue;
    int i0, i1;
    float c = 1.f, sn = 0.f;
    const bool rotates = i < rot_half;
    if (rotates) {
      if (pairing == 0) {
        i0 = 2 * i;
        i1 = 2 * i + 1;
      } else {
        i0 = i;
        i1 = i + rot_half;
      }
      if (cos_sin) {
        const float2 cs = cos_sin[(size_t)t * rot_half + i];
        c = cs.x;
        sn = cs.y;
      } else {
        const float ang = pos * inv_freq[i];
        c = cosf(ang);
        sn = sinf(ang);
      }
    } else {
      // channels beyond rotary_dim pass unchanged
      i0 = rotary_dim + 2 * (i - rot_half);
      i1 = i0 + 1;
    }
    for (int h = hgrp + head_groups * blockIdx.y; h < n_rot_heads; h += head_groups * gridDim.y) {
      T* head = base + (size_t)h * head_dim;
      const float a0 = to_f32(head[i0]);
      const float a1 = to_f32(head[i1]);
      const float x0 = rotates ? a0 * c - a1 * sn : a0;
      const float x1 = rotates ? a1 * c + a0 * sn : a1;
      const T r0 = from_f32<T>(x0);
      const T r1 = from_f32<T>(x1);
      if (h < n_q_heads || k_pages == nullptr) {
        head[i0] = r0;
        head[i1] = r1;
      }
      if (h >= n_q_heads && store) {
        const int kh = h - n_q_heads;
        T* dst = k_pages + (((size_t)page * n_kv_heads + kh) * page_size + off) * head_dim;
        dst[i0] = r0;
        dst[i1] = r1;
      }
    }
  }
  // values
  if (store && v_pages != nullptr) {
    const T* vsrc = base + (size_t)(n_q_heads + n_kv_heads) * head_dim;
    for (int w = threadIdx.x + blockDim.x * blockIdx.y; w < n_kv_heads * head_dim; w += blockDim.x * gridDim.y) {
      const int kh = w / head_dim;
      const int d = w % head_dim;
      v_pages[(((size_t)page * n_kv_heads + kh) * page_size + off) * head_dim + d] = vsrc[w];
    }
  }
}

// The same work with 16-byte accesses, for the common case: interleaved pairs, the step's table of
// cosines and sines, head and rotary sizes that are multiples of the V elements a thread takes.
// One thread = V consecutive channels of one head of one token.
template <typename T, int V>
__global__ void rope_kv_write_vec_kernel(T* __restrict__ qkv, int n_tokens, int n_q_heads, int n_kv_heads, int head_dim,
                                         const float2* __restrict__ cos_sin, int rotary_dim,
                                         T* __restrict__ k_pages, T* __restrict__ v_pages,
                                         const int32_t* __restrict__ slot_mapping, int page_size) {
  struct alignas(sizeof(T) * V) Vec { T e[V]; };
  const int chunks_per_head = head_dim / V;
  const int heads = n_q_heads + (k_pages ? 2 : 1) * n_kv_heads;  // values only move when there are pages
  const int per_token = heads * chunks_per_head;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)n_tokens * per_token) return;
  const int t = (int)(idx / per_token);
  const int c = (int)(idx % per_token);
  const int head = c / chunks_per_head;
  const int d0 = (c % chunks_per_head) * V;
  const int row = (n_q_heads + 2 * n_kv_heads) * head_dim;
  T* src = qkv + (size_t)t * row + (size_t)head * head_dim + d0;
  Vec v = *reinterpret_cast<const Vec*>(src);
  const bool rotates = head < n_q_heads + n_kv_heads;
  if (rotates && d0 < rotary_dim) {
    const float2* cs = cos_sin + (size_t)t * (rotary_dim / 2) + d0 / 2;
#pragma unroll
    for (int j = 0; j < V / 2; ++j) {
      if (d0 + 2 * j < rotary_dim) {
        const float2 f = cs[j];
        const float a0 = to_f32(v.e[2 * j]), a1 = to_f32(v.e[2 * j + 1]);
        v.e[2 * j] = from_f32<T>(a0 * f.x - a1 * f.y);
        v.e[2 * j + 1] = from_f32<T>(a1 * f.x + a0 * f.y);
      }
    }
  }
  if (head < n_q_heads || k_pages == nullptr) {
    if (rotates) *reinterpret_cast<Vec*>(src) = v;
    return;
  }
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  const int page = slot / page_size, off = slot % page_size;
  const bool is_key = head < n_q_heads + n_kv_heads;
  const int kh = is_key ? head - n_q_heads : head - n_q_heads - n_kv_heads;
  T* dst = (is_key ? k_pages : v_pages) + (((size_t)page * n_kv_heads + kh) * page_size + off) * head_dim + d0;
  *reinterpret_cast<Vec*>(dst) = v;
}

template <typename T>
bool rope_vec_launch(T* qkv, int n_tokens, int n_q_heads, int n_kv_heads, int head_dim, const float2* cos_sin,
                     int rotary_dim, int pairing, T* k_pages, T* v_pages, const int32_t* slot_mapping, int page_size,
                     hipStream_t stream) {
  constexpr int V = 16 / sizeof(T);
  if (pairing != 0 || (rotary_dim > 0 && cos_sin == nullptr) || head_dim % V || rotary_dim % 2) return false;
  if (((uintptr_t)qkv % 16) || (k_pages && (((uintptr_t)k_pages % 16) || ((uintptr_t)v_pages % 16)))) return false;
  const long long threads_needed = (long long)n_tokens * (n_q_heads + (k_pages ? 2 : 1) * n_kv_heads) * (head_dim / V);
  const long long blocks = (threads_needed + 255) / 256;
  if (blocks > 0x7fffffffLL) return false;
  rope_kv_write_vec_kernel<T, V><<<(unsigned)blocks, 256, 0, stream>>>(
      qkv, n_tokens, n_q_heads, n_kv_heads, head_dim, cos_sin, rotary_dim, k_pages, v_pages, slot_mapping, page_size);
  return true;
}

TL_EXPORT int tl_rope_kv_write(void* qkv, int n_tokens, int n_q_heads, int n_kv_heads, int head_dim,
                               const int32_t* positions, const float* inv_freq, const float* cos_sin,
                               int rotary_dim, int pairing, void* k_pages, void* v_pages,
                               const int32_t* slot_mapping, int page_size, int dtype, hipStream_t stream) {
  TL_REQUIRE(n_tokens >= 0 && n_q_heads > 0 && n_kv_heads >= 0 && head_dim > 0, "rope: bad sizes");
  TL_REQUIRE(head_dim % 2 == 0, "rope: head_dim=%d must be even", head_dim);
  TL_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0,
             "rope: rotary_dim=%d must be even and at most head_dim=%d", rotary_dim, head_dim);
  TL_REQUIRE(pairing == 0 || pairing == 1, "rope: pairing must be 0 (interleaved) or 1 (half split)");
  TL_REQUIRE(rotary_dim == 0 || inv_freq != nullptr || cos_sin != nullptr, "rope: neither inv_freq nor a table given");
  TL_REQUIRE(k_pages == nullptr || (slot_mapping != nullptr && page_size > 0),
             "rope: pages given without slot_mapping/page_size");
  if (n_tokens == 0) return TL_OK;
  if (dtype != TL_F32 && dtype != TL_BF16) return tl_fail(TL_ERR_ARG, "rope: unknown dtype %d", dtype);
  if (dtype == TL_F32
          ? rope_vec_launch((float*)qkv, n_tokens, n_q_heads, n_kv_heads, head_dim, (const float2*)cos_sin, rotary_dim,
                            pairing, (float*)k_pages, (float*)v_pages, slot_mapping, page_size, stream)
          : rope_vec_launch((bf16_t*)qkv, n_tokens, n_q_heads, n_kv_heads, head_dim, (const float2*)cos_sin, rotary_dim,
                            pairing, (bf16_t*)k_pages, (bf16_t*)v_pages, slot_mapping, page_size, stream))
    return tl_check_launch("rope_kv_write");
  const int threads = 256;
  // heads per block column: all of them when the tokens alone fill the GPU, one pass otherwise
  const int head_groups = threads / (head_dim / 2) > 0 ? threads / (head_dim / 2) : 1;
  const int passes = (n_q_heads + n_kv_heads + head_groups - 1) / head_groups;
  int columns = 2048 / n_tokens;
  columns = columns < 1 ? 1 : (columns > passes ? passes : columns);
  const dim3 grid(n_tokens, columns);
  if (dtype == TL_F32)
    rope_kv_write_kernel<float><<<grid, threads, 0, stream>>>(
        (float*)qkv, n_q_heads, n_kv_heads, head_dim, positions, inv_freq, (const float2*)cos_sin, rotary_dim, pairing,
        (float*)k_pages, (float*)v_pages, slot_mapping, page_size);
  else if (dtype == TL_BF16)
    rope_kv_write_kernel<bf16_t><<<grid, threads, 0, stream>>>(
        (bf16_t*)qkv, n_q_heads, n_kv_heads, head_dim, positions, inv_freq, (const float2*)cos_sin, rotary_dim, pairing,
        (bf16_t*)k_pages, (bf16_t*)v_pages, slot_mapping, page_size);
  else
    return tl_fail(TL_ERR_ARG, "rope: unknown dtype %d", dtype);
  return tl_check_launch("rope_kv_write");
}

// ----------------------------------------------------------------------------- SwiGLU gate
// gate_up: [n, 2F] = gate | up.  out[n, F] = T(float(T(silu(gate))) * float(up)), silu(z) = z / (1 + e^-z).
// A thread takes V consecutive columns of one row (V elements = 16 bytes when the row allows it).
template <typename T, int V>
__global__ void silu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int n, int inter) {
  const int c0 = (blockIdx.x * blockDim.x + threadIdx.x) * V;
  if (c0 >= inter) return;
  for (int r = blockIdx.y; r < n; r += gridDim.y) {
    const T* gp = gate_up + (size_t)r * 2 * inter + c0;
    T* op = out + (size_t)r * inter + c0;
    struct alignas(sizeof(T) * V) Vec { T e[V]; };
    const Vec g = *reinterpret_cast<const Vec*>(gp);
    const Vec u = *reinterpret_cast<const Vec*>(gp + inter);
    Vec o;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const float gf = to_f32(g.e[i]);
      const float act = to_f32(from_f32<T>(gf / (1.0f + expf(-gf))));
      o.e[i] = from_f32<T>(act * to_f32(u.e[i]));
    }
    *reinterpret_cast<Vec*>(op) = o;
  }
}

template <typename T>
int silu_mul_launch(const T* gate_up, T* out, int n, int inter, hipStream_t stream) {
  constexpr int kVec = 16 / sizeof(T);
  const bool wide = inter % kVec == 0 && ((uintptr_t)gate_up % 16) == 0 && ((uintptr_t)out % 16) == 0;
  const int threads = 256;
  const int per_block = threads * (wide ? kVec : 1);
  const dim3 grid((inter + per_block - 1) / per_block, n < 65535 ? n : 65535);
  if (wide)
    silu_mul_kernel<T, kVec><<<grid, threads, 0, stream>>>(gate_up, out, n, inter);
  else
    silu_mul_kernel<T, 1><<<grid, threads, 0, stream>>>(gate_up, out, n, inter);
  return tl_check_launch("silu_mul");
}

TL_EXPORT int tl_silu_mul(const void* gate_up, void* out, int n, int inter, int dtype, hipStream_t stream) {
  TL_REQUIRE(n >= 0 && inter > 0, "silu_mul: bad sizes n=%d inter=%d", n, inter);
  if (n == 0) return TL_OK;
  if (dtype == TL_F32) return silu_mul_launch((const float*)gate_up, (float*)out, n, inter, stream);
  if (dtype == TL_BF16) return silu_mul_launch((const bf16_t*)gate_up, (bf16_t*)out, n, inter, stream);
  return tl_fail(TL_ERR_ARG, "silu_mul: unknown dtype %d", dtype);
}

// ----------------------------------------------------------------------------- bias
// x[n, width] += bias[width]  (sum in 32-bit, one rounding)
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ x, const T* __restrict__ bias, int n, int width, int row_stride) {
  const size_t total = (size_t)n * width;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * blockDim.x) {
    const size_t r = idx / width;
    const int c = (int)(idx % width);
    T* p = x + r * row_stride + c;
    *p = from_f32<T>(to_f32(*p) + to_f32(bias[c]));
  }
}

TL_EXPORT int tl_add_bias(void* x, const void* bias, int n, int width, int row_stride, int dtype,
                          hipStream_t stream) {
  TL_REQUIRE(n >= 0 && width > 0 && row_stride >= width, "add_bias: bad sizes");
  if (n == 0) return TL_OK;
  const size_t total = (size_t)n * width;
  const int threads = 256;
  const int blocks = (int)((total + threads - 1) / threads < 65536 ? (total + threads - 1) / threads : 65536);
  if (dtype == TL_F32)
    add_bias_kernel<float><<<blocks, threads, 0, stream>>>((float*)x, (const float*)bias, n, width, row_stride);
  else if (dtype == TL_BF16)
    add_bias_kernel<bf16_t><<<blocks, threads, 0, stream>>>((bf16_t*)x, (const bf16_t*)bias, n, width, row_stride);
  else
    return tl_fail(TL_ERR_ARG, "add_bias: unknown dtype %d", dtype);
  return tl_check_launch("add_bias");
}
