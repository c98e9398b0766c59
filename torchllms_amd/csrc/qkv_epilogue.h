// The end of a query/key/value projection, shared by the matrix-product kernels that fuse it:
// rotation of query and key heads by position and the scatter of keys and values into their pages.
#pragma once

#include "common.h"

// What the epilogue needs beside the product.
struct QkvArgs {
  int n_q_heads, n_kv_heads, head_dim;
  int rotary_dim;                 // leading channels of a head that rotate (even; 0: none)
  const float2* cos_sin;          // [row of A][rotary_dim / 2] = (cos, sin) of the row's position
  bf16_t* k_pages;                // [page][kv head][page_size][head_dim], or null: keys and values stay in C
  bf16_t* v_pages;
  const int32_t* slot_mapping;    // per row of A: page * page_size + offset, < 0: not stored
  int page_size;
};

// What the epilogue reads from memory for one thread's four columns: the cosines and sines of its two
// rotary pairs and its row's place in the pages.  Fetched apart from the arithmetic so that a kernel
// can ask for them together with everything else it loads (indices are clamped to what exists; what
// a thread does not need it does not use).
struct QkvOperands {
  float2 cs[2];
  int slot;
};

__device__ __forceinline__ QkvOperands qkv_fetch(int row, int n, const QkvArgs& qa) {
  QkvOperands o;
  const int half = qa.rotary_dim / 2;
  const int pair = (n % qa.head_dim) / 2;
  o.cs[0] = o.cs[1] = float2{1.f, 0.f};
  if (half > 0) {
    o.cs[0] = qa.cos_sin[(size_t)row * half + min(pair, half - 1)];
    o.cs[1] = qa.cos_sin[(size_t)row * half + min(pair + 1, half - 1)];
  }
  o.slot = qa.k_pages != nullptr ? qa.slot_mapping[row] : -1;
  return o;
}

// sums[0..3]: the 32-bit products of row `row` and columns n .. n + 3, which are channels d .. d + 3
// of one head (the host checks head_dim % 4 == 0): two rotary pairs (interleaved pairing).  They are
// rounded to bfloat16 first, as the stored product of the unfused sequence would read, rotated in
// 32-bit, rounded again and stored: queries into C, keys and values into their pages (or into C when
// there are no pages).
__device__ __forceinline__ void qkv_finish(const float* sums, int row, int n, const QkvArgs& qa, bf16_t* C, int ldc,
                                           const QkvOperands& o) {
  typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
  const int head = n / qa.head_dim;
  const int d = n % qa.head_dim;
  float x[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) x[i] = to_f32(from_f32<bf16_t>(sums[i]));
  if (head < qa.n_q_heads + qa.n_kv_heads) {
#pragma unroll
    for (int pi = 0; pi < 2; ++pi) {
      if (d + 2 * pi < qa.rotary_dim) {
        const float2 cs = o.cs[pi];
        const float x0 = x[2 * pi], x1 = x[2 * pi + 1];
        x[2 * pi] = x0 * cs.x - x1 * cs.y;
        x[2 * pi + 1] = x1 * cs.x + x0 * cs.y;
      }
    }
  }
  const u32x2_t packed = {
      (uint32_t)__builtin_bit_cast(uint16_t, from_f32<bf16_t>(x[0])) | ((uint32_t)__builtin_bit_cast(uint16_t, from_f32<bf16_t>(x[1])) << 16),
      (uint32_t)__builtin_bit_cast(uint16_t, from_f32<bf16_t>(x[2])) | ((uint32_t)__builtin_bit_cast(uint16_t, from_f32<bf16_t>(x[3])) << 16)};
  bf16_t* dst = C + (size_t)row * ldc + n;
  bool store = true;
  if (head >= qa.n_q_heads && qa.k_pages != nullptr) {
    const int slot = o.slot;
    store = slot >= 0;
    const int kvh = head < qa.n_q_heads + qa.n_kv_heads ? head - qa.n_q_heads : head - qa.n_q_heads - qa.n_kv_heads;
    bf16_t* pages = head < qa.n_q_heads + qa.n_kv_heads ? qa.k_pages : qa.v_pages;
    const int page = store ? slot / qa.page_size : 0;
    const int off = store ? slot % qa.page_size : 0;
    dst = pages + (((size_t)page * qa.n_kv_heads + kvh) * qa.page_size + off) * qa.head_dim + d;
  }
  if (store) *reinterpret_cast<u32x2_t*>(dst) = packed;
}

__device__ __forceinline__ void qkv_finish(const float* sums, int row, int n, const QkvArgs& qa, bf16_t* C, int ldc) {
  qkv_finish(sums, row, n, qa, C, ldc, qkv_fetch(row, n, qa));
}

// The argument checks of the entry points that take these arguments; fills `qa`.
inline int qkv_args(const char* who, int n_q_heads, int n_kv_heads, int head_dim, int rotary_dim, const float* cos_sin,
                    void* k_pages, void* v_pages, const int32_t* slot_mapping, int page_size, const void* C, int ldc,
                    QkvArgs* qa) {
  if (!(n_q_heads > 0 && n_kv_heads >= 0 && head_dim > 0 && head_dim % 4 == 0)) return tl_fail(TL_ERR_ARG, "%s: bad head sizes", who);
  if (!(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0)) return tl_fail(TL_ERR_ARG, "%s: bad rotary_dim=%d", who, rotary_dim);
  if (rotary_dim != 0 && cos_sin == nullptr) return tl_fail(TL_ERR_ARG, "%s: the table of cosines and sines is missing", who);
  if (k_pages != nullptr && !(v_pages != nullptr && slot_mapping != nullptr && page_size > 0))
    return tl_fail(TL_ERR_ARG, "%s: pages given without v_pages/slot_mapping/page_size", who);
  if (!(ldc % 4 == 0 && ((uintptr_t)C % 8) == 0)) return tl_fail(TL_ERR_ARG, "%s: rows of C must start on 8-byte boundaries", who);
  qa->n_q_heads = n_q_heads; qa->n_kv_heads = n_kv_heads; qa->head_dim = head_dim; qa->rotary_dim = rotary_dim;
  qa->cos_sin = (const float2*)cos_sin; qa->k_pages = (bf16_t*)k_pages; qa->v_pages = (bf16_t*)v_pages;
  qa->slot_mapping = slot_mapping; qa->page_size = page_size;
  return TL_OK;
}
