// Two micro-benchmarks that say what this GPU reaches at its current clocks, for the roofline figures
// of bench.py: a read of a large buffer with 16-byte loads (HBM bandwidth as a kernel can see it), and
// a loop of bfloat16 MFMA 16x16x32 instructions on registers alone (the matrix cores' issue rate).
// They are measurements, not model code: a library of their own, built when bench.py asks for it.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>

namespace {
char g_error[256];

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

// Every thread reads 16 bytes per round, rounds a whole grid apart; four loads are in flight per
// thread.  The xor of everything read decides a store that never happens, so no load can be dropped.
__global__ void __launch_bounds__(256) stream_read_kernel(const u32x4_t* __restrict__ p, size_t n_vec, unsigned int* sink) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  u32x4_t acc = {0u, 0u, 0u, 0u};
  for (; i + 3 * stride < n_vec; i += 4 * stride) {
    const u32x4_t a = __builtin_nontemporal_load(p + i);
    const u32x4_t b = __builtin_nontemporal_load(p + i + stride);
    const u32x4_t c = __builtin_nontemporal_load(p + i + 2 * stride);
    const u32x4_t d = __builtin_nontemporal_load(p + i + 3 * stride);
    acc ^= a ^ b ^ c ^ d;
  }
  for (; i < n_vec; i += stride) acc ^= __builtin_nontemporal_load(p + i);
  const unsigned int x = acc.x ^ acc.y ^ acc.z ^ acc.w;
  if (x == 0x9E3779B9u && sink) sink[0] = x;
}

// Eight independent accumulators per wave: an MFMA 16x16x32 has a latency of several issue slots, and
// only independent ones can follow each other back to back.
__global__ void __launch_bounds__(256) mfma_rate_kernel(int iters, float* sink) {
  const int lane = threadIdx.x % kWave;
  u32x4_t bits = {0x3F803F80u + lane, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};  // bfloat16 ones, more or less
  const bf16x8_t a = __builtin_bit_cast(bf16x8_t, bits);
  bits.y += 1u;
  const bf16x8_t b = __builtin_bit_cast(bf16x8_t, bits);
  float4_t acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = float4_t{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[j], 0, 0, 0);
  }
  float total = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) total += acc[j].x + acc[j].y + acc[j].z + acc[j].w;
  if (total == -1.f && sink) sink[0] = total;
}
// Sixteen independent 32-bit multiply-adds per lane and pass: what the vector units give the 32-bit
// path's products, which are plain FMAs (compiled, like everything here, without packed 32-bit
// instructions).
__global__ void __launch_bounds__(256) fma_rate_kernel(int iters, float* sink) {
  float acc[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) acc[j] = (float)(threadIdx.x + j);
  const float a = 1.0f + 1e-7f * (float)threadIdx.x, b = 1e-9f * (float)blockIdx.x;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[j] = __builtin_fmaf(acc[j], a, b);
  }
  float total = 0.f;
#pragma unroll
  for (int j = 0; j < 16; ++j) total += acc[j];
  if (total == -1.f && sink) sink[0] = total;
}
}  // namespace

TL_EXPORT const char* tl_variant_last_error() { return g_error; }

// Reads `bytes` (a multiple of 16) from `p` once with `blocks` blocks of 256 threads.
TL_EXPORT int tl_peak_stream_read(const void* p, size_t bytes, int blocks, void* sink, hipStream_t stream) {
  if (!p || bytes % 16 || blocks <= 0 || ((uintptr_t)p % 16)) return fail(TL_ERR_ARG, "peak_stream_read: bad arguments");
  stream_read_kernel<<<blocks, 256, 0, stream>>>((const u32x4_t*)p, bytes / 16, (unsigned int*)sink);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? TL_OK : fail(TL_ERR_HIP, "peak_stream_read: %s", hipGetErrorString(e));
}

// `blocks` blocks of four waves, each wave issuing iters * 8 MFMA 16x16x32 (2 * 16 * 16 * 32 flop each).
TL_EXPORT int tl_peak_mfma_bf16(int iters, int blocks, void* sink, hipStream_t stream) {
  if (iters <= 0 || blocks <= 0) return fail(TL_ERR_ARG, "peak_mfma_bf16: bad arguments");
  mfma_rate_kernel<<<blocks, 256, 0, stream>>>(iters, (float*)sink);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? TL_OK : fail(TL_ERR_HIP, "peak_mfma_bf16: %s", hipGetErrorString(e));
}

// `blocks` blocks of 256 threads, each thread doing iters * 16 multiply-adds (2 flop each).
TL_EXPORT int tl_peak_fma_f32(int iters, int blocks, void* sink, hipStream_t stream) {
  if (iters <= 0 || blocks <= 0) return fail(TL_ERR_ARG, "peak_fma_f32: bad arguments");
  fma_rate_kernel<<<blocks, 256, 0, stream>>>(iters, (float*)sink);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? TL_OK : fail(TL_ERR_HIP, "peak_fma_f32: %s", hipGetErrorString(e));
}
