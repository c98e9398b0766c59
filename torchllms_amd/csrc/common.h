// Shared helpers of the gfx950 kernels: element types, wave-level reductions, error reporting.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define TL_EXPORT extern "C" __attribute__((visibility("default")))

// Element type codes of the C interface.
enum : int { TL_F32 = 0, TL_BF16 = 1 };

// Status codes of the C interface.  0 = launched.  Negative = refused before any launch.
enum : int { TL_OK = 0, TL_ERR_ARG = -1, TL_ERR_UNSUPPORTED = -2, TL_ERR_HIP = -3 };

constexpr int kWave = 64;  // wavefront width on CDNA

typedef __bf16 bf16_t;

// Records the message that tl_last_error() returns; returns `code`.
int tl_fail(int code, const char* fmt, ...);
// Checks hipGetLastError() after a launch.
int tl_check_launch(const char* what);

// What the current device says of itself (hipGetDeviceProperties, read once per device and process):
// its compute units and the bytes of LDS a block may use.  Launch rules and size checks take these,
// not a literal of the GPU they were first written for.
struct TlDeviceFacts {
  int compute_units;
  int lds_bytes;
};
const TlDeviceFacts& tl_device_facts();

#define TL_REQUIRE(cond, ...)                          \
  do {                                                 \
    if (!(cond)) return tl_fail(TL_ERR_ARG, __VA_ARGS__); \
  } while (0)

template <typename T>
__device__ __forceinline__ float to_f32(T v) {
  return static_cast<float>(v);
}
template <typename T>
__device__ __forceinline__ T from_f32(float v) {
  return static_cast<T>(v);
}

// Sum over the 64 lanes of a wave in a fixed butterfly order; every lane gets the result.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Sum over a block of `NWAVES` waves; `scratch` holds NWAVES floats of LDS.  The order of the
// additions is fixed, so the result does not depend on timing.
template <int NWAVES>
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int w = 0; w < NWAVES; ++w) total += scratch[w];
  return total;
}
