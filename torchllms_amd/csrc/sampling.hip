// Next-token choice from 32-bit logits, one block per row, or several blocks per row and a second
// kernel that picks among their candidates (same result: maxima and the race's winner do not depend
// on the order in which elements are visited).
//   temperature == 0 : argmax(logits), the lowest index among equal maxima.
//   temperature  > 0 : x = logits / max(temperature, 1e-5); optionally everything below the k-th
//                      largest x is dropped (ties kept); the token is argmax_i exp(x_i - max x) / q_i
//                      with q_i ~ Exponential(1): an exponential race, which draws from softmax(x).
// q_i comes from a counter-based generator (Philox 4x32-10) keyed by the row's seed; the counter is
// (i / 4, step), so a row's draw depends on its own seed and step only, never on the batch.
#include "common.h"
#include "no_alloc.h"

#include <mutex>

namespace {

constexpr int kThreads = 1024;
constexpr int kWaves = kThreads / kWave;

__device__ __forceinline__ void philox_round(uint32_t (&c)[4], uint32_t k0, uint32_t k1) {
  const uint64_t p0 = (uint64_t)0xD2511F53u * c[0];
  const uint64_t p1 = (uint64_t)0xCD9E8D57u * c[2];
  const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0;
  const uint32_t n1 = (uint32_t)p1;
  const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1;
  const uint32_t n3 = (uint32_t)p0;
  c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
}

// Four 32-bit words for (block index `blk`, step) under `seed`.
__device__ __forceinline__ void philox4(uint64_t seed, uint32_t blk, uint64_t step, uint32_t (&out)[4]) {
  uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
  uint32_t c[4] = {blk, (uint32_t)step, (uint32_t)(step >> 32), 0u};
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    philox_round(c, k0, k1);
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c[0]; out[1] = c[1]; out[2] = c[2]; out[3] = c[3];
}

// Uniform in (0, 1): 24 random bits, centred in their cell, so neither 0 nor 1 can occur.
__device__ __forceinline__ float uniform_open(uint32_t bits) {
  return ((float)(bits >> 8) + 0.5f) * (1.0f / 16777216.0f);
}

__device__ __forceinline__ float uniform_at(uint64_t seed, uint64_t step, int i) {
  uint32_t r[4];
  philox4(seed, (uint32_t)i >> 2, step, r);
  return uniform_open(r[i & 3]);
}

// Order-preserving map float -> uint32 (larger float, larger key).
__device__ __forceinline__ uint32_t float_key(float v) {
  const uint32_t u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct Best {
  float val;
  int idx;
};
__device__ __forceinline__ Best better(Best a, Best b) {
  if (b.val > a.val || (b.val == a.val && b.idx < a.idx)) return b;
  return a;
}
__device__ __forceinline__ Best block_best(Best v, Best* scratch) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    Best o;
    o.val = __shfl_xor(v.val, off, kWave);
    o.idx = __shfl_xor(v.idx, off, kWave);
    v = better(v, o);
  }
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  Best total = scratch[0];
  for (int w = 1; w < kWaves; ++w) total = better(total, scratch[w]);
  return total;
}

// The thread's share of argmax(x): 16-byte loads, four of them in flight, where the row allows it.
// `better` keeps the lowest index among equal maxima whatever the order of the visits.
__device__ __forceinline__ Best row_best(const float* __restrict__ x, int vocab, int tid) {
  constexpr int kNone = 0x7fffffff;
  Best b = {-INFINITY, kNone};
  int done = 0;
  if ((reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    const int n4 = vocab / 4;
    const float4* x4 = reinterpret_cast<const float4*>(x);
    int i = tid;
    for (; i + 3 * kThreads < n4; i += 4 * kThreads) {
      float4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = x4[i + u * kThreads];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int at = 4 * (i + u * kThreads);
        b = better(b, Best{v[u].x, at});
        b = better(b, Best{v[u].y, at + 1});
        b = better(b, Best{v[u].z, at + 2});
        b = better(b, Best{v[u].w, at + 3});
      }
    }
    for (; i < n4; i += kThreads) {
      const float4 v = x4[i];
      b = better(b, Best{v.x, 4 * i});
      b = better(b, Best{v.y, 4 * i + 1});
      b = better(b, Best{v.z, 4 * i + 2});
      b = better(b, Best{v.w, 4 * i + 3});
    }
    done = 4 * n4;
  }
  for (int i = done + tid; i < vocab; i += kThreads) b = better(b, Best{x[i], i});
  return b;
}

// The race over indices [lo, hi) of a row scaled by 1 / tdiv, with maximum m of the scaled row:
// each thread handles whole groups of four indices, so one generator call serves four draws; an
// aligned row gives the four logits in one 16-byte load.  lo is a multiple of 4.
__device__ __forceinline__ Best race(const float* __restrict__ x, int lo, int hi, float tdiv, float m, float pivot,
                                     uint64_t seed, uint64_t step, int tid) {
  constexpr int kNone = 0x7fffffff;
  Best b = {-INFINITY, kNone};
  const bool wide = (reinterpret_cast<uintptr_t>(x) & 15) == 0;
  for (int i4 = lo + tid * 4; i4 < hi; i4 += kThreads * 4) {
    uint32_t r[4];
    philox4(seed, (uint32_t)i4 >> 2, step, r);
    float xs[4];
    if (wide && i4 + 3 < hi) {
      const float4 v = *reinterpret_cast<const float4*>(x + i4);
      xs[0] = v.x; xs[1] = v.y; xs[2] = v.z; xs[3] = v.w;
    } else {
#pragma unroll
      for (int u = 0; u < 4; ++u) xs[u] = i4 + u < hi ? x[i4 + u] : -INFINITY;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i4 + u;
      if (i >= hi) break;
      const float xi = xs[u] / tdiv;
      if (xi < pivot) continue;
      const float q = -logf(uniform_open(r[u]));
      b = better(b, Best{expf(xi - m) / q, i});
    }
  }
  return b;
}

__global__ void __launch_bounds__(kThreads)
sample_kernel(const float* __restrict__ logits, int row_stride, int vocab,
              const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
              const uint64_t* __restrict__ seeds, const uint64_t* __restrict__ steps,
              int32_t* __restrict__ out) {
  __shared__ Best best_scratch[kWaves];
  __shared__ uint32_t hist[256];
  __shared__ uint32_t sel_prefix, sel_remaining;
  const int row = blockIdx.x;
  const float* x = logits + (size_t)row * row_stride;
  const float temp = temperature[row];
  const int tid = threadIdx.x;
  constexpr int kNone = 0x7fffffff;

  if (temp == 0.f) {
    const Best b = block_best(row_best(x, vocab, tid), best_scratch);
    if (tid == 0) out[row] = b.idx;
    return;
  }
  const float tdiv = fmaxf(temp, 1e-5f);

  // k-th largest scaled logit by radix selection over the order-preserving keys, 8 bits a pass
  float pivot = -INFINITY;
  int k = top_k ? top_k[row] : 0;
  if (k > 0 && k < vocab) {
    if (tid == 0) {
      sel_prefix = 0;
      sel_remaining = (uint32_t)k;
    }
    for (int shift = 24; shift >= 0; shift -= 8) {
      for (int i = tid; i < 256; i += kThreads) hist[i] = 0;
      __syncthreads();
      const uint32_t prefix = sel_prefix;
      const uint32_t mask = shift == 24 ? 0u : (0xFFFFFFFFu << (shift + 8));
      for (int i = tid; i < vocab; i += kThreads) {
        const uint32_t key = float_key(x[i] / tdiv);
        if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
      }
      __syncthreads();
      if (tid == 0) {
        uint32_t remaining = sel_remaining;
        int bin = 255;
        for (; bin > 0; --bin) {
          if (hist[bin] >= remaining) break;
          remaining -= hist[bin];
        }
        sel_prefix = prefix | ((uint32_t)bin << shift);
        sel_remaining = remaining;
      }
      __syncthreads();
    }
    const uint32_t key = sel_prefix;
    const uint32_t u = (key & 0x80000000u) ? (key & 0x7FFFFFFFu) : ~key;
    pivot = __uint_as_float(u);
  }

  // the largest scaled logit: dividing by a positive number keeps the order, so the maximum of the
  // raw row is found with wide loads and scaled once
  const float m = block_best(row_best(x, vocab, tid), best_scratch).val / tdiv;

  const uint64_t seed = seeds[row];
  const uint64_t step = steps[row];
  Best b = race(x, 0, vocab, tdiv, m, pivot, seed, step, tid);
  b = block_best(b, best_scratch);
  if (tid == 0) out[row] = b.idx;
}

// Several blocks per row (no top-k): block (chunk, row) finds the row's maximum by itself (the row
// is read from L2 by all but the first to come) and runs the race, or the argmax, over its chunk of
// `chunk_len` indices (a multiple of 4); candidates[row][chunk] receives its winner.
__global__ void __launch_bounds__(kThreads)
sample_chunks_kernel(const float* __restrict__ logits, int row_stride, int vocab, const float* __restrict__ temperature,
                     const uint64_t* __restrict__ seeds, const uint64_t* __restrict__ steps, int chunk_len,
                     Best* __restrict__ candidates) {
  __shared__ Best best_scratch[kWaves];
  const int row = blockIdx.y;
  const int chunk = blockIdx.x;
  const float* x = logits + (size_t)row * row_stride;
  const float temp = temperature[row];
  const int tid = threadIdx.x;
  const int lo = chunk * chunk_len;
  const int hi = min(lo + chunk_len, vocab);
  Best b;
  if (temp == 0.f) {
    b = row_best(x + lo, hi - lo, tid);  // (lo * 4 bytes is a multiple of 16: the chunk is aligned as the row is)
    if (b.idx != 0x7fffffff) b.idx += lo;
  } else {
    const float tdiv = fmaxf(temp, 1e-5f);
    const float m = block_best(row_best(x, vocab, tid), best_scratch).val / tdiv;
    b = race(x, lo, hi, tdiv, m, -INFINITY, seeds[row], steps[row], tid);
  }
  b = block_best(b, best_scratch);
  if (tid == 0) candidates[(size_t)row * gridDim.x + chunk] = b;
}

__global__ void __launch_bounds__(kWave)
sample_pick_kernel(const Best* __restrict__ candidates, int chunks, int32_t* __restrict__ out) {
  const int row = blockIdx.x;
  Best b = {-INFINITY, 0x7fffffff};
  for (int c = threadIdx.x; c < chunks; c += kWave) b = better(b, candidates[(size_t)row * chunks + c]);
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    Best o;
    o.val = __shfl_xor(b.val, off, kWave);
    o.idx = __shfl_xor(b.idx, off, kWave);
    b = better(b, o);
  }
  if (threadIdx.x == 0) out[row] = b.idx;
}

__global__ void philox_uniform_kernel(uint64_t seed, uint64_t step, float* out, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = uniform_at(seed, step, i);
}

}  // namespace

// logits: [n_rows, vocab] 32-bit with row stride `row_stride`.  temperature[n_rows]; top_k[n_rows] or
// null (entries <= 0: no cut); seeds[n_rows], steps[n_rows]: generator key and counter of each row.
TL_EXPORT int tl_sample(const float* logits, int row_stride, int n_rows, int vocab, const float* temperature,
                        const int32_t* top_k, const uint64_t* seeds, const uint64_t* steps, int32_t* out,
                        hipStream_t stream) {
  TL_REQUIRE(n_rows >= 0 && vocab > 0 && row_stride >= vocab, "sample: bad sizes");
  TL_REQUIRE(temperature && seeds && steps && out, "sample: null argument");
  if (n_rows == 0) return TL_OK;
  sample_kernel<<<n_rows, kThreads, 0, stream>>>(logits, row_stride, vocab, temperature, top_k, seeds, steps, out);
  return tl_check_launch("sample");
}

// Both kernels of the choice in pieces; `candidates` holds n_rows * used entries.
static int launch_sample_chunks(const float* logits, int row_stride, int n_rows, int vocab, const float* temperature,
                                const uint64_t* seeds, const uint64_t* steps, int chunk_len, int used, Best* candidates,
                                int32_t* out, hipStream_t stream) {
  sample_chunks_kernel<<<dim3(used, n_rows), kThreads, 0, stream>>>(logits, row_stride, vocab, temperature, seeds, steps,
                                                                   chunk_len, candidates);
  int rc = tl_check_launch("sample_chunks");
  if (rc != TL_OK) return rc;
  sample_pick_kernel<<<n_rows, kWave, 0, stream>>>(candidates, used, out);
  return tl_check_launch("sample_pick");
}

// The same choice without top-k, every row cut into `chunks` pieces that blocks of their own work
// on: for few rows of a large vocabulary, where one block per row leaves most of the GPU idle.
// candidates: workspace of n_rows * chunks * 8 bytes.  The tokens equal tl_sample's.
TL_EXPORT int tl_sample_chunks(const float* logits, int row_stride, int n_rows, int vocab, const float* temperature,
                               const uint64_t* seeds, const uint64_t* steps, int chunks, void* candidates,
                               int32_t* out, hipStream_t stream) {
  TL_REQUIRE(n_rows >= 0 && vocab > 0 && row_stride >= vocab, "sample_chunks: bad sizes");
  TL_REQUIRE(temperature && seeds && steps && out && candidates, "sample_chunks: null argument");
  TL_REQUIRE(chunks >= 1 && chunks <= 1024 && n_rows <= 65535, "sample_chunks: chunks must be 1..1024, rows at most 65535");
  TL_REQUIRE(row_stride % 4 == 0 && ((uintptr_t)logits % 16) == 0, "sample_chunks: rows must start on 16-byte boundaries");
  if (n_rows == 0) return TL_OK;
  const int chunk_len = ((vocab + chunks - 1) / chunks + 3) / 4 * 4;
  const int used = (vocab + chunk_len - 1) / chunk_len;  // no chunk is empty
  return launch_sample_chunks(logits, row_stride, n_rows, vocab, temperature, seeds, steps, chunk_len, used,
                              (Best*)candidates, out, stream);
}

// ----------------------------------------------------------------------------- without a workspace
// The candidates of tl_sample_chunks_static (see no_alloc.h).  In host code this name is a stand-in,
// not a device address: the address on each GPU comes from hipGetSymbolAddress, once per device.
// (No `used` attribute here: with it the compiler keeps the device-side symbol local, and the
// runtime, which looks the array up by name in the code object, aborts the process.)
static __device__ __align__(256) unsigned char scratch[TL_STATIC_CANDIDATES * sizeof(Best)];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};  // per device: where that GPU holds its copy of `scratch`

// The current device's copy of `scratch`; looked up at the first call on that device.
int static_candidates(Best** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return tl_fail(TL_ERR_HIP, "sample_chunks_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return tl_fail(TL_ERR_UNSUPPORTED, "sample_chunks_static: device %d beyond %d", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return tl_fail(TL_ERR_HIP, "sample_chunks_static: hipGetSymbolAddress on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *ptr = (Best*)g_scratch_ptr[dev];
  return TL_OK;
}
}  // namespace

// tl_sample_chunks with the candidates in the library's own fixed array: allocates nothing.  The
// stream must belong to the current device.  Calls that overlap on one GPU race (no_alloc.h).
TL_EXPORT int tl_sample_chunks_static(const float* logits, int row_stride, int n_rows, int vocab,
                                      const float* temperature, const uint64_t* seeds, const uint64_t* steps, int chunks,
                                      int32_t* out, hipStream_t stream) {
  TL_REQUIRE(n_rows >= 0 && vocab > 0 && row_stride >= vocab, "sample_chunks_static: bad sizes");
  TL_REQUIRE(logits && temperature && seeds && steps && out, "sample_chunks_static: null argument");
  TL_REQUIRE(chunks >= 1 && chunks <= 1024 && n_rows <= 65535,
             "sample_chunks_static: chunks must be 1..1024, rows at most 65535");
  TL_REQUIRE(row_stride % 4 == 0 && ((uintptr_t)logits % 16) == 0,
             "sample_chunks_static: rows must start on 16-byte boundaries");
  if (n_rows == 0) return TL_OK;
  const int chunk_len = ((vocab + chunks - 1) / chunks + 3) / 4 * 4;
  const int used = (vocab + chunk_len - 1) / chunk_len;
  TL_REQUIRE((long long)n_rows * used <= TL_STATIC_CANDIDATES,
             "sample_chunks_static: %d rows in %d pieces need %lld candidates, the fixed array holds %d", n_rows, used,
             (long long)n_rows * used, TL_STATIC_CANDIDATES);
  Best* candidates = nullptr;
  int rc = static_candidates(&candidates);
  if (rc != TL_OK) return rc;
  return launch_sample_chunks(logits, row_stride, n_rows, vocab, temperature, seeds, steps, chunk_len, used, candidates, out,
                              stream);
}

// The uniforms the sampler uses for (seed, step), indices 0..n-1; for tests of the sampler.
TL_EXPORT int tl_philox_uniform(uint64_t seed, uint64_t step, float* out, int n, hipStream_t stream) {
  TL_REQUIRE(n >= 0, "philox_uniform: bad size");
  if (n == 0) return TL_OK;
  philox_uniform_kernel<<<(n + 255) / 256, 256, 0, stream>>>(seed, step, out, n);
  return tl_check_launch("philox_uniform");
}
