// An entry point for callers that cannot allocate device memory.
//
// This has no counterpart in the reference.  It exists for callers that may not call hipMalloc
// (or anything that does): code under HIP graph capture, tight serving loops, harnesses that
// forbid allocation.  tl_sample_chunks() takes a workspace (`candidates`) that somebody has to
// allocate; tl_sample_chunks_static() takes none: the winners of the row pieces go through a
// file-scope device array of fixed size inside the library.
//
//   * Limit: n_rows * (pieces actually used) <= TL_STATIC_CANDIDATES (8,192 candidates of 8 bytes,
//     64 KiB per GPU, held by every GPU the library runs on until the process ends).  A larger call
//     is refused with TL_ERR_ARG and a message; nothing is launched.
//   * Same kernels, same tokens as tl_sample_chunks() and tl_sample() without top-k.
//   * It calls no hipMalloc, hipFree or allocating library routine.  The array's device address is
//     looked up once per device (hipGetSymbolAddress) at the entry point's first call there.
//   * All calls on one GPU share that GPU's array: two calls that overlap in time on one GPU (on
//     different streams) race.  Calls on one stream are ordered and safe.  Nothing in the array has
//     to start at zero: every candidate a call reads was written by that call.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define TL_STATIC_CANDIDATES 8192

extern "C" __attribute__((visibility("default"))) int tl_sample_chunks_static(
    const float* logits, int row_stride, int n_rows, int vocab, const float* temperature, const uint64_t* seeds,
    const uint64_t* steps, int chunks, int32_t* out, hipStream_t stream);
