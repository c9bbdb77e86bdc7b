// An entry point that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory:
// code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
// The first call on a device looks up that device's copy of the buffer (hipGetSymbolAddress, under a
// mutex), which is not a launch: make it outside a capture, any later call is launches only.
#pragma once

#include <hip/hip_runtime.h>

// The most rows one call takes.  The two-stage argmax keeps 64 (value, index) pairs per row between
// its kernels: 512 KiB for 1,024 rows, in a fixed device array that every GPU the library runs on
// holds until the process ends.
#define LLMSERVE_ARGMAX_STATIC_MAX_ROWS 1024

// Returned (after a line on stderr) when `rows` exceeds LLMSERVE_ARGMAX_STATIC_MAX_ROWS.
#define LLMSERVE_ERR_TOO_LARGE 1002

// out[r] = index of the first maximum of logits[r, 0:vocab] (float32, row-major), as `llmserve_argmax`
// computes it with the same kernels, but with the pieces' results in the library's own fixed buffer
// instead of buffers the caller brings.  Calls no hipMalloc, hipFree or other allocating routine.
// The kernels go to `stream` on the current device; returns 0, a HIP error code, 1001 for a bad
// argument or LLMSERVE_ERR_TOO_LARGE.
// All calls on one GPU share that GPU's buffer, which keeps the last call's contents: calls that
// overlap on one GPU (different streams, different threads) race; calls on one stream do not.
extern "C" int llmserve_argmax_static(const float* logits, int* out, int rows, int vocab, hipStream_t stream);
