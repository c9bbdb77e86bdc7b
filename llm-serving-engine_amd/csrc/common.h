// Shared by every kernel file: element types, wave and block reductions, launch checks.
// Everything here is for gfx950 (CDNA4): 64-wide waves, MFMA, 160 KB LDS per CU.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;

#define WAVE 64

// Every entry point returns 0 or a HIP error code; the Python side raises on non-zero.
#define LAUNCH_STATUS() ((int)hipGetLastError())

// Argument errors that the host can detect before a launch.
#define ERR_BAD_ARGUMENT 1001

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return (bf16_t)v; }

// Loads element i of a tensor whose element type is chosen at run time (0: bf16, 1: float).
__device__ __forceinline__ float load_as_float(const void* base, int is_float, size_t i) {
  return is_float ? ((const float*)base)[i] : (float)((const bf16_t*)base)[i];
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int offset = WAVE / 2; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int offset = WAVE / 2; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  The order of the
// additions depends only on the block size, so equal inputs give equal bits in every launch.
__device__ __forceinline__ float block_sum(float v, float* shared /* >= 17 floats */) {
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, waves = (blockDim.x + WAVE - 1) / WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) shared[wave] = v;
  __syncthreads();
  float total = 0.f;  // every thread adds the waves' sums itself, in the same order
  for (int i = 0; i < waves; ++i) total += shared[i];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* shared /* >= 17 floats */) {
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, waves = (blockDim.x + WAVE - 1) / WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) shared[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    float best = shared[0];
    for (int i = 1; i < waves; ++i) best = fmaxf(best, shared[i]);
    shared[16] = best;
  }
  __syncthreads();
  return shared[16];
}

// Where a key lies in its page.  The keys of one (page, kv head) are kept in pieces of KEY_PIECE
// elements, the same piece of all the page's keys side by side: [dim / KEY_PIECE][page_size][KEY_PIECE].
// The matrix cores take a key as a row of their A operand, a lane holding eight elements of one key and
// its neighbours the same eight of the next keys: laid out like this, four neighbouring lanes read 64
// bytes in a row and the address unit serves them in one go, where whole rows (256 bytes apart at head
// size 128) took it four (prefill attention over 2,048 keys: 44 -> 31 us).  A head size that is no
// multiple of KEY_PIECE has one piece, the whole row.
#define KEY_PIECE 8
__device__ __host__ __forceinline__ int key_piece_width(int dim) { return dim % KEY_PIECE == 0 ? KEY_PIECE : dim; }
// element index of dimension d of the key at `offset`, counted from the start of its (page, kv head)
__device__ __forceinline__ size_t key_element(int d, int offset, int page_size, int dim) {
  const int width = key_piece_width(dim);
  return ((size_t)(d / width) * page_size + offset) * width + d % width;
}

// Where a value lies in its page.  Attention sums over keys, and the matrix cores want the summed index
// contiguous, so a page keeps its values transposed; and as with the keys a lane holds one piece (eight keys of
// one dimension) and its neighbours the same piece of the next dimensions, so the values of one (page, kv head)
// are kept in pieces of VALUE_PIECE keys, the same piece of all dimensions side by side:
// [page_size / VALUE_PIECE][dim][VALUE_PIECE].  Sixteen lanes then read 256 bytes in a row whatever the page size,
// where whole rows of keys ([dim][page_size]) lay page_size elements apart (a 64-key page: a cache line a lane,
// the prefill attention over 8,192 keys 474 us against 292 at 16-key pages).  A page size that is no multiple of
// VALUE_PIECE has one piece, the whole row of keys.
#define VALUE_PIECE 8
__device__ __host__ __forceinline__ int value_piece_width(int page_size) { return page_size % VALUE_PIECE == 0 ? VALUE_PIECE : page_size; }
// element index of dimension d of the value at `offset`, counted from the start of its (page, kv head)
__device__ __forceinline__ size_t value_element(int d, int offset, int page_size, int dim) {
  const int width = value_piece_width(page_size);
  return ((size_t)(offset / width) * dim + d) * width + offset % width;
}
