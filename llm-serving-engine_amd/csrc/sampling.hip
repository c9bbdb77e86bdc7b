// Choosing the next token from float32 logits: argmax, temperature sampling, top-p.
//
// The reference samples with torch.multinomial from a per-request generator
// (engine.py:29-72).  A generator's stream cannot be reproduced here, so the engine defines
// its own rule, the same in its plain implementation: the host passes one uniform u in
// [0, 1) per row (a counter-based draw from the request's seed and its number of sampled
// tokens) and the kernel inverts the distribution's CDF at u:
//   top_p >= 1: p = softmax(logits / T); token = first index whose running sum of p, in
//               index order, exceeds u * sum(p);
//   top_p <  1: entries are ranked by descending p (ties by ascending index); an entry is
//               kept if the mass ranked before it is < top_p (engine.py:34-37); token =
//               first kept entry, in rank order, whose running sum exceeds u * (kept mass).
// Sums are accumulated in float64 in an order fixed by the block size.
#include "common.h"
#include "no_alloc.h"

#include <mutex>
#include <stdio.h>

#define SAMPLE_THREADS 1024

__device__ __forceinline__ double block_sum_f64(double v, double* shared /* >= 17 */) {
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, waves = blockDim.x / WAVE;
#pragma unroll
  for (int offset = WAVE / 2; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, WAVE);
  __syncthreads();
  if (lane == 0) shared[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    double total = 0.0;
    for (int i = 0; i < waves; ++i) total += shared[i];
    shared[16] = total;
  }
  __syncthreads();
  return shared[16];
}

// (value, index) of the first maximum of a row; every thread gets it.
__device__ __forceinline__ void block_argmax(const float* row, int n, float* best_value, int* best_index,
                                             float* shared_v, int* shared_i) {
  float value = -INFINITY;
  int index = 0x7fffffff;  // no entry seen yet
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = row[i];
    if (v > value || index == 0x7fffffff) {  // strided indices ascend, so ties keep the first
      value = v;
      index = i;
    }
  }
#pragma unroll
  for (int offset = WAVE / 2; offset > 0; offset >>= 1) {
    const float ov = __shfl_xor(value, offset, WAVE);
    const int oi = __shfl_xor(index, offset, WAVE);
    if (ov > value || (ov == value && oi < index)) {
      value = ov;
      index = oi;
    }
  }
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, waves = blockDim.x / WAVE;
  __syncthreads();
  if (lane == 0) {
    shared_v[wave] = value;
    shared_i[wave] = index;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float bv = shared_v[0];
    int bi = shared_i[0];
    for (int i = 1; i < waves; ++i)
      if (shared_v[i] > bv || (shared_v[i] == bv && shared_i[i] < bi)) {
        bv = shared_v[i];
        bi = shared_i[i];
      }
    shared_v[16] = bv;
    shared_i[16] = bi;
  }
  __syncthreads();
  *best_value = shared_v[16];
  *best_index = shared_i[16];
}

// Two stages, so that a few rows still fill the chip: each row is cut into `pieces` pieces,
// a block finds the first maximum of its piece, and one more block per row picks among them.
__global__ __launch_bounds__(SAMPLE_THREADS) void argmax_pieces_kernel(const float* __restrict__ logits,
                                                                       float* __restrict__ piece_values,
                                                                       int* __restrict__ piece_indices, int vocab,
                                                                       int pieces) {
  __shared__ float sv[17];
  __shared__ int si[17];
  const int per = (vocab + pieces - 1) / pieces;
  const int begin = min(vocab, (int)blockIdx.y * per), count = min(vocab, begin + per) - begin;
  float value;
  int index;
  block_argmax(logits + (size_t)blockIdx.x * vocab + begin, count, &value, &index, sv, si);
  if (threadIdx.x == 0) {
    piece_values[blockIdx.x * pieces + blockIdx.y] = count > 0 ? value : -INFINITY;
    piece_indices[blockIdx.x * pieces + blockIdx.y] = count > 0 ? begin + index : 0x7fffffff;
  }
}

__global__ void argmax_pick_kernel(const float* __restrict__ piece_values, const int* __restrict__ piece_indices,
                                   int* __restrict__ out, int pieces) {
  // one wave per row; pieces ascend in index, so the first maximum among them is the row's
  float value = -INFINITY;
  int index = 0x7fffffff;
  for (int i = threadIdx.x; i < pieces; i += WAVE) {
    const float v = piece_values[blockIdx.x * pieces + i];
    const int at = piece_indices[blockIdx.x * pieces + i];
    if (at != 0x7fffffff && (v > value || index == 0x7fffffff)) {
      value = v;
      index = at;
    }
  }
#pragma unroll
  for (int offset = WAVE / 2; offset > 0; offset >>= 1) {
    const float ov = __shfl_xor(value, offset, WAVE);
    const int oi = __shfl_xor(index, offset, WAVE);
    if (oi != 0x7fffffff && (index == 0x7fffffff || ov > value || (ov == value && oi < index))) {
      value = ov;
      index = oi;
    }
  }
  if (threadIdx.x == 0) out[blockIdx.x] = index == 0x7fffffff ? 0 : index;
}

#define ARGMAX_PIECES 64

// Into how many pieces a row is cut: 64 for a few rows (so that they fill the chip), fewer for many (a piece
// of 2,400 logits leaves a thread of its block two or three of them and the block's reduction dominates:
// 64 rows of 151,936 took 33 us in 64 pieces each).  About a thousand blocks in all, at least 8 pieces a row.
static int argmax_pieces(int rows) {
  int pieces = ARGMAX_PIECES;
  while (pieces > 8 && rows * pieces > 1024) pieces /= 2;
  return pieces;
}

// scratch: at least rows * 64 floats and rows * 64 ints
extern "C" int llmserve_argmax(const float* logits, float* piece_values, int* piece_indices, int* out, int rows,
                               int vocab, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0) return ERR_BAD_ARGUMENT;
  const int pieces = argmax_pieces(rows);
  hipLaunchKernelGGL(argmax_pieces_kernel, dim3(rows, pieces), dim3(SAMPLE_THREADS), 0, stream, logits,
                     piece_values, piece_indices, vocab, pieces);
  hipLaunchKernelGGL(argmax_pick_kernel, dim3(rows), dim3(WAVE), 0, stream, piece_values, piece_indices, out, pieces);
  return LAUNCH_STATUS();
}

// The pieces' (value, index) pairs of `llmserve_argmax_static`: values first, then indices.  Each GPU
// holds its own copy of the array at its own address; host code reaches it only through the address
// that hipGetSymbolAddress gave for that device, never through the array's name.
#define ARGMAX_STATIC_SLOTS (LLMSERVE_ARGMAX_STATIC_MAX_ROWS * ARGMAX_PIECES)
static __device__ __align__(256) unsigned char argmax_static_scratch[ARGMAX_STATIC_SLOTS * (sizeof(float) + sizeof(int))];

#define ARGMAX_STATIC_MAX_DEVICES 64
static void* argmax_static_address[ARGMAX_STATIC_MAX_DEVICES];  // by device; null until that device's first call
static std::mutex argmax_static_lock;

extern "C" int llmserve_argmax_static(const float* logits, int* out, int rows, int vocab, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0) return ERR_BAD_ARGUMENT;
  if (rows > LLMSERVE_ARGMAX_STATIC_MAX_ROWS) {
    fprintf(stderr, "llmserve_argmax_static: %d rows are more than the %d its fixed scratch buffer holds\n", rows,
            LLMSERVE_ARGMAX_STATIC_MAX_ROWS);
    return LLMSERVE_ERR_TOO_LARGE;
  }
  int device = -1;
  hipError_t status = hipGetDevice(&device);
  if (status != hipSuccess) return (int)status;
  if (device < 0 || device >= ARGMAX_STATIC_MAX_DEVICES) return ERR_BAD_ARGUMENT;
  void* base = nullptr;
  {
    std::lock_guard<std::mutex> guard(argmax_static_lock);
    base = argmax_static_address[device];
    if (base == nullptr) {  // once per device, with that device current
      status = hipGetSymbolAddress(&base, HIP_SYMBOL(argmax_static_scratch));
      if (status != hipSuccess || base == nullptr) return status != hipSuccess ? (int)status : ERR_BAD_ARGUMENT;
      argmax_static_address[device] = base;
    }
  }
  // Nothing has to start at zero: the first kernel writes every slot that the second one reads.
  float* piece_values = (float*)base;
  int* piece_indices = (int*)((unsigned char*)base + ARGMAX_STATIC_SLOTS * sizeof(float));
  const int pieces = argmax_pieces(rows);
  hipLaunchKernelGGL(argmax_pieces_kernel, dim3(rows, pieces), dim3(SAMPLE_THREADS), 0, stream, logits,
                     piece_values, piece_indices, vocab, pieces);
  hipLaunchKernelGGL(argmax_pick_kernel, dim3(rows), dim3(WAVE), 0, stream, piece_values, piece_indices, out, pieces);
  return LAUNCH_STATUS();
}

// Mass and number of the entries of p whose bits are above `threshold` (p >= 0, so float
// order is the order of the bit patterns).
__device__ __forceinline__ double mass_above(const float* p, int n, unsigned threshold, double* shared) {
  double mass = 0.0;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = p[i];
    if (__float_as_uint(v) > threshold) mass += (double)v;
  }
  return block_sum_f64(mass, shared);
}

// Smallest bit pattern t in [0, top] with mass_above(t) < limit (strict) or <= limit.
__device__ __forceinline__ unsigned lowest_threshold(const float* p, int n, unsigned top, double limit, bool strict,
                                                     double* shared) {
  unsigned low = 0, high = top;  // the predicate holds at `high`
  while (low < high) {
    const unsigned middle = low + (high - low) / 2;
    const double mass = mass_above(p, n, middle, shared);
    const bool holds = strict ? mass < limit : mass <= limit;
    if (holds) high = middle; else low = middle + 1;
  }
  return high;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(const float* __restrict__ logits,
                                                                const float* __restrict__ temperatures,
                                                                const float* __restrict__ top_ps,
                                                                const float* __restrict__ uniforms,
                                                                float* __restrict__ scratch, int* __restrict__ out,
                                                                int vocab) {
  __shared__ float sv[17];
  __shared__ int si[17];
  __shared__ double sd[17];
  __shared__ double chunk_sums[SAMPLE_THREADS];
  __shared__ int found;
  const float* row = logits + (size_t)blockIdx.x * vocab;
  float* p = scratch + (size_t)blockIdx.x * vocab;
  const float temperature = temperatures[blockIdx.x];
  float best;
  int best_index;
  block_argmax(row, vocab, &best, &best_index, sv, si);
  if (temperature <= 0.f) {  // engine.py:30-31
    if (threadIdx.x == 0) out[blockIdx.x] = best_index;
    return;
  }
  // p = exp((logit - max) / T), not yet divided by its sum Z (engine.py:32)
  const float top_logit = best / temperature;
  double partial = 0.0;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float v = expf(row[i] / temperature - top_logit);
    p[i] = v;
    partial += (double)v;
  }
  const double total = block_sum_f64(partial, sd);
  const float top_p = top_ps[blockIdx.x];
  const double u = (double)uniforms[blockIdx.x];
  __syncthreads();

  if (top_p >= 1.f) {
    // inverse CDF in index order: each thread owns a contiguous run of entries
    const int per = (vocab + blockDim.x - 1) / blockDim.x;
    const int begin = min(vocab, (int)threadIdx.x * per), end = min(vocab, begin + per);
    double mine = 0.0;
    for (int i = begin; i < end; ++i) mine += (double)p[i];
    chunk_sums[threadIdx.x] = mine;
    if (threadIdx.x == 0) found = vocab - 1;
    __syncthreads();
    if (threadIdx.x == 0) {
      const double target = u * total;
      double running = 0.0;
      int owner = -1;
      for (int t = 0; t < (int)blockDim.x; ++t) {
        if (running + chunk_sums[t] > target) { owner = t; break; }
        running += chunk_sums[t];
      }
      if (owner >= 0) {
        const int b = min(vocab, owner * per), e = min(vocab, b + per);
        for (int i = b; i < e; ++i) {
          running += (double)p[i];
          if (running > target) { found = i; break; }
        }
      }
    }
    __syncthreads();
    if (threadIdx.x == 0) out[blockIdx.x] = found;
    return;
  }

  // top-p.  `cut`: the smallest value whose preceding mass is < top_p * Z; everything above it
  // is kept, and of the entries equal to it as many as still start below the limit.
  const unsigned top_bits = __float_as_uint(1.0f);  // the maximum's p is exp(0)
  const double limit = (double)top_p * total;
  const unsigned cut = lowest_threshold(p, vocab, top_bits, limit, true, sd);
  const double above_cut = mass_above(p, vocab, cut, sd);
  const double cut_value = (double)__uint_as_float(cut);
  double count_at_cut = 0.0;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) count_at_cut += (__float_as_uint(p[i]) == cut) ? 1.0 : 0.0;
  count_at_cut = block_sum_f64(count_at_cut, sd);
  double kept_at_cut = count_at_cut;
  if (cut_value > 0.0) kept_at_cut = fmin(count_at_cut, ceil((limit - above_cut) / cut_value));
  if (kept_at_cut < 1.0) kept_at_cut = 1.0;
  const double kept_mass = above_cut + kept_at_cut * cut_value;
  const double target = u * kept_mass;
  // the chosen value: the smallest one whose preceding mass is <= target (never below `cut`)
  unsigned chosen = lowest_threshold(p, vocab, top_bits, target, false, sd);
  if (chosen < cut) chosen = cut;
  const double above_chosen = mass_above(p, vocab, chosen, sd);
  const double chosen_value = (double)__uint_as_float(chosen);
  // among equal entries, in index order, the one the target falls into
  double which = chosen_value > 0.0 ? floor((target - above_chosen) / chosen_value) : 0.0;
  if (which < 0.0) which = 0.0;
  if (chosen == cut && which > kept_at_cut - 1.0) which = kept_at_cut - 1.0;
  // find the (which)-th index whose bits equal `chosen`: contiguous runs per thread again
  const int per = (vocab + blockDim.x - 1) / blockDim.x;
  const int begin = min(vocab, (int)threadIdx.x * per), end = min(vocab, begin + per);
  double matches = 0.0;
  for (int i = begin; i < end; ++i) matches += (__float_as_uint(p[i]) == chosen) ? 1.0 : 0.0;
  chunk_sums[threadIdx.x] = matches;
  if (threadIdx.x == 0) found = -1;
  __syncthreads();
  if (threadIdx.x == 0) {
    double seen = 0.0;
    int last_chunk = -1;
    for (int t = 0; t < (int)blockDim.x; ++t) {
      if (chunk_sums[t] == 0.0) continue;
      last_chunk = t;
      if (seen + chunk_sums[t] <= which) {
        seen += chunk_sums[t];
        continue;
      }
      const int b = min(vocab, t * per), e = min(vocab, b + per);
      for (int i = b; i < e; ++i)
        if (__float_as_uint(p[i]) == chosen) {
          if (seen == which) { found = i; break; }
          seen += 1.0;
        }
      break;
    }
    if (found < 0 && last_chunk >= 0) {  // rounding put the target past the last equal entry
      const int b = min(vocab, last_chunk * per), e = min(vocab, b + per);
      for (int i = e - 1; i >= b; --i)
        if (__float_as_uint(p[i]) == chosen) { found = i; break; }
    }
    if (found < 0) found = best_index;
  }
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = found;
}

// scratch: float32 [rows, vocab], overwritten.
extern "C" int llmserve_sample(const float* logits, const float* temperatures, const float* top_ps,
                               const float* uniforms, float* scratch, int* out, int rows, int vocab,
                               hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0) return ERR_BAD_ARGUMENT;
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, logits, temperatures, top_ps,
                     uniforms, scratch, out, vocab);
  return LAUNCH_STATUS();
}
