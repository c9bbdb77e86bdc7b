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
// p is exp((logit - max) / T), never divided by its sum Z: bounds are multiplied by Z instead.  Sums of
// p are float64 in an order that the sizes fix, or exact integers (see below): a call gives the same
// token on every run.
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
// `zero` (may be null): `zero_words` words that the launch clears, for whoever runs after it.
__global__ __launch_bounds__(SAMPLE_THREADS) void argmax_pieces_kernel(const float* __restrict__ logits,
                                                                       float* __restrict__ piece_values,
                                                                       int* __restrict__ piece_indices, int vocab,
                                                                       int pieces, unsigned* __restrict__ zero,
                                                                       size_t zero_words) {
  __shared__ float sv[17];
  __shared__ int si[17];
  if (zero != nullptr) {
    const size_t block = (size_t)blockIdx.y * gridDim.x + blockIdx.x, blocks = (size_t)gridDim.x * gridDim.y;
    for (size_t i = block * blockDim.x + threadIdx.x; i < zero_words; i += blocks * blockDim.x) zero[i] = 0u;
  }
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

// One wave picks among a row's pieces, which ascend in index, so the first maximum among them is the
// row's; every lane gets its index (0 for a row without entries).
__device__ __forceinline__ int wave_pick_argmax(const float* __restrict__ piece_values,
                                                const int* __restrict__ piece_indices, int pieces) {
  const int lane = threadIdx.x % WAVE;
  float value = -INFINITY;
  int index = 0x7fffffff;
  for (int i = lane; i < pieces; i += WAVE) {
    const float v = piece_values[i];
    const int at = piece_indices[i];
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
  return index == 0x7fffffff ? 0 : index;
}

__global__ void argmax_pick_kernel(const float* __restrict__ piece_values, const int* __restrict__ piece_indices,
                                   int* __restrict__ out, int pieces) {
  const int index = wave_pick_argmax(piece_values + blockIdx.x * pieces, piece_indices + blockIdx.x * pieces, pieces);
  if (threadIdx.x == 0) out[blockIdx.x] = index;
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
                     piece_values, piece_indices, vocab, pieces, (unsigned*)nullptr, (size_t)0);
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
                     piece_values, piece_indices, vocab, pieces, (unsigned*)nullptr, (size_t)0);
  hipLaunchKernelGGL(argmax_pick_kernel, dim3(rows), dim3(WAVE), 0, stream, piece_values, piece_indices, out, pieces);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------
// Sampling with a temperature and top-p.
//
// A row is cut into `pieces` contiguous pieces and every stage runs one block per (row, piece), so
// that a few rows of a large vocabulary use the whole chip; what a stage needs of the whole row it
// takes from what the stages before it wrote, every block for itself and all alike.
//
// Top-p needs, twice, the smallest float t with mass_above(t) below a bound, where mass_above(t) is the
// sum of the entries of p greater than t: first the value at which the kept set ends (bound top_p * Z,
// strict), then the value in which u falls (bound u * kept mass).  p >= 0, so float order is the order
// of the bit patterns, and p <= 1 = exp(0), so a pattern has 30 bits.  A search fixes them ten at a
// time: a stage adds up the mass and the number of the entries in each of the 1,024 bins that the next
// ten bits cut the present bucket into, and the head of the next stage takes the lowest bin at whose
// end the bound is met and goes on inside it.  After three levels the bucket is one value.  Both
// searches start from the same first histogram, so the second has two stages of its own.
//
// The entries of a bin share their exponent (it lies in the ten bits that are fixed first), so their
// sum is 2^exponent times the sum of their 24-bit significands, an integer below 2^42: a bin's mass is
// kept as that integer.  Integer sums do not depend on their order, so the blocks of a row add into
// one histogram with atomic additions and the result is the same on every run.

#define SAMPLE_BLOCK 256  // threads of a block that works on a piece of a row
#define SAMPLE_BINS 1024
#define SAMPLE_BINS_EACH (SAMPLE_BINS / SAMPLE_BLOCK)  // bins that a thread of the head looks at
#define SAMPLE_LEVEL_BITS 10
#define SAMPLE_PIECES_MAX 64  // a wave looks at a row's pieces, a lane at each
#define SAMPLE_HISTOGRAMS 5   // the cut search's three levels, then levels 1 and 2 of the chosen search

static int sample_pieces(int rows) {
  int pieces = SAMPLE_PIECES_MAX;
  while (pieces > 4 && rows * pieces > 2048) pieces /= 2;
  return pieces;
}

__device__ __forceinline__ int level_shift(int level) { return (2 - level) * SAMPLE_LEVEL_BITS; }

// value = significand * 2^(binary_exponent): what a float's pattern says, also for the subnormal ones
__device__ __forceinline__ unsigned long long significand_of(unsigned pattern) {
  return (pattern & 0x7fffffu) | ((pattern >> 23) != 0u ? 0x800000u : 0u);
}
__device__ __forceinline__ int binary_exponent_of(unsigned pattern) {
  const int exponent = (int)(pattern >> 23);
  return (exponent != 0 ? exponent : 1) - 150;
}

// What the searches of one row have found so far.  A stage reads what the stage before wrote and
// writes its own (so that no block reads what another block of the same launch writes).
struct SampleState {
  double limit;        // top_p * Z: the bound of the cut search
  double target;       // u * (kept mass): the bound of the chosen search
  double above_cut;    // mass above the cut value
  double kept_at_cut;  // how many of the entries equal to the cut value are kept
  double above[2];     // per search: mass above the bucket it is in
  unsigned base[2];    // per search: first pattern of that bucket
  unsigned cut;        // pattern of the cut value
  unsigned unused;
};

struct Picked {
  int bin;
  double above;    // mass above the end of that bin
  unsigned count;  // entries in it
};

// The lowest of the bins of one level at whose end the mass above (that of the bucket, `above`, and
// of the bins after it) meets the bound: < limit if strict, else <= limit.  `sums`, `counts`: the
// row's histogram; `base`: the bucket's first pattern; `level`: which ten bits the bins are.  Every
// thread of the block calls it (blockDim.x >= SAMPLE_BLOCK); after: SAMPLE_BLOCK / WAVE doubles of LDS.
__device__ Picked pick_bin(const unsigned long long* __restrict__ sums, const unsigned* __restrict__ counts,
                           unsigned base, int level, double above, double limit, bool strict, double* after,
                           int* lowest, double* lowest_above, unsigned* lowest_count) {
  const int t = threadIdx.x;
  double mass[SAMPLE_BINS_EACH];
  unsigned count[SAMPLE_BINS_EACH];
  double mine = 0.0;
  __syncthreads();  // whoever read the LDS arrays before is done
  if (t < SAMPLE_BLOCK) {
#pragma unroll
    for (int j = SAMPLE_BINS_EACH - 1; j >= 0; --j) {
      const int bin = t * SAMPLE_BINS_EACH + j;
      const unsigned first = base + ((unsigned)bin << level_shift(level));  // the bin's first pattern
      mass[j] = ldexp((double)sums[bin], binary_exponent_of(first));
      count[j] = counts[bin];
      mine += mass[j];
    }
  }
  // the sum of the threads after this one: inside a wave by shuffles, then the waves after it
  const int lane = t % WAVE, wave = t / WAVE;
  double inclusive = mine;
#pragma unroll
  for (int offset = 1; offset < WAVE; offset <<= 1) {
    const double other = __shfl_down(inclusive, offset, WAVE);
    if (lane + offset < WAVE) inclusive += other;
  }
  const double after_in_wave = __shfl_down(inclusive, 1, WAVE);
  if (t < SAMPLE_BLOCK && lane == 0) after[wave] = inclusive;
  if (t == 0) *lowest = SAMPLE_BINS;
  __syncthreads();
  double after_mine = lane == WAVE - 1 ? 0.0 : after_in_wave;
  if (t < SAMPLE_BLOCK)
    for (int w = SAMPLE_BLOCK / WAVE - 1; w > wave; --w) after_mine += after[w];
  int my_bin = SAMPLE_BINS;
  double my_above = 0.0;
  unsigned my_count = 0;
  if (t < SAMPLE_BLOCK) {
    double later = after_mine;  // mass of the bins after the one looked at
#pragma unroll
    for (int j = SAMPLE_BINS_EACH - 1; j >= 0; --j) {
      const double m = above + later;
      if (strict ? m < limit : m <= limit) {
        my_bin = t * SAMPLE_BINS_EACH + j;
        my_above = m;
        my_count = count[j];
      }
      later += mass[j];
    }
    if (my_bin < SAMPLE_BINS) atomicMin(lowest, my_bin);
  }
  __syncthreads();
  if (my_bin < SAMPLE_BINS && my_bin == *lowest) {
    *lowest_above = my_above;
    *lowest_count = my_count;
  }
  __syncthreads();
  Picked picked;
  picked.bin = *lowest;
  if (picked.bin == SAMPLE_BINS) {  // the bound is met nowhere (it cannot be: nothing lies above the maximum)
    picked.bin = SAMPLE_BINS - 1;
    picked.above = above;
    picked.count = 0;
    return picked;
  }
  picked.above = *lowest_above;
  picked.count = *lowest_count;
  return picked;
}

__device__ __forceinline__ void clear_histogram(unsigned long long* lds_sums, unsigned* lds_counts) {
  for (int i = threadIdx.x; i < SAMPLE_BINS; i += blockDim.x) {
    lds_sums[i] = 0ull;
    lds_counts[i] = 0u;
  }
}

// Adds this piece's entries inside the bucket `base` of `level` into the row's histogram.  The block
// has cleared lds_sums and lds_counts and passed a barrier since.
__device__ __forceinline__ void add_histogram(const float* __restrict__ p, int begin, int end, unsigned base, int level,
                                              unsigned long long* lds_sums, unsigned* lds_counts,
                                              unsigned long long* __restrict__ sums, unsigned* __restrict__ counts,
                                              unsigned* __restrict__ piece_counts) {
  const int shift = level_shift(level);
  const unsigned bucket = base >> (shift + SAMPLE_LEVEL_BITS);
  for (int i = begin + threadIdx.x; i < end; i += blockDim.x) {
    const unsigned pattern = __float_as_uint(p[i]);
    if ((pattern >> (shift + SAMPLE_LEVEL_BITS)) == bucket) {
      const unsigned bin = (pattern >> shift) & (SAMPLE_BINS - 1);
      atomicAdd(lds_sums + bin, significand_of(pattern));
      atomicAdd(lds_counts + bin, 1u);
    }
  }
  __syncthreads();
  for (int bin = threadIdx.x; bin < SAMPLE_BINS; bin += blockDim.x) {
    const unsigned count = lds_counts[bin];
    if (count != 0u) {
      atomicAdd(sums + bin, lds_sums[bin]);
      atomicAdd(counts + bin, count);
    }
    if (piece_counts != nullptr) piece_counts[bin] = count;
  }
}

// The layout of what the stages share, per row: SAMPLE_HISTOGRAMS histograms (cleared by the first
// launch), the entries of each piece in every bin of the two last levels, the states.
struct SampleBuffers {
  float* p;                     // [rows, vocab]
  double* piece_sums;           // [rows, pieces]
  unsigned long long* sums;     // [SAMPLE_HISTOGRAMS, rows, SAMPLE_BINS]
  unsigned* counts;             // [SAMPLE_HISTOGRAMS, rows, SAMPLE_BINS]
  unsigned* piece_counts;       // [2, rows, pieces, SAMPLE_BINS]: of the last level of the cut search, of the chosen search
  SampleState* states;          // [SAMPLE_HISTOGRAMS, rows]
  const float* piece_values;    // [rows, argmax_pieces]
  const int* piece_indices;
};

// The row's argmax (to out), p = exp((logit - max) / T) of one piece, not yet divided by its sum Z
// (engine.py:32), the piece's sum, and for a row with top-p the first histogram, which depends on no bucket.
__global__ __launch_bounds__(SAMPLE_BLOCK) void sample_exp_kernel(const float* __restrict__ logits,
                                                                  const float* __restrict__ temperatures,
                                                                  const float* __restrict__ top_ps, SampleBuffers buffers,
                                                                  int* __restrict__ out, int rows, int vocab, int pieces,
                                                                  int argmax_pieces, int with_top_p) {
  __shared__ double sd[17];
  __shared__ int best_index;
  __shared__ unsigned long long lds_sums[SAMPLE_BINS];
  __shared__ unsigned lds_counts[SAMPLE_BINS];
  const int r = blockIdx.x, piece = blockIdx.y;
  clear_histogram(lds_sums, lds_counts);
  if (threadIdx.x < WAVE) {
    const int index = wave_pick_argmax(buffers.piece_values + r * argmax_pieces,
                                       buffers.piece_indices + r * argmax_pieces, argmax_pieces);
    if (threadIdx.x == 0) {
      best_index = index;
      if (piece == 0) out[r] = index;
    }
  }
  __syncthreads();
  const float temperature = temperatures[r];
  if (temperature <= 0.f) return;  // engine.py:30-31: the argmax stands
  const float* row = logits + (size_t)r * vocab;
  float* p = buffers.p + (size_t)r * vocab;
  const int per = (vocab + pieces - 1) / pieces;
  const int begin = min(vocab, piece * per), end = min(vocab, begin + per);
  const float top_logit = row[best_index] / temperature;
  double partial = 0.0;
  for (int i = begin + threadIdx.x; i < end; i += blockDim.x) {
    const float v = expf(row[i] / temperature - top_logit);
    p[i] = v;
    partial += (double)v;
  }
  const double sum = block_sum_f64(partial, sd);
  if (threadIdx.x == 0) buffers.piece_sums[r * pieces + piece] = sum;
  if (!with_top_p || top_ps[r] >= 1.f) return;
  add_histogram(p, begin, end, 0u, 0, lds_sums, lds_counts, buffers.sums + (size_t)r * SAMPLE_BINS,
                buffers.counts + (size_t)r * SAMPLE_BINS, nullptr);
}

// One stage of the two searches of the rows with top-p.  stage 1, 2: levels 1, 2 of the cut search;
// 3, 4: levels 1, 2 of the chosen search.  The head takes from the histogram of the stage before the
// bucket to go on in (stage 3: the cut value from the histogram of stage 2, what is kept, and the
// chosen search's first bucket from the first histogram); the body adds up this piece's entries
// inside that bucket into histogram `stage`.
__global__ __launch_bounds__(SAMPLE_BLOCK) void sample_level_kernel(const float* __restrict__ temperatures,
                                                                    const float* __restrict__ top_ps,
                                                                    const float* __restrict__ uniforms,
                                                                    SampleBuffers buffers, int rows, int vocab,
                                                                    int pieces, int stage) {
  __shared__ double after[SAMPLE_BLOCK / WAVE];
  __shared__ int lowest;
  __shared__ double lowest_above;
  __shared__ unsigned lowest_count;
  __shared__ unsigned long long lds_sums[SAMPLE_BINS];
  __shared__ unsigned lds_counts[SAMPLE_BINS];
  const int r = blockIdx.x, piece = blockIdx.y;
  const float top_p = top_ps[r];
  if (temperatures[r] <= 0.f || top_p >= 1.f) return;
  clear_histogram(lds_sums, lds_counts);  // the head's barriers lie between this and the additions
  const size_t per_histogram = (size_t)rows * SAMPLE_BINS, of_row = (size_t)r * SAMPLE_BINS;
  const int search = stage <= 2 ? 0 : 1, level = stage <= 2 ? stage : stage - 2;

  SampleState st;
  if (stage == 1) {
    double total = 0.0;
    for (int q = 0; q < pieces; ++q) total += buffers.piece_sums[r * pieces + q];
    // the bound is strict, so a bound of 0 would be met nowhere: the least positive one keeps the maximum alone
    st.limit = fmax((double)top_p * total, 2.2250738585072014e-308);
    st.target = st.above_cut = st.kept_at_cut = st.above[0] = st.above[1] = 0.0;
    st.base[0] = st.base[1] = st.cut = st.unused = 0u;
  } else {
    st = buffers.states[(size_t)(stage - 1) * rows + r];
  }
  if (stage <= 2) {  // one more level of the cut search
    const size_t at = (size_t)(stage - 1) * per_histogram + of_row;
    const Picked got = pick_bin(buffers.sums + at, buffers.counts + at, st.base[0], stage - 1, st.above[0], st.limit,
                                true, after, &lowest, &lowest_above, &lowest_count);
    st.base[0] += (unsigned)got.bin << level_shift(stage - 1);
    st.above[0] = got.above;
  } else if (stage == 3) {
    // the cut value: everything above it is kept, and of the entries equal to it as many as still
    // start below the bound (engine.py:34-37)
    size_t at = (size_t)2 * per_histogram + of_row;
    Picked got = pick_bin(buffers.sums + at, buffers.counts + at, st.base[0], 2, st.above[0], st.limit, true, after,
                          &lowest, &lowest_above, &lowest_count);
    st.cut = st.base[0] + (unsigned)got.bin;
    st.above_cut = got.above;
    const double cut_value = (double)__uint_as_float(st.cut), count_at_cut = (double)got.count;
    double kept_at_cut = count_at_cut;
    if (cut_value > 0.0) kept_at_cut = fmin(count_at_cut, ceil((st.limit - st.above_cut) / cut_value));
    if (kept_at_cut < 1.0) kept_at_cut = 1.0;
    st.kept_at_cut = kept_at_cut;
    st.target = (double)uniforms[r] * (st.above_cut + kept_at_cut * cut_value);
    // the chosen value: the smallest one whose preceding mass is <= target
    got = pick_bin(buffers.sums + of_row, buffers.counts + of_row, 0u, 0, 0.0, st.target, false, after, &lowest,
                   &lowest_above, &lowest_count);
    st.base[1] = (unsigned)got.bin << level_shift(0);
    st.above[1] = got.above;
  } else {
    const size_t at = (size_t)3 * per_histogram + of_row;
    const Picked got = pick_bin(buffers.sums + at, buffers.counts + at, st.base[1], 1, st.above[1], st.target, false,
                                after, &lowest, &lowest_above, &lowest_count);
    st.base[1] += (unsigned)got.bin << level_shift(1);
    st.above[1] = got.above;
  }
  if (piece == 0 && threadIdx.x == 0) buffers.states[(size_t)stage * rows + r] = st;

  const int per = (vocab + pieces - 1) / pieces;
  const int begin = min(vocab, piece * per), end = min(vocab, begin + per);
  unsigned* piece_counts = nullptr;  // the last level: the final stage asks which piece holds the entry
  if (level == 2) piece_counts = buffers.piece_counts + (((size_t)search * rows + r) * pieces + piece) * SAMPLE_BINS;
  const size_t to = (size_t)stage * per_histogram + of_row;
  add_histogram(buffers.p + (size_t)r * vocab, begin, end, st.base[search], level, lds_sums, lds_counts,
                buffers.sums + to, buffers.counts + to, piece_counts);
}

// Sums of v over the threads before this one, in thread order.  shared: at least 16 of its kind.
__device__ __forceinline__ double block_sum_before_f64(double v, double* shared) {
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  double inclusive = v;
#pragma unroll
  for (int offset = 1; offset < WAVE; offset <<= 1) {
    const double other = __shfl_up(inclusive, offset, WAVE);
    if (lane >= offset) inclusive += other;
  }
  __syncthreads();
  if (lane == WAVE - 1) shared[wave] = inclusive;
  __syncthreads();
  double before = 0.0;
  for (int w = 0; w < wave; ++w) before += shared[w];
  const double in_wave = __shfl_up(inclusive, 1, WAVE);
  return lane == 0 ? before : before + in_wave;
}

__device__ __forceinline__ int block_sum_before_int(int v, int* shared) {
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  int inclusive = v;
#pragma unroll
  for (int offset = 1; offset < WAVE; offset <<= 1) {
    const int other = __shfl_up(inclusive, offset, WAVE);
    if (lane >= offset) inclusive += other;
  }
  __syncthreads();
  if (lane == WAVE - 1) shared[wave] = inclusive;
  __syncthreads();
  int before = 0;
  for (int w = 0; w < wave; ++w) before += shared[w];
  return before + inclusive - v;
}

// The token of every row with a temperature: one block per row.  `out` holds the argmax already.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_pick_kernel(const float* __restrict__ temperatures,
                                                                     const float* __restrict__ top_ps,
                                                                     const float* __restrict__ uniforms,
                                                                     SampleBuffers buffers, int* __restrict__ out,
                                                                     int rows, int vocab, int pieces, int with_top_p) {
  __shared__ double after[SAMPLE_BLOCK / WAVE];
  __shared__ int lowest;
  __shared__ double lowest_above;
  __shared__ unsigned lowest_count;
  __shared__ double sd[17];
  __shared__ int si[17];
  __shared__ int owner_piece, owner_thread;
  __shared__ double before_piece, shared_target;
  __shared__ int wanted;  // which of the entries equal to the chosen value, counted inside the owner piece
  const int r = blockIdx.x;
  if (temperatures[r] <= 0.f) return;  // engine.py:30-31
  const float* p = buffers.p + (size_t)r * vocab;
  const float top_p = top_ps[r];
  const int per_piece = (vocab + pieces - 1) / pieces;
  const int lane = threadIdx.x % WAVE;

  if (top_p >= 1.f || !with_top_p) {
    // inverse CDF in index order: the piece first, from the pieces' sums, then inside it
    if (threadIdx.x == 0) owner_thread = 0x7fffffff;
    if (threadIdx.x < WAVE) {  // a lane per piece
      const double sum = lane < pieces ? buffers.piece_sums[r * pieces + lane] : 0.0;
      double inclusive = sum;
#pragma unroll
      for (int offset = 1; offset < WAVE; offset <<= 1) {
        const double other = __shfl_up(inclusive, offset, WAVE);
        if (lane >= offset) inclusive += other;
      }
      const double total = __shfl(inclusive, WAVE - 1, WAVE);
      const double target = (double)uniforms[r] * total;
      const double from_below = __shfl_up(inclusive, 1, WAVE);  // every lane takes part in it
      const double before = lane == 0 ? 0.0 : from_below;
      const unsigned long long holds = __ballot(lane < pieces && before + sum > target);
      const int owner = holds != 0ull ? __ffsll((long long)holds) - 1 : -1;
      if (lane == (owner < 0 ? 0 : owner)) {
        owner_piece = owner;
        before_piece = before;
        shared_target = target;
      }
    }
    __syncthreads();
    if (owner_piece < 0) {
      if (threadIdx.x == 0) out[r] = vocab - 1;
      return;
    }
    const double target = shared_target;
    const int begin = min(vocab, owner_piece * per_piece), end = min(vocab, begin + per_piece);
    const int per = (end - begin + blockDim.x - 1) / blockDim.x;  // each thread owns a contiguous run
    const int b = min(end, begin + (int)threadIdx.x * per), e = min(end, b + per);
    double mine = 0.0;
    for (int i = b; i < e; ++i) mine += (double)p[i];
    const double before = before_piece + block_sum_before_f64(mine, sd);
    if (before + mine > target) atomicMin(&owner_thread, (int)threadIdx.x);
    __syncthreads();
    if (owner_thread == 0x7fffffff) {  // rounding put the target past the piece's end
      if (threadIdx.x == 0) out[r] = end - 1;
    } else if ((int)threadIdx.x == owner_thread) {
      double running = before;
      int found = e - 1;
      for (int i = b; i < e; ++i) {
        running += (double)p[i];
        if (running > target) { found = i; break; }
      }
      out[r] = found;
    }
    return;
  }

  // top-p: the chosen search's last level, then the entry among the equal ones, in index order
  const size_t per_histogram = (size_t)rows * SAMPLE_BINS, of_row = (size_t)r * SAMPLE_BINS;
  const SampleState st = buffers.states[(size_t)(SAMPLE_HISTOGRAMS - 1) * rows + r];
  const size_t at = (size_t)(SAMPLE_HISTOGRAMS - 1) * per_histogram + of_row;
  const Picked got = pick_bin(buffers.sums + at, buffers.counts + at, st.base[1], 2, st.above[1], st.target, false,
                              after, &lowest, &lowest_above, &lowest_count);
  unsigned chosen = st.base[1] + (unsigned)got.bin;
  double above_chosen = got.above;
  int search = 1;
  if (chosen < st.cut) {  // never below the cut
    chosen = st.cut;
    above_chosen = st.above_cut;
    search = 0;
  }
  // how many entries of each piece equal the chosen value: the last level of that search has counted them
  const unsigned* equal_in = buffers.piece_counts + ((size_t)search * rows + r) * pieces * SAMPLE_BINS + (chosen & (SAMPLE_BINS - 1));
  if (threadIdx.x < WAVE) {  // a lane per piece
    const int here = lane < pieces ? (int)equal_in[(size_t)lane * SAMPLE_BINS] : 0;
    int inclusive = here;
#pragma unroll
    for (int offset = 1; offset < WAVE; offset <<= 1) {
      const int other = __shfl_up(inclusive, offset, WAVE);
      if (lane >= offset) inclusive += other;
    }
    const int equal = __shfl(inclusive, WAVE - 1, WAVE);
    const double chosen_value = (double)__uint_as_float(chosen);
    double which = chosen_value > 0.0 ? floor((st.target - above_chosen) / chosen_value) : 0.0;
    if (which < 0.0) which = 0.0;
    if (chosen == st.cut && which > st.kept_at_cut - 1.0) which = st.kept_at_cut - 1.0;
    // rounding may put the target past the last equal entry: then that one
    const int index = which > (double)(equal - 1) ? equal - 1 : (int)which;
    const int before = inclusive - here;
    const unsigned long long holds = __ballot(equal > 0 && before <= index && index < inclusive);
    const int owner = holds != 0ull ? __ffsll((long long)holds) - 1 : -1;
    if (lane == (owner < 0 ? 0 : owner)) {
      owner_piece = owner;
      wanted = index - before;
    }
  }
  __syncthreads();
  if (owner_piece < 0) return;  // no entry has the chosen value: the argmax stands
  const int begin = min(vocab, owner_piece * per_piece), end = min(vocab, begin + per_piece);
  const int per = (end - begin + blockDim.x - 1) / blockDim.x;
  const int b = min(end, begin + (int)threadIdx.x * per), e = min(end, b + per);
  int mine = 0;
  for (int i = b; i < e; ++i) mine += __float_as_uint(p[i]) == chosen ? 1 : 0;
  const int before = block_sum_before_int(mine, si);
  if (before <= wanted && wanted < before + mine) {
    int seen = before;
    for (int i = b; i < e; ++i)
      if (__float_as_uint(p[i]) == chosen) {
        if (seen == wanted) { out[r] = i; break; }
        ++seen;
      }
  }
}

static size_t rounded(size_t bytes) { return (bytes + 255) / 256 * 256; }

struct SampleWorkspace {
  size_t sums, counts, cleared_words;  // the histograms come first: the first launch clears them
  size_t p, piece_sums, piece_counts, states, piece_values, piece_indices, bytes;
};

static SampleWorkspace sample_workspace(int rows, int vocab) {
  const size_t pieces = sample_pieces(rows), bins = (size_t)SAMPLE_HISTOGRAMS * rows * SAMPLE_BINS;
  SampleWorkspace w;
  size_t at = 0;
  w.sums = at, at += rounded(bins * sizeof(unsigned long long));
  w.counts = at, at += rounded(bins * sizeof(unsigned));
  w.cleared_words = at / sizeof(unsigned);
  w.p = at, at += rounded((size_t)rows * vocab * sizeof(float));
  w.piece_sums = at, at += rounded((size_t)rows * pieces * sizeof(double));
  w.piece_counts = at, at += rounded((size_t)2 * rows * pieces * SAMPLE_BINS * sizeof(unsigned));
  w.states = at, at += rounded((size_t)SAMPLE_HISTOGRAMS * rows * sizeof(SampleState));
  w.piece_values = at, at += rounded((size_t)rows * ARGMAX_PIECES * sizeof(float));
  w.piece_indices = at, at += rounded((size_t)rows * ARGMAX_PIECES * sizeof(int));
  w.bytes = at;
  return w;
}

// The size, in KiB, of the workspace that llmserve_sample needs for these sizes; -1 if they are not positive.
extern "C" int llmserve_sample_workspace_kib(int rows, int vocab) {
  if (rows <= 0 || vocab <= 0) return -1;
  return (int)((sample_workspace(rows, vocab).bytes + 1023) / 1024);
}

// out[r]: the token of row r.  workspace: 256-byte aligned device memory of llmserve_sample_workspace_kib
// KiB, overwritten.  with_top_p = 0 promises that no row with a temperature has top_p < 1, and leaves the
// searches out.
extern "C" int llmserve_sample(const float* logits, const float* temperatures, const float* top_ps,
                               const float* uniforms, void* workspace, int workspace_kib, int* out, int rows,
                               int vocab, int with_top_p, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0 || workspace == nullptr || ((size_t)workspace & 255) != 0) return ERR_BAD_ARGUMENT;
  const SampleWorkspace w = sample_workspace(rows, vocab);
  if ((size_t)workspace_kib * 1024 < w.bytes) return ERR_BAD_ARGUMENT;
  unsigned char* base = (unsigned char*)workspace;
  float* piece_values = (float*)(base + w.piece_values);
  int* piece_indices = (int*)(base + w.piece_indices);
  SampleBuffers buffers;
  buffers.p = (float*)(base + w.p);
  buffers.piece_sums = (double*)(base + w.piece_sums);
  buffers.sums = (unsigned long long*)(base + w.sums);
  buffers.counts = (unsigned*)(base + w.counts);
  buffers.piece_counts = (unsigned*)(base + w.piece_counts);
  buffers.states = (SampleState*)(base + w.states);
  buffers.piece_values = piece_values;
  buffers.piece_indices = piece_indices;
  const int first_pieces = argmax_pieces(rows), pieces = sample_pieces(rows);
  hipLaunchKernelGGL(argmax_pieces_kernel, dim3(rows, first_pieces), dim3(SAMPLE_THREADS), 0, stream, logits,
                     piece_values, piece_indices, vocab, first_pieces, with_top_p ? (unsigned*)base : (unsigned*)nullptr,
                     with_top_p ? w.cleared_words : (size_t)0);
  hipLaunchKernelGGL(sample_exp_kernel, dim3(rows, pieces), dim3(SAMPLE_BLOCK), 0, stream, logits, temperatures, top_ps,
                     buffers, out, rows, vocab, pieces, first_pieces, with_top_p);
  if (with_top_p)
    for (int stage = 1; stage < SAMPLE_HISTOGRAMS; ++stage)
      hipLaunchKernelGGL(sample_level_kernel, dim3(rows, pieces), dim3(SAMPLE_BLOCK), 0, stream, temperatures, top_ps,
                         uniforms, buffers, rows, vocab, pieces, stage);
  hipLaunchKernelGGL(sample_pick_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, temperatures, top_ps, uniforms,
                     buffers, out, rows, vocab, pieces, with_top_p);
  return LAUNCH_STATUS();
}
