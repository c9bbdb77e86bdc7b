// bfloat16 products on the matrix cores (MFMA), float32 accumulation.
//
// gemm_skinny: out[M, N] = x[M, K] . w[N, K]^T (+ bias) for M <= 64, the shape of decoding.
// Such a product is a stream of the weight matrix from HBM, so the kernel is built around
// that stream: a workgroup owns 16 weight rows and its waves split K between them; every
// lane keeps two groups of four 16-byte loads of its weight row in flight; the weights go
// straight from global memory into the A operand of v_mfma_f32_16x16x32_bf16 (lane l holds
// row l % 16, k = (l / 16) * 8 .. + 8 of a 32-wide step), the few activation rows into the B
// operand, so the result tile D[n][m] leaves four consecutive n of one token in each lane.
// The waves' partial tiles are added through LDS in wave order, so a row's bits depend on
// the shape of the weight only, not on what else is in the batch.
//
// With `gated`, weight rows alternate gate_j, up_j and the epilogue writes
// silu(gate) * up (reference model.py:188) to out[M, N / 2].
#include "common.h"
#include <type_traits>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define STEP 32   // k per MFMA
#define GROUP 4   // MFMA steps a wave loads at once: 128 k, 256 bytes of each weight row

__device__ __forceinline__ bf16x8 load8(const bf16_t* p) { return *(const bf16x8*)p; }
// The weight stream uses plain loads: non-temporal ones were measured 8-12 % slower here.
__device__ __forceinline__ bf16x8 load8_stream(const bf16_t* p) { return *(const bf16x8*)p; }
#ifndef TARGET_WAVES
#define TARGET_WAVES 2048
#endif

template <int WAVES, int MT, typename TO, bool GATED>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ x,
                                                                 const bf16_t* __restrict__ w,
                                                                 const void* __restrict__ bias, int bias_is_float,
                                                                 TO* __restrict__ out, int M, int N, int K,
                                                                 int k_split) {
  extern __shared__ float partial[];  // [WAVES][MT][64 lanes][4]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int n = min((int)blockIdx.x * 16 + r, N - 1);
  // blockIdx.y picks a slice of K, `k_split` long; its sums go to its own copy of `out`
  const int k_first = blockIdx.y * k_split;
  const bf16_t* w_row = w + (size_t)n * K + k_first + g * 8;
  const bf16_t* x_row[MT];
  bool x_live[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + r;
    x_live[t] = m < M;
    x_row[t] = x + (size_t)min(m, M - 1) * K + k_first + g * 8;
  }
  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  // the bias of this lane's four outputs is asked for now and used at the end
  const bool with_bias = bias && blockIdx.y == 0;
  // (as 16-bit halves, so that both types of bias take the same loads: a float32 is two of them, a
  // bfloat16 the upper one alone)
  // (without a branch: where there is no bias the same loads read the start of the weights and
  // their result is dropped; loads inside a branch would be waited for at its end)
  unsigned short bias_low[4], bias_high[4];
  {
    const unsigned short* source = with_bias ? (const unsigned short*)bias : (const unsigned short*)w;
    const int halves = with_bias && bias_is_float ? 2 : 1;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int at = min((int)blockIdx.x * 16 + g * 4 + i, N - 1) * halves;
      bias_low[i] = source[at];
      bias_high[i] = source[at + halves - 1];
    }
  }

  const int groups = k_split / (STEP * GROUP);
  bf16x8 a[GROUP], a_next[GROUP];
  int group = wave;
  if (group < groups) {
#pragma unroll
    for (int u = 0; u < GROUP; ++u) a[u] = load8_stream(w_row + (group * GROUP + u) * STEP);
  }
  while (group < groups) {
    const int next = group + WAVES;
    // this group's x is asked for before the next group's weights: loads come back in the order they
    // were asked for, and the products below wait for x
    bf16x8 b[MT][GROUP];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int u = 0; u < GROUP; ++u) b[t][u] = x_live[t] ? load8(x_row[t] + (group * GROUP + u) * STEP) : zero;
    asm volatile("" ::: "memory");  // (the compiler would put the weights first again)
    if (next < groups) {
#pragma unroll
      for (int u = 0; u < GROUP; ++u) a_next[u] = load8_stream(w_row + (next * GROUP + u) * STEP);
    }
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int u = 0; u < GROUP; ++u) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b[t][u], acc[t], 0, 0, 0);
#pragma unroll
    for (int u = 0; u < GROUP; ++u) a[u] = a_next[u];
    group = next;
  }
  // the steps left over when K is not a multiple of 128
  for (int step = groups * GROUP + wave; step < k_split / STEP; step += WAVES) {
    const bf16x8 a_tail = load8_stream(w_row + step * STEP);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const bf16x8 b_tail = x_live[t] ? load8(x_row[t] + step * STEP) : zero;
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_tail, b_tail, acc[t], 0, 0, 0);
    }
  }

#pragma unroll
  for (int t = 0; t < MT; ++t) *(f32x4*)(partial + ((wave * MT + t) * 64 + lane) * 4) = acc[t];
  __syncthreads();
  if (wave >= MT) return;
  // wave t finishes token tile t: lane holds token m = t * 16 + r, rows n0 + g * 4 .. + 4
  const int t = wave;
  f32x4 total = (f32x4){0.f, 0.f, 0.f, 0.f};
  for (int v = 0; v < WAVES; ++v) total += *(const f32x4*)(partial + ((v * MT + t) * 64 + lane) * 4);
  const int m = t * 16 + r;
  const int n_first = blockIdx.x * 16 + g * 4;
  if (m >= M) return;
  if (with_bias) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      total[i] += __uint_as_float((unsigned)bias_high[i] << 16 | (bias_is_float ? (unsigned)bias_low[i] : 0u));
  }
  if (GATED) {
    TO* dst = out + (size_t)m * (N / 2) + n_first / 2;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (n_first + 2 * i + 1 < N) {
        const float gate = total[2 * i], up = total[2 * i + 1];
        dst[i] = from_float<TO>(gate / (1.f + expf(-gate)) * up);
      }
    }
  } else {
    TO* dst = out + ((size_t)blockIdx.y * M + m) * N + n_first;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n_first + i < N) dst[i] = from_float<TO>(total[i]);
  }
}

template <int WAVES, int MT, typename TO, bool GATED>
static int launch_skinny(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int M, int N,
                         int K, int splits, hipStream_t stream) {
  const size_t lds = (size_t)WAVES * MT * 64 * 4 * sizeof(float);
  hipLaunchKernelGGL((gemm_skinny_kernel<WAVES, MT, TO, GATED>), dim3((N + 15) / 16, splits), dim3(WAVES * 64), lds,
                     stream, (const bf16_t*)x, (const bf16_t*)w, bias, bias_is_float, (TO*)out, M, N, K, K / splits);
  return LAUNCH_STATUS();
}

template <int WAVES, typename TO, bool GATED>
static int pick_tiles(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int M, int N, int K,
                      int splits, hipStream_t stream) {
  if (M <= 16) return launch_skinny<WAVES, 1, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
  if (M <= 32) return launch_skinny<WAVES, 2, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
  return launch_skinny<WAVES, 4, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
}

template <typename TO, bool GATED>
static int pick_waves(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int M, int N, int K,
                      int splits, hipStream_t stream) {
  // enough waves to cover the chip (about 2,048), but no more than there are 128-wide groups of K
  const int tiles = (N + 15) / 16 * splits, groups = max(1, K / splits / (STEP * GROUP));
  int waves = 4;
  while (waves < 16 && waves * tiles < TARGET_WAVES && waves * 2 <= groups) waves *= 2;
  if (waves == 4) return pick_tiles<4, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
  if (waves == 8) return pick_tiles<8, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
  return pick_tiles<16, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
}

// gemm_pair: gemm_skinny for up to 16 rows of x with NT tiles of 16 weight rows a wave, which share
// the wave's x: every workgroup reads all of x for its K range, M / (16 NT) of what it reads of the
// weights, and the chiplets' L2 delivers little more than HBM does, so at 16 rows and NT = 1 the
// x doubles the traffic.  More tiles a wave also means more bytes under way a wave and fewer
// workgroups: it pays for long K ranges and big weights (7B sizes at 8 rows: gate/up 57.7 -> 52.1 us
// with two tiles, down 32.1 -> 26.3 us with four; 1.5B sizes at 16 rows: gate/up 18.0 -> 16.9 us).
template <int WAVES, int NT, typename TO, bool GATED>
__global__ __launch_bounds__(WAVES * 64) void gemm_pair_kernel(const bf16_t* __restrict__ x,
                                                               const bf16_t* __restrict__ w,
                                                               const void* __restrict__ bias, int bias_is_float,
                                                               TO* __restrict__ out, int M, int N, int K,
                                                               int k_split) {
  extern __shared__ float partial[];  // [WAVES][NT][64 lanes][4]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int k_first = blockIdx.y * k_split;
  const bf16_t* w_row[NT];
#pragma unroll
  for (int s = 0; s < NT; ++s)
    w_row[s] = w + (size_t)min(((int)blockIdx.x * NT + s) * 16 + r, N - 1) * K + k_first + g * 8;
  const bool x_live = r < M;
  const bf16_t* x_row = x + (size_t)min(r, M - 1) * K + k_first + g * 8;
  f32x4 acc[NT];
#pragma unroll
  for (int s = 0; s < NT; ++s) acc[s] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  // the bias of the four outputs this lane will finish (wave s finishes tile s) is asked for now
  float bias_here[4] = {0.f, 0.f, 0.f, 0.f};
  if (bias && blockIdx.y == 0 && wave < NT) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      bias_here[i] = load_as_float(bias, bias_is_float, min(((int)blockIdx.x * NT + wave) * 16 + g * 4 + i, N - 1));
  }
  const int groups = k_split / (STEP * GROUP);
  bf16x8 a[NT][GROUP], a_next[NT][GROUP];
  int group = wave;
  if (group < groups) {
#pragma unroll
    for (int s = 0; s < NT; ++s)
#pragma unroll
      for (int u = 0; u < GROUP; ++u) a[s][u] = load8_stream(w_row[s] + (group * GROUP + u) * STEP);
  }
  while (group < groups) {
    const int next = group + WAVES;
    bf16x8 b[GROUP];
#pragma unroll
    for (int u = 0; u < GROUP; ++u) b[u] = x_live ? load8(x_row + (group * GROUP + u) * STEP) : zero;
    asm volatile("" ::: "memory");
    if (next < groups) {
#pragma unroll
      for (int s = 0; s < NT; ++s)
#pragma unroll
        for (int u = 0; u < GROUP; ++u) a_next[s][u] = load8_stream(w_row[s] + (next * GROUP + u) * STEP);
    }
#pragma unroll
    for (int u = 0; u < GROUP; ++u)
#pragma unroll
      for (int s = 0; s < NT; ++s) acc[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s][u], b[u], acc[s], 0, 0, 0);
#pragma unroll
    for (int s = 0; s < NT; ++s)
#pragma unroll
      for (int u = 0; u < GROUP; ++u) a[s][u] = a_next[s][u];
    group = next;
  }
#pragma unroll
  for (int s = 0; s < NT; ++s) *(f32x4*)(partial + ((wave * NT + s) * 64 + lane) * 4) = acc[s];
  __syncthreads();
  if (wave >= NT) return;
  const int s = wave;
  f32x4 total = (f32x4){0.f, 0.f, 0.f, 0.f};
  for (int v = 0; v < WAVES; ++v) total += *(const f32x4*)(partial + ((v * NT + s) * 64 + lane) * 4);
  const int m = r;
  const int n_first = ((int)blockIdx.x * NT + s) * 16 + g * 4;
  if (m >= M) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) total[i] += bias_here[i];
  if (GATED) {
    TO* dst = out + (size_t)m * (N / 2) + n_first / 2;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (n_first + 2 * i + 1 < N) {
        const float gate = total[2 * i], up = total[2 * i + 1];
        dst[i] = from_float<TO>(gate / (1.f + expf(-gate)) * up);
      }
    }
  } else {
    TO* dst = out + ((size_t)blockIdx.y * M + m) * N + n_first;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n_first + i < N) dst[i] = from_float<TO>(total[i]);
  }
}

template <int NT, typename TO, bool GATED>
static int launch_pair(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int M, int N,
                       int K, int splits, hipStream_t stream) {
  const size_t lds = (size_t)4 * NT * 64 * 4 * sizeof(float);
  hipLaunchKernelGGL((gemm_pair_kernel<4, NT, TO, GATED>), dim3((N + 16 * NT - 1) / (16 * NT), splits), dim3(256), lds,
                     stream, (const bf16_t*)x, (const bf16_t*)w, bias, bias_is_float, (TO*)out, M, N, K, K / splits);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- the streams through LDS
// gemm_stream: gemm_skinny / gemm_pair for up to 16 rows of x with both operands brought through LDS.
// The matrix cores take a weight row as a row of the A operand, lane (r, g) holding k = 8g .. 8g+7 of
// row r, so the four lanes the address unit serves together (r .. r+3 at one g) would read 16 bytes
// of four different rows, four cache lines, and a load of a wave costs that unit four times what
// 64 bytes in a row cost it; x is read the same way.  Here lane L instead asks for piece L % 4 of row
// L / 4 (a quad reads 64 bytes of one row), straight into LDS (global_load_lds_dwordx4: the wave's 1 KB
// lands in lane order), and lane (r, g) reads its operand back from slot 4 r + g.  The pieces of a
// row are swizzled by bits 1-2 of the row so that the eight lanes LDS serves together hit all banks.
// Every wave has STAGES stages of its own, a stage holding one group of G steps of 32 k of its NT
// weight tiles and of x; nothing is shared between waves before the end, so the only waits are the
// wave's own: for its loads to land (counted, so that the younger stage may still be under way) and
// for its reads to come back before the stage is asked for anew.  The reads of LDS are written as
// instructions: left to the compiler, every read of LDS waits for all loads into LDS under way.
#define STREAM_STAGES 2
#define STREAM_CHUNK 1024  // one 32-k step of 16 rows

template <int OFFSET>
__device__ __forceinline__ void stream_read(bf16x8& operand, unsigned at) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(operand) : "v"(at), "n"(OFFSET) : "memory");
}
template <int I, int COUNT>
struct StreamReads {
  static __device__ __forceinline__ void run(bf16x8* operands, unsigned at) {
    stream_read<I * STREAM_CHUNK>(operands[I], at);
    StreamReads<I + 1, COUNT>::run(operands, at);
  }
};
template <int COUNT>
struct StreamReads<COUNT, COUNT> {
  static __device__ __forceinline__ void run(bf16x8*, unsigned) {}
};
template <int N>
__device__ __forceinline__ void stream_wait_loads() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// MT: 16-row tiles of x (up to 16 MT rows).  A stage then holds MT chunks of x beside the NT of the
// weights for every step, and each weight operand meets MT operands of x.
template <int WAVES, int NT, int MT, int G, typename TO, bool GATED>
__global__ __launch_bounds__(WAVES * 64) void gemm_stream_kernel(const bf16_t* __restrict__ x,
                                                                 const bf16_t* __restrict__ w,
                                                                 const void* __restrict__ bias, int bias_is_float,
                                                                 TO* __restrict__ out, int M, int N, int K,
                                                                 int k_split) {
  extern __shared__ __attribute__((aligned(16))) unsigned char stream_lds[];
  constexpr int OPERANDS = (NT + MT) * G;                // of one group: the weight tiles' steps, then x's
  constexpr int STAGE_BYTES = OPERANDS * STREAM_CHUNK;
  constexpr int WAVE_BYTES = STREAM_STAGES * STAGE_BYTES;
  constexpr int TILES = NT * MT;                         // of the result
  static_assert(OPERANDS <= 31, "a group's loads are counted in vmcnt beside a second group's");
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int k_first = blockIdx.y * k_split;
  // what this lane asks for: piece (L % 4) ^ f(row) of row L / 4, and where lane (r, g) finds its own
  const int load_row = lane >> 2, load_piece = (lane & 3) ^ ((load_row >> 1) & 3);
  const bf16_t* w_src[NT];
#pragma unroll
  for (int s = 0; s < NT; ++s)
    w_src[s] = w + (size_t)min(((int)blockIdx.x * NT + s) * 16 + load_row, N - 1) * K + k_first + load_piece * 8;
  // rows of x beyond M are read as row M - 1: their columns of the result are dropped at the end
  const bf16_t* x_src[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) x_src[t] = x + (size_t)min(t * 16 + load_row, M - 1) * K + k_first + load_piece * 8;
  unsigned char* mine = stream_lds + (size_t)wave * WAVE_BYTES;
  const unsigned read_at = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)mine +
                           (unsigned)(4 * r + (g ^ ((r >> 1) & 3))) * 16;

  // the bias of the four outputs this lane will finish first (wave v finishes tile v, of weight tile
  // v / MT) is asked for now
  float bias_here[4] = {0.f, 0.f, 0.f, 0.f};
  if (bias && blockIdx.y == 0 && wave < TILES) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      bias_here[i] =
          load_as_float(bias, bias_is_float, min(((int)blockIdx.x * NT + wave / MT) * 16 + g * 4 + i, N - 1));
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // so that the counts below count the stream alone

  auto request = [&](int group, int stage) {
    unsigned char* to = mine + (size_t)stage * STAGE_BYTES;
    const int k = group * G * STEP;
#pragma unroll
    for (int u = 0; u < G; ++u) {
#pragma unroll
      for (int s = 0; s < NT; ++s)
        __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(w_src[s] + k + u * STEP),
                                         (void __attribute__((address_space(3)))*)(to + (s * G + u) * STREAM_CHUNK), 16,
                                         0, 0);
#pragma unroll
      for (int t = 0; t < MT; ++t)
        __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(x_src[t] + k + u * STEP),
                                         (void __attribute__((address_space(3)))*)(to + ((NT + t) * G + u) * STREAM_CHUNK),
                                         16, 0, 0);
    }
  };

  f32x4 acc[NT][MT];
#pragma unroll
  for (int s = 0; s < NT; ++s)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[s][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const int groups = k_split / (STEP * G);
  int group = wave;
  if (group < groups) request(group, 0);
  if (group + WAVES < groups) request(group + WAVES, 1);
  for (int stage = 0; group < groups; group += WAVES, stage ^= 1) {
    // this stage has landed once at most the next group's loads are under way
    if (group + WAVES < groups) stream_wait_loads<OPERANDS>();
    else stream_wait_loads<0>();
    bf16x8 operands[OPERANDS];
    StreamReads<0, OPERANDS>::run(operands, read_at + (unsigned)stage * STAGE_BYTES);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < OPERANDS; ++i) asm volatile("" : "+v"(operands[i]));  // used only after the wait
    if (group + 2 * WAVES < groups) request(group + 2 * WAVES, stage);       // the stage is read: ask anew
#pragma unroll
    for (int u = 0; u < G; ++u)
#pragma unroll
      for (int s = 0; s < NT; ++s)
#pragma unroll
        for (int t = 0; t < MT; ++t)
          acc[s][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(operands[s * G + u], operands[(NT + t) * G + u],
                                                              acc[s][t], 0, 0, 0);
  }

  __syncthreads();  // every wave is done with its stages: LDS is free for the waves' sums
  float* partial = (float*)stream_lds;  // [WAVES][TILES][64 lanes][4]
#pragma unroll
  for (int s = 0; s < NT; ++s)
#pragma unroll
    for (int t = 0; t < MT; ++t) *(f32x4*)(partial + ((wave * TILES + s * MT + t) * 64 + lane) * 4) = acc[s][t];
  __syncthreads();
  for (int tile = wave; tile < TILES; tile += WAVES) {
    const int s = tile / MT;
    f32x4 total = (f32x4){0.f, 0.f, 0.f, 0.f};
    for (int v = 0; v < WAVES; ++v) total += *(const f32x4*)(partial + ((v * TILES + tile) * 64 + lane) * 4);
    const int m = (tile % MT) * 16 + r;
    const int n_first = ((int)blockIdx.x * NT + s) * 16 + g * 4;
    if (m >= M) continue;
    if (tile == wave) {
#pragma unroll
      for (int i = 0; i < 4; ++i) total[i] += bias_here[i];
    } else if (bias && blockIdx.y == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) total[i] += load_as_float(bias, bias_is_float, min(n_first + i, N - 1));
    }
    if (GATED) {
      TO* dst = out + (size_t)m * (N / 2) + n_first / 2;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if (n_first + 2 * i + 1 < N) {
          const float gate = total[2 * i], up = total[2 * i + 1];
          dst[i] = from_float<TO>(gate / (1.f + expf(-gate)) * up);
        }
      }
    } else {
      TO* dst = out + ((size_t)blockIdx.y * M + m) * N + n_first;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n_first + i < N) dst[i] = from_float<TO>(total[i]);
    }
  }
}

template <int WAVES, int NT, int MT, int G, typename TO, bool GATED>
static int launch_stream(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int M, int N,
                         int K, int splits, hipStream_t stream) {
  const size_t stages = (size_t)WAVES * STREAM_STAGES * (NT + MT) * G * STREAM_CHUNK;
  const size_t sums = (size_t)WAVES * NT * MT * 64 * 4 * sizeof(float);
  const size_t lds = stages > sums ? stages : sums;
  if (lds > 64 * 1024) {
    static bool asked = false;
    if (!asked) {
      if (hipFuncSetAttribute((const void*)gemm_stream_kernel<WAVES, NT, MT, G, TO, GATED>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return ERR_BAD_ARGUMENT;
      asked = true;
    }
  }
  hipLaunchKernelGGL((gemm_stream_kernel<WAVES, NT, MT, G, TO, GATED>), dim3((N + 16 * NT - 1) / (16 * NT), splits),
                     dim3(WAVES * 64), lds, stream, (const bf16_t*)x, (const bf16_t*)w, bias, bias_is_float, (TO*)out, M,
                     N, K, K / splits);
  return LAUNCH_STATUS();
}

// One tile a wave in groups of four steps, or two tiles in groups of two.  Measured at 8 rows against
// gemm_skinny / gemm_pair, in a captured chain over different weights: 1.5B sizes qkv 4.9 -> 4.1 us,
// gate/up 15.7 -> 13.0, down 9.5 -> 8.7, o 4.8 -> 3.4; 7B sizes qkv 13.8 -> 10.6 (two tiles), o 9.8 ->
// 7.9, gate/up 54.7 -> 52.1; 32B sizes qkv 20.9 -> 16.3 (two tiles).  Where a wave walks a long K
// for four tiles that share its x (the down projections and the 32B sizes' gate/up) gemm_pair's
// registers stay ahead, and the caller keeps it there.
// M <= 16, K / splits a multiple of 128.
template <typename TO, bool GATED>
static int pick_stream(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int M, int N, int K,
                       int splits, hipStream_t stream, int nt = 0, int g = 0) {
  const long tiles = (N + 15) / 16;
  if (M > 16) {
    // 17 to 64 rows: two or four tiles of x.  nt, g: 0 = by the sizes, else as asked (measurements)
    if (nt == 0) nt = tiles * splits >= 2048 ? 2 : 1;
    if (g == 0) g = 1;
#define ROWS_CASE(NT_, MT_, G_)                                                                              \
  if (nt == NT_ && g == G_ && M <= 16 * MT_)                                                                 \
    return launch_stream<4, NT_, MT_, G_, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
    ROWS_CASE(1, 2, 1)
    ROWS_CASE(2, 2, 1)
    ROWS_CASE(1, 2, 2)
    ROWS_CASE(2, 2, 2)
    ROWS_CASE(1, 4, 1)
    ROWS_CASE(2, 4, 1)
    ROWS_CASE(1, 4, 2)
    ROWS_CASE(2, 4, 2)
    ROWS_CASE(4, 2, 1)
    ROWS_CASE(4, 4, 1)
#undef ROWS_CASE
    return ERR_BAD_ARGUMENT;
  }
  // two tiles a wave for a middling number of weight rows over a K that is not cut (the qkv products of the
  // 7B and 32B sizes: 11.6 -> 10.6 and 20.0 -> 17.5 us); with K cut over workgroups one tile is as good or
  // better (the 32B sizes' o in two parts: 13.5 us against 16.9)
  if (splits == 1 && tiles >= 256 && tiles < 1024 && tiles * K >= 1000000L)
    return launch_stream<4, 2, 1, 2, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
  return launch_stream<4, 1, 1, 4, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
}

// The same product as llmserve_gemm_skinny, always through gemm_stream (tests and measurements); up to 64 rows.
static int stream_entry(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int out_is_float,
                        int gated, int M, int N, int K, int splits, hipStream_t stream, int nt, int g) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || splits < 1 || K % splits || (K / splits) % (STEP * GROUP) || (gated && N % 2))
    return ERR_BAD_ARGUMENT;
  if (splits > 1 && (gated || !out_is_float)) return ERR_BAD_ARGUMENT;
  if (gated)
    return out_is_float ? pick_stream<float, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream, nt, g)
                        : pick_stream<bf16_t, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream, nt, g);
  return out_is_float ? pick_stream<float, false>(x, w, bias, bias_is_float, out, M, N, K, splits, stream, nt, g)
                      : pick_stream<bf16_t, false>(x, w, bias, bias_is_float, out, M, N, K, 1, stream, nt, g);
}

extern "C" int llmserve_gemm_stream(const void* x, const void* w, const void* bias, int bias_is_float, void* out,
                                    int out_is_float, int gated, int M, int N, int K, int splits,
                                    hipStream_t stream) {
  return stream_entry(x, w, bias, bias_is_float, out, out_is_float, gated, M, N, K, splits, stream, 0, 0);
}

// The same for 17 to 64 rows with the shape asked for (measurements): nt weight tiles a workgroup (1, 2),
// groups of g steps (1, 2).
extern "C" int llmserve_gemm_stream_shaped(const void* x, const void* w, const void* bias, int bias_is_float,
                                           void* out, int out_is_float, int gated, int M, int N, int K, int splits,
                                           int nt, int g, hipStream_t stream) {
  if (M <= 16) return ERR_BAD_ARGUMENT;
  return stream_entry(x, w, bias, bias_is_float, out, out_is_float, gated, M, N, K, splits, stream, nt, g);
}

// ---------------------------------------------------------------------------- key splits merged on the way in
// gemm_merged: gemm_skinny for up to 16 rows whose x is the output of decode attention that was left in
// key splits (attention_bf16.hip, `unmerged`): for every (row, head) S results, each divided by its own sum
// of weights, with each split's maximum m_s (in units of log2) and sum of weights l_s.  The row's true
// x[head] = sum_s c_s x_s[head] with c_s = l_s 2^(m_s - m) / sum_t l_t 2^(m_t - m), m the largest m_s.
// A kernel of its own that merges costs a decode step as much as the attention itself (a launch and two
// trips to memory); here the lanes that load x for the MFMA's B operand merge as they load.  Heads are
// 128 wide, a group of K (128 k), so a wave's group is one head and its S coefficients are made once.
template <int WAVES, int S>
__global__ __launch_bounds__(WAVES * 64) void gemm_merged_kernel(const bf16_t* __restrict__ split_x,
                                                                 const float* __restrict__ split_ml,
                                                                 const bf16_t* __restrict__ w,
                                                                 const void* __restrict__ bias, int bias_is_float,
                                                                 float* __restrict__ out, int M, int N, int K,
                                                                 int k_split) {
  extern __shared__ float partial[];  // [WAVES][64 lanes][4]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int n = min((int)blockIdx.x * 16 + r, N - 1);
  const int heads = K / (STEP * GROUP);
  const int head_first = blockIdx.y * (k_split / (STEP * GROUP));
  const bf16_t* w_row = w + (size_t)n * K + (size_t)head_first * (STEP * GROUP) + g * 8;
  const bool x_live = r < M;
  const int row = min(r, M - 1);
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  const bool with_bias = bias && blockIdx.y == 0;
  float bias_here[4] = {0.f, 0.f, 0.f, 0.f};
  if (with_bias) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      bias_here[i] = load_as_float(bias, bias_is_float, min((int)blockIdx.x * 16 + g * 4 + i, N - 1));
  }
  const int groups = k_split / (STEP * GROUP);
  for (int group = wave; group < groups; group += WAVES) {
    bf16x8 a[GROUP];
#pragma unroll
    for (int u = 0; u < GROUP; ++u) a[u] = load8_stream(w_row + (group * GROUP + u) * STEP);
    // split_x is [head][split][piece of 8][16 rows][8]: this lane's piece 4 u + g of row `row`, beside the
    // same piece of the next rows, which the next lanes ask for
    const size_t slot = (size_t)(head_first + group) * S;
    float2 ml[S];
    bf16x8 piece[S][GROUP];
#pragma unroll
    for (int s = 0; s < S; ++s) {
      ml[s] = *(const float2*)(split_ml + ((slot + s) * 16 + row) * 2);
#pragma unroll
      for (int u = 0; u < GROUP; ++u)
        piece[s][u] = load8(split_x + (((slot + s) * (STEP * GROUP / 8) + u * 4 + g) * 16 + row) * 8);
    }
    float best = -INFINITY;
#pragma unroll
    for (int s = 0; s < S; ++s) best = fmaxf(best, ml[s].x);
    float share[S], total = 0.f;
#pragma unroll
    for (int s = 0; s < S; ++s) {
      share[s] = ml[s].x == -INFINITY ? 0.f : ml[s].y * __builtin_amdgcn_exp2f(ml[s].x - best);  // a split that saw no key
      total += share[s];
    }
    const float inverse = total > 0.f ? 1.f / total : 0.f;
#pragma unroll
    for (int u = 0; u < GROUP; ++u) {
      float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < S; ++s) {
        const float c = share[s] * inverse;
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = fmaf(c, share[s] > 0.f ? (float)piece[s][u][i] : 0.f, x[i]);
      }
      bf16x8 b;
#pragma unroll
      for (int i = 0; i < 8; ++i) b[i] = x_live ? (bf16_t)x[i] : (bf16_t)0.f;
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b, acc, 0, 0, 0);
    }
  }
  *(f32x4*)(partial + (wave * 64 + lane) * 4) = acc;
  __syncthreads();
  if (wave > 0) return;
  f32x4 total_tile = {0.f, 0.f, 0.f, 0.f};
  for (int v = 0; v < WAVES; ++v) total_tile += *(const f32x4*)(partial + (v * 64 + lane) * 4);
  const int n_first = blockIdx.x * 16 + g * 4;
  if (r >= M) return;
  float* dst = out + ((size_t)blockIdx.y * M + r) * N + n_first;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (n_first + i < N) dst[i] = total_tile[i] + bias_here[i];
}

template <int S>
static int launch_merged(const void* split_x, const float* split_ml, const void* w, const void* bias, int bias_is_float,
                         float* out, int M, int N, int K, int k_splits, hipStream_t stream) {
  const int groups = K / k_splits / (STEP * GROUP);
  const dim3 grid((N + 15) / 16, k_splits);
  if (groups <= 4)
    hipLaunchKernelGGL((gemm_merged_kernel<4, S>), grid, dim3(256), 4 * 64 * 4 * sizeof(float), stream,
                       (const bf16_t*)split_x, split_ml, (const bf16_t*)w, bias, bias_is_float, out, M, N, K, K / k_splits);
  else
    hipLaunchKernelGGL((gemm_merged_kernel<8, S>), grid, dim3(512), 8 * 64 * 4 * sizeof(float), stream,
                       (const bf16_t*)split_x, split_ml, (const bf16_t*)w, bias, bias_is_float, out, M, N, K, K / k_splits);
  return LAUNCH_STATUS();
}

// out [k_splits, M, N] float32 partial sums of x . w^T (+ bias in the first), x [M, K] being the merge of
// split_x bfloat16 [K / 128, splits, 16, 16 rows, 8] with split_ml float32 [K / 128, splits, 16 rows, 2] as above.
// M <= 16; K a multiple of 128 * k_splits; splits 2, 3, 4, 6 or 8.
extern "C" int llmserve_gemm_merged(const void* split_x, const float* split_ml, int splits, const void* w,
                                    const void* bias, int bias_is_float, float* out, int M, int N, int K,
                                    int k_splits, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 16 || K <= 0 || k_splits < 1 || K % (STEP * GROUP * k_splits)) return ERR_BAD_ARGUMENT;
  switch (splits) {
    case 2: return launch_merged<2>(split_x, split_ml, w, bias, bias_is_float, out, M, N, K, k_splits, stream);
    case 3: return launch_merged<3>(split_x, split_ml, w, bias, bias_is_float, out, M, N, K, k_splits, stream);
    case 4: return launch_merged<4>(split_x, split_ml, w, bias, bias_is_float, out, M, N, K, k_splits, stream);
    case 6: return launch_merged<6>(split_x, split_ml, w, bias, bias_is_float, out, M, N, K, k_splits, stream);
    case 8: return launch_merged<8>(split_x, split_ml, w, bias, bias_is_float, out, M, N, K, k_splits, stream);
    default: return ERR_BAD_ARGUMENT;
  }
}

// ---------------------------------------------------------------------------- 16 < M <= 64
// gemm_medium: the same product for up to 64 rows of x.  With more than one 16-row tile of x,
// loading x per wave would cost more than streaming the weights, so a workgroup takes 64
// weight rows (four waves, one 16-row tile each) times four slices of its K range (sixteen
// waves), and the four waves of a K slice share the slice's 128 columns of x through LDS
// (rows padded by 16 bytes, so that the 16-byte reads of an MFMA operand spread over all
// banks).  K may be cut over workgroups too (blockIdx.y), leaving partial sums as above.
#define MEDIUM_ROWS 64
#define X_STRIDE (STEP * GROUP + 8)  // bf16 elements per staged row of x: 128 + padding

template <int MT, typename TO, bool GATED>
__global__ __launch_bounds__(1024) void gemm_medium_kernel(const bf16_t* __restrict__ x,
                                                           const bf16_t* __restrict__ w,
                                                           const void* __restrict__ bias, int bias_is_float,
                                                           TO* __restrict__ out, int M, int N, int K,
                                                           int groups_per_block) {
  extern __shared__ float shared_medium[];
  bf16_t* staged = (bf16_t*)shared_medium;  // [4 slices][MT * 16 rows][X_STRIDE]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int row_tile = wave & 3, slice = wave >> 2;
  const int r = lane & 15, g = lane >> 4;
  const int n = min((int)blockIdx.x * MEDIUM_ROWS + row_tile * 16 + r, N - 1);
  const int total_groups = K / (STEP * GROUP);
  const int group_begin = blockIdx.y * groups_per_block;
  const int group_end = min(total_groups, group_begin + groups_per_block);
  const bf16_t* w_row = w + (size_t)n * K + g * 8;
  bf16_t* my_stage = staged + (size_t)slice * (MT * 16) * X_STRIDE;
  const int slice_thread = threadIdx.x & 255;  // index among the four waves of this K slice

  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // The slice's 256 threads bring x[0 .. MT*16)[a group's 128 columns] into LDS, 16 bytes a piece,
  // MT pieces a thread: first into registers (issued a round ahead), then into LDS.
  bf16x8 x_piece[MT];
  auto fetch_x = [&](int group) {
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int piece = slice_thread + i * 256, row = piece >> 4, part = piece & 15;
      x_piece[i] = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
      if (row < M) x_piece[i] = load8(x + (size_t)row * K + (size_t)group * (STEP * GROUP) + part * 8);
    }
  };
  auto stage_x = [&]() {
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int piece = slice_thread + i * 256, row = piece >> 4, part = piece & 15;
      *(bf16x8*)(my_stage + (size_t)row * X_STRIDE + part * 8) = x_piece[i];
    }
  };
  // Rounds go in runs of three whose weights are all requested before the first is used, so the
  // weight stream never waits for the arithmetic or for x.
  constexpr int RUN = 3;
  const int rounds = (groups_per_block + 3) / 4;
  auto group_of = [&](int round) { return group_begin + round * 4 + slice; };
  if (rounds > 0 && group_of(0) < group_end) fetch_x(group_of(0));
  for (int base = 0; base < rounds; base += RUN) {
    bf16x8 a[RUN][GROUP];
#pragma unroll
    for (int j = 0; j < RUN; ++j) {
      if (base + j < rounds && group_of(base + j) < group_end) {
#pragma unroll
        for (int u = 0; u < GROUP; ++u) a[j][u] = load8_stream(w_row + (group_of(base + j) * GROUP + u) * STEP);
      }
    }
#pragma unroll
    for (int j = 0; j < RUN; ++j) {
      const int round = base + j;
      if (round >= rounds) break;
      const bool live = group_of(round) < group_end;
      __syncthreads();  // the previous round's reads of the staged x are done
      if (live) stage_x();
      if (round + 1 < rounds && group_of(round + 1) < group_end) fetch_x(group_of(round + 1));
      __syncthreads();
      if (live) {
#pragma unroll
        for (int t = 0; t < MT; ++t) {
#pragma unroll
          for (int u = 0; u < GROUP; ++u) {
            const bf16x8 b = *(const bf16x8*)(my_stage + (size_t)(t * 16 + r) * X_STRIDE + u * STEP + g * 8);
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j][u], b, acc[t], 0, 0, 0);
          }
        }
      }
    }
  }
  __syncthreads();
  // add the four K slices of each row tile through LDS: [slice][row_tile][MT][64 lanes][4]
  float* partial = shared_medium;
#pragma unroll
  for (int t = 0; t < MT; ++t) *(f32x4*)(partial + (((slice * 4 + row_tile) * MT + t) * 64 + lane) * 4) = acc[t];
  __syncthreads();
  if (slice != 0) return;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    f32x4 total = (f32x4){0.f, 0.f, 0.f, 0.f};
    for (int v = 0; v < 4; ++v) total += *(const f32x4*)(partial + (((v * 4 + row_tile) * MT + t) * 64 + lane) * 4);
    const int m = t * 16 + r;
    const int n_first = blockIdx.x * MEDIUM_ROWS + row_tile * 16 + g * 4;
    if (m >= M) continue;
    if (bias && blockIdx.y == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n_first + i < N) total[i] += load_as_float(bias, bias_is_float, n_first + i);
    }
    if (GATED) {
      TO* dst = out + (size_t)m * (N / 2) + n_first / 2;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if (n_first + 2 * i + 1 < N) {
          const float gate = total[2 * i], up = total[2 * i + 1];
          dst[i] = from_float<TO>(gate / (1.f + expf(-gate)) * up);
        }
      }
    } else {
      TO* dst = out + ((size_t)blockIdx.y * M + m) * N + n_first;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n_first + i < N) dst[i] = from_float<TO>(total[i]);
    }
  }
}

template <int MT, typename TO, bool GATED>
static int launch_medium(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int M, int N,
                         int K, int splits, hipStream_t stream) {
  const size_t stage = (size_t)4 * MT * 16 * X_STRIDE * sizeof(bf16_t);
  const size_t merge = (size_t)4 * 4 * MT * 64 * 4 * sizeof(float);
  const size_t lds = stage > merge ? stage : merge;
  if (lds > 64 * 1024) {
    static bool asked = false;
    if (!asked) {
      if (hipFuncSetAttribute((const void*)gemm_medium_kernel<MT, TO, GATED>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return ERR_BAD_ARGUMENT;
      asked = true;
    }
  }
  const int groups = K / (STEP * GROUP);
  const int per_block = (groups + splits - 1) / splits;
  hipLaunchKernelGGL((gemm_medium_kernel<MT, TO, GATED>), dim3((N + MEDIUM_ROWS - 1) / MEDIUM_ROWS, splits),
                     dim3(1024), lds, stream, (const bf16_t*)x, (const bf16_t*)w, bias, bias_is_float, (TO*)out, M, N,
                     K, per_block);
  return LAUNCH_STATUS();
}

template <typename TO, bool GATED>
static int pick_medium(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int M, int N,
                       int K, int splits, hipStream_t stream) {
  if (M <= 32) return launch_medium<2, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
  return launch_medium<4, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
}

// As llmserve_gemm_skinny, for 16 < M <= 64 and K a multiple of 128.  With splits > 1 the K
// range is cut into `splits` runs of ceil(K / 128 / splits) groups of 128 and `out` is
// [splits, M, N] partial sums.
extern "C" int llmserve_gemm_medium(const void* x, const void* w, const void* bias, int bias_is_float, void* out,
                                    int out_is_float, int gated, int M, int N, int K, int splits,
                                    hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || K % (STEP * GROUP) || (gated && N % 2) || splits < 1) return ERR_BAD_ARGUMENT;
  if (splits > 1 && (gated || !out_is_float)) return ERR_BAD_ARGUMENT;
  if (gated)
    return out_is_float ? pick_medium<float, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream)
                        : pick_medium<bf16_t, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream);
  return out_is_float ? pick_medium<float, false>(x, w, bias, bias_is_float, out, M, N, K, splits, stream)
                      : pick_medium<bf16_t, false>(x, w, bias, bias_is_float, out, M, N, K, 1, stream);
}

// ---------------------------------------------------------------------------- 17 to 64 rows through a ring
// gemm_ring: the product for 17 to 64 rows of x, bound by how fast the weights come from memory.  A
// workgroup of four waves owns NT tiles of 16 weight rows over its whole K range and MT tiles of x; both
// go through a ring of DEPTH stages of KSTEPS * 32 k in LDS that the waves share, filled straight from
// memory (global_load_lds_dwordx4, a chunk of 16 rows x 32 k in lane order, laid out and swizzled as in
// gemm_stream) DEPTH - 1 stages ahead of the one being multiplied: what a CU has under way is then that
// many stages of weights whatever the compiler does with the registers, and a weight row is read from memory
// once for all rows of x.  The waves divide a stage's chunks between them; one barrier a stage says that
// everyone's loads have landed and that the stage before may be filled again.  A wave multiplies one tile of x
// (two, with eight tiles of x: up to 128 rows) with its share of the weight tiles, so no sums meet at the end.
__device__ __forceinline__ void ring_load(const bf16_t* from, unsigned to) {
  // (M0 names the place in LDS; it is put back, the compiler keeps other things there)
  unsigned kept;
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, off\n\ts_mov_b32 m0, %0"
               : "=&s"(kept)
               : "s"(to), "v"(from)
               : "memory");
}

// waits until at most `younger` stages' loads of this wave (PER_WAVE each) are under way; younger <= MOST
template <int PER_WAVE, int MOST>
__device__ __forceinline__ void ring_wait(int younger) {
  if constexpr (MOST == 0) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  } else {
    if (younger >= MOST) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(MOST * PER_WAVE) : "memory");
    else ring_wait<PER_WAVE, MOST - 1>(younger);
  }
}

template <int NT, int MT, int KSTEPS, int DEPTH, typename TO, bool GATED>
__global__ __launch_bounds__(256) void gemm_ring_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                        const void* __restrict__ bias, int bias_is_float,
                                                        TO* __restrict__ out, int M, int N, int K, int k_split) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ring[];
  constexpr int XPW = MT > 4 ? MT / 4 : 1;   // tiles of x a wave multiplies
  constexpr int XGROUPS = MT / XPW;          // groups of waves by their tiles of x
  constexpr int WAYS = 4 / XGROUPS;          // groups of waves that divide the weight tiles between them
  constexpr int MINE = NT / WAYS;            // weight tiles a wave multiplies
  constexpr int TILES = NT + MT;        // of a stage, each KSTEPS chunks of 1 KB
  constexpr int STAGE_BYTES = TILES * KSTEPS * STREAM_CHUNK;
  constexpr int PER_WAVE = TILES * KSTEPS / 4;  // chunks a wave brings per stage
  constexpr int APART = 4 / KSTEPS;             // tiles between two chunks of a wave
  static_assert(MT == 2 || MT == 4 || MT == 8, "two, four or eight tiles of x");
  static_assert(KSTEPS == 2 || KSTEPS == 4, "stages of 64 or 128 k");
  static_assert(NT % WAYS == 0, "the waves divide the weight tiles evenly");
  static_assert(TILES * KSTEPS % 4 == 0, "the waves divide a stage's chunks evenly");
  static_assert((DEPTH - 2) * PER_WAVE <= 63, "the loads under way are counted in vmcnt");
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int k_first = blockIdx.y * k_split;
  const int load_row = lane >> 2, load_piece = (lane & 3) ^ ((load_row >> 1) & 3);
  // chunk j of this wave: k-step wave % KSTEPS of tile j * APART + wave / KSTEPS (the weight tiles, then x's)
  const int my_step = wave % KSTEPS, my_first = wave / KSTEPS;
  const bf16_t* src[PER_WAVE];  // this lane's piece of each, in the first stage
#pragma unroll
  for (int j = 0; j < PER_WAVE; ++j) {
    const int tile = j * APART + my_first;
    // rows of x beyond M are read as row M - 1: their columns of the result are dropped at the end
    const bf16_t* row = tile < NT ? w + (size_t)min(((int)blockIdx.x * NT + tile) * 16 + load_row, N - 1) * K
                                  : x + (size_t)min((tile - NT) * 16 + load_row, M - 1) * K;
    src[j] = row + k_first + my_step * STEP + load_piece * 8;
  }
  const unsigned base = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)ring;
  const int x_tile = (wave % XGROUPS) * XPW, first_tile = wave / XGROUPS;  // the wave's first tile of x, of weights
  const unsigned read_at = base + (unsigned)(4 * r + (g ^ ((r >> 1) & 3))) * 16;
  const unsigned read_w = read_at + (unsigned)first_tile * KSTEPS * STREAM_CHUNK;
  const unsigned read_x = read_at + (unsigned)(NT + x_tile) * KSTEPS * STREAM_CHUNK;

  // the bias of the outputs this lane will finish: all asked for at once, of either type
  float bias_here[MINE][4];
  bf16_t bias_short[MINE][4];
  const bool biased = bias && blockIdx.y == 0;
#pragma unroll
  for (int i = 0; i < MINE; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = min(((int)blockIdx.x * NT + first_tile + WAYS * i) * 16 + g * 4 + j, N - 1);
      bias_here[i][j] = 0.f;
      if (biased && bias_is_float) bias_here[i][j] = ((const float*)bias)[n];
      if (biased && !bias_is_float) bias_short[i][j] = ((const bf16_t*)bias)[n];
    }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // so that the counts below count the ring's loads alone
  if (biased && !bias_is_float) {
#pragma unroll
    for (int i = 0; i < MINE; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) bias_here[i][j] = (float)bias_short[i][j];
  }

  const int stages = k_split / (KSTEPS * STEP);
  auto request = [&](int stage) {
    const unsigned to = base + (unsigned)(stage % DEPTH) * STAGE_BYTES + (unsigned)(my_first * KSTEPS + my_step) * STREAM_CHUNK;
#pragma unroll
    for (int j = 0; j < PER_WAVE; ++j)
      ring_load(src[j] + (size_t)stage * (KSTEPS * STEP), to + (unsigned)(j * APART * KSTEPS) * STREAM_CHUNK);
  };
  f32x4 acc[MINE][XPW];
#pragma unroll
  for (int i = 0; i < MINE; ++i)
#pragma unroll
    for (int j = 0; j < XPW; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < DEPTH - 1; ++s)
    if (s < stages) request(s);
  for (int stage = 0; stage < stages; ++stage) {
    // this wave's loads of the stage have landed once only the younger stages' are under way
    ring_wait<PER_WAVE, DEPTH - 2>(stages - 1 - stage);
    // everyone's have, and everyone has read the stage before this one: it may be filled again
    asm volatile("s_barrier" ::: "memory");
    if (stage + DEPTH - 1 < stages) request(stage + DEPTH - 1);
    const unsigned slot = (unsigned)(stage % DEPTH) * STAGE_BYTES;
    bf16x8 from_x[XPW][KSTEPS], from_w[MINE][KSTEPS];
#pragma unroll
    for (int j = 0; j < XPW; ++j) StreamReads<0, KSTEPS>::run(from_x[j], read_x + slot + (unsigned)(j * KSTEPS) * STREAM_CHUNK);
#pragma unroll
    for (int i = 0; i < MINE; ++i) StreamReads<0, KSTEPS>::run(from_w[i], read_w + slot + (unsigned)(WAYS * i * KSTEPS) * STREAM_CHUNK);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int j = 0; j < XPW; ++j)
#pragma unroll
      for (int u = 0; u < KSTEPS; ++u) asm volatile("" : "+v"(from_x[j][u]));  // used only after the wait
#pragma unroll
    for (int i = 0; i < MINE; ++i)
#pragma unroll
      for (int u = 0; u < KSTEPS; ++u) asm volatile("" : "+v"(from_w[i][u]));
#pragma unroll
    for (int u = 0; u < KSTEPS; ++u)
#pragma unroll
      for (int i = 0; i < MINE; ++i)
#pragma unroll
        for (int j = 0; j < XPW; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(from_w[i][u], from_x[j][u], acc[i][j], 0, 0, 0);
  }

  // The results leave through LDS as whole rows of the workgroup's tile, 16 bytes a lane, where the sizes allow it
  // (each lane holds four neighbouring columns of one row: stored from the registers, an instruction writes 8 or 16
  // bytes to each of sixteen rows).
  constexpr int COLUMNS = GATED ? NT * 8 : NT * 16;        // of the workgroup's tile of the result
  constexpr int PER_PIECE = 16 / (int)sizeof(TO);           // columns in 16 bytes
  const int pitch = GATED ? N / 2 : N;                      // of a row of out
  const int column0 = (int)blockIdx.x * COLUMNS;
  const int valid = min(COLUMNS, pitch - column0);
  TO* plane = out + (size_t)blockIdx.y * M * pitch;
  const bool whole_pieces = pitch % PER_PIECE == 0 && valid % PER_PIECE == 0 && COLUMNS % PER_PIECE == 0 &&
                            ((size_t)out & 15) == 0;
  if (whole_pieces) {
    asm volatile("s_barrier" ::: "memory");  // everyone has read the last stage: the ring is free
    TO* tile = (TO*)ring;                    // [16 MT rows][COLUMNS]
#pragma unroll
    for (int t = 0; t < XPW; ++t) {
      const int m = (x_tile + t) * 16 + r;
#pragma unroll
      for (int i = 0; i < MINE; ++i) {
        f32x4 total = acc[i][t];
#pragma unroll
        for (int j = 0; j < 4; ++j) total[j] += bias_here[i][j];
        const int c_first = (first_tile + WAYS * i) * 16 + g * 4;  // column of the tile before gating
        if (GATED) {
          TO* dst = tile + m * COLUMNS + c_first / 2;
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const float gate = total[2 * j], up = total[2 * j + 1];
            dst[j] = from_float<TO>(gate / (1.f + expf(-gate)) * up);
          }
        } else {
          TO* dst = tile + m * COLUMNS + c_first;
#pragma unroll
          for (int j = 0; j < 4; ++j) dst[j] = from_float<TO>(total[j]);
        }
      }
    }
    __syncthreads();
    const int pieces_a_row = valid / PER_PIECE;
    const int rows_here = min(M, 16 * MT);
    for (int piece = threadIdx.x; piece < rows_here * pieces_a_row; piece += 256) {
      const int row = piece / pieces_a_row, at = (piece - row * pieces_a_row) * PER_PIECE;
      *(f32x4*)(plane + (size_t)row * pitch + column0 + at) = *(const f32x4*)(tile + row * COLUMNS + at);
    }
    return;
  }
#pragma unroll
  for (int t = 0; t < XPW; ++t) {
    const int m = (x_tile + t) * 16 + r;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < MINE; ++i) {
      const int n_first = ((int)blockIdx.x * NT + first_tile + WAYS * i) * 16 + g * 4;
      f32x4 total = acc[i][t];
#pragma unroll
      for (int j = 0; j < 4; ++j) total[j] += bias_here[i][j];
      if (GATED) {
        TO* dst = out + (size_t)m * (N / 2) + n_first / 2;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          if (n_first + 2 * j + 1 < N) {
            const float gate = total[2 * j], up = total[2 * j + 1];
            dst[j] = from_float<TO>(gate / (1.f + expf(-gate)) * up);
          }
        }
      } else {
        TO* dst = out + ((size_t)blockIdx.y * M + m) * N + n_first;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (n_first + j < N) dst[j] = from_float<TO>(total[j]);
      }
    }
  }
}

template <int NT, int MT, int KSTEPS, int DEPTH, typename TO, bool GATED>
static int launch_ring(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int M, int N, int K,
                       int splits, hipStream_t stream) {
  const size_t lds = (size_t)DEPTH * (NT + MT) * KSTEPS * STREAM_CHUNK;
  if ((K / splits) % (KSTEPS * STEP)) return ERR_BAD_ARGUMENT;
  if (lds > 64 * 1024) {
    static bool asked = false;
    if (!asked) {
      if (hipFuncSetAttribute((const void*)gemm_ring_kernel<NT, MT, KSTEPS, DEPTH, TO, GATED>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return ERR_BAD_ARGUMENT;
      asked = true;
    }
  }
  hipLaunchKernelGGL((gemm_ring_kernel<NT, MT, KSTEPS, DEPTH, TO, GATED>), dim3((N + 16 * NT - 1) / (16 * NT), splits),
                     dim3(256), lds, stream, (const bf16_t*)x, (const bf16_t*)w, bias, bias_is_float, (TO*)out, M, N, K,
                     K / splits);
  return LAUNCH_STATUS();
}

// nt tiles of 16 weight rows a workgroup, stages of 128 k; four stages, or three with eight tiles of x (65 to 128
// rows), which fill the LDS with five weight tiles beside them
template <typename TO, bool GATED>
static int pick_ring(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int M, int N, int K,
                     int splits, hipStream_t stream, int nt) {
#define RING_CASE(NT_)                                                                                                  \
  if (nt == NT_ && M <= 64)                                                                                             \
    return M <= 32 ? launch_ring<NT_, 2, 4, 4, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream)      \
                   : launch_ring<NT_, 4, 4, 4, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
  RING_CASE(2)
  RING_CASE(4)
  RING_CASE(6)
#undef RING_CASE
  if (nt == 5 && M > 32 && M <= 64) return launch_ring<5, 4, 4, 4, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
#define ROWS_CASE(NT_)                                                                                                  \
  if (nt == NT_ && M > 64) return launch_ring<NT_, 8, 4, 3, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
  ROWS_CASE(2)
  ROWS_CASE(4)
  ROWS_CASE(5)
#undef ROWS_CASE
  // many weight tiles a workgroup, in stages of 64 k: for a weight of so many rows that fewer tiles make several rounds
#define MANY_CASE(NT_)                                                                                                  \
  if (nt == NT_ && M <= 64)                                                                                             \
    return M <= 32 ? launch_ring<NT_, 2, 2, 4, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream)      \
                   : launch_ring<NT_, 4, 2, 4, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
  MANY_CASE(8)
  MANY_CASE(10)
  MANY_CASE(12)
  MANY_CASE(14)
#undef MANY_CASE
  if (nt == 8 && M > 64) return launch_ring<8, 8, 2, 4, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
  if (nt == 10 && M > 64) return launch_ring<10, 8, 2, 4, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
  return ERR_BAD_ARGUMENT;
}

// As llmserve_gemm_skinny, for M <= 128 and K / splits a multiple of 128, through gemm_ring with `nt` tiles of
// 16 weight rows a workgroup: 2, 4 or 6 (up to 64 rows), 5 (more than 32 rows), 8 or 10, or 12 or 14 (up to 64 rows).
extern "C" int llmserve_gemm_ring(const void* x, const void* w, const void* bias, int bias_is_float, void* out,
                                  int out_is_float, int gated, int M, int N, int K, int splits, int nt,
                                  hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 128 || K <= 0 || splits < 1 || K % splits || (gated && N % 2)) return ERR_BAD_ARGUMENT;
  if (splits > 1 && (gated || !out_is_float)) return ERR_BAD_ARGUMENT;
  if (gated)
    return out_is_float ? pick_ring<float, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream, nt)
                        : pick_ring<bf16_t, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream, nt);
  return out_is_float ? pick_ring<float, false>(x, w, bias, bias_is_float, out, M, N, K, splits, stream, nt)
                      : pick_ring<bf16_t, false>(x, w, bias, bias_is_float, out, M, N, K, 1, stream, nt);
}

// ---------------------------------------------------------------------------- many rows
// gemm_tiled: the same product for any number of rows of x (prompt portions), a tiled product:
// a workgroup of four waves (2 x 2) computes a square tile of 64 * WT weight rows by 64 * WT rows
// of x; steps of 32 over K go through LDS (two buffers: the next step's 16-byte pieces are
// requested before the current step is multiplied); each wave owns WT x WT tiles of
// v_mfma_f32_32x32x16_bf16.  WT = 4 (256 x 256, 128 x 128 a wave) halves the LDS traffic per
// multiply of WT = 2 and is used when the product has enough such tiles to fill the chip.
// As in the kernels above the weights are the A operand, so a lane ends up with four consecutive
// weight rows n of one row m of x: bias, SiLU(gate) * up over interleaved rows, and the stores
// work the same way; K may be cut over workgroups (blockIdx.z) into partial sums.
typedef float f32x16 __attribute__((ext_vector_type(16)));
#define TILE_K 32
#define TILE_STRIDE (TILE_K + 8)  // bf16 elements per staged row: 64 bytes + 16 of padding

// The end of a tiled product.  D[n][m] of a 32 x 32 tile: a lane holds column m = lane % 32 and rows
// n = 8 * (e / 4) + 4 * (lane / 32) + e % 4, so its values lie in 32 different rows of `out`.  They go
// through LDS (`mine`: 32 x (32 WT + 4) floats of this wave's own), 32 rows of x at a time, and leave as
// whole rows: 4 WT lanes write the 32 WT columns of a row, eight columns (16 bytes of bfloat16) a lane.
// n_wave, m_wave: where the wave's WT x WT tiles begin; `slice` the K split (its own copy of `out`).
template <int WT, typename TO, bool GATED>
__device__ __forceinline__ void store_tiles(const f32x16 (&acc)[WT][WT], float* mine, TO* __restrict__ out,
                                            const void* __restrict__ bias, int bias_is_float, int slice, int M, int N,
                                            int n_wave, int m_wave, int lane) {
  constexpr int ROW = 32 * WT + 4;           // floats of a transposed row, padded
  constexpr int LANES_A_ROW = 4 * WT, ROWS_A_PASS = 64 / LANES_A_ROW;
  const int r32 = lane & 31, half = lane >> 5;
  const int piece = lane % LANES_A_ROW, row_in_pass = lane / LANES_A_ROW;
  const int n_piece = n_wave + piece * 8;
  const bool with_bias = bias && slice == 0;
  float bias_here[8];
#pragma unroll
  for (int e = 0; e < 8; ++e)
    bias_here[e] = with_bias && n_piece + e < N ? load_as_float(bias, bias_is_float, n_piece + e) : 0.f;
#pragma unroll
  for (int j = 0; j < WT; ++j) {
#pragma unroll
    for (int i = 0; i < WT; ++i)
#pragma unroll
      for (int quad = 0; quad < 4; ++quad)
        *(f32x4*)(mine + (size_t)r32 * ROW + i * 32 + quad * 8 + half * 4) =
            (f32x4){acc[i][j][quad * 4], acc[i][j][quad * 4 + 1], acc[i][j][quad * 4 + 2], acc[i][j][quad * 4 + 3]};
    // (a wave reads only what it wrote itself: no barrier, the LDS operations of a wave complete in order)
#pragma unroll
    for (int pass = 0; pass < 32 / ROWS_A_PASS; ++pass) {
      const int row = pass * ROWS_A_PASS + row_in_pass;
      const int m = m_wave + j * 32 + row;
      const f32x4 lo = *(const f32x4*)(mine + (size_t)row * ROW + piece * 8);
      const f32x4 hi = *(const f32x4*)(mine + (size_t)row * ROW + piece * 8 + 4);
      float value[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
      for (int e = 0; e < 8; ++e) value[e] += bias_here[e];
      if (m >= M) continue;
      if (GATED) {
        TO* dst = out + (size_t)m * (N / 2) + n_piece / 2;
        float gated[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          // a bfloat16 result takes the hardware's 2^x and 1/x (a tile has 128 of these a lane; the
          // library routines are some forty instructions each and took most of a tile's way out)
          const float gate = value[2 * e], up = value[2 * e + 1];
          gated[e] = sizeof(TO) == 2 ? gate * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(gate * -1.44269504088896f)) * up
                                     : gate / (1.f + expf(-gate)) * up;
        }
        if (n_piece + 8 <= N && sizeof(TO) == 2 && (N / 2) % 4 == 0) {
          bf16_t packed[4] = {(bf16_t)gated[0], (bf16_t)gated[1], (bf16_t)gated[2], (bf16_t)gated[3]};
          *(uint2*)dst = *(const uint2*)packed;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n_piece + 2 * e + 1 < N) dst[e] = from_float<TO>(gated[e]);
        }
      } else {
        TO* dst = out + ((size_t)slice * M + m) * N + n_piece;
        if (n_piece + 8 <= N && N % 8 == 0) {
          if (sizeof(TO) == 2) {
            bf16_t packed[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) packed[e] = (bf16_t)value[e];
            *(uint4*)dst = *(const uint4*)packed;
          } else {
            *(f32x4*)dst = (f32x4){value[0], value[1], value[2], value[3]};
            *(f32x4*)((float*)dst + 4) = (f32x4){value[4], value[5], value[6], value[7]};
          }
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (n_piece + e < N) dst[e] = from_float<TO>(value[e]);
        }
      }
    }
  }
}

// Which tile a workgroup takes.  The chip hands workgroups to its eight chiplets (XCDs) in turn,
// workgroup i to chiplet i % 8, and every chiplet has an L2 of its own: tiles dealt out in launch
// order would make every chiplet read all of both operands.  So chiplet c takes a contiguous run
// of the tiles instead, counted through bands of eight tile rows of x, down the band first, then
// along the weight rows: what runs on a chiplet at one time is a few columns of one band, whose
// operand rows it fetches once and shares through its L2.
#define CHIPLETS 8
#define BAND 8
__device__ __forceinline__ void tile_of_workgroup(int index, int tiles_n, int tiles_m, int& tile_n, int& tile_m) {
  const int tiles = tiles_n * tiles_m;
  const int chiplet = index % CHIPLETS, turn = index / CHIPLETS;
  const int place = chiplet * (tiles / CHIPLETS) + min(chiplet, tiles % CHIPLETS) + turn;
  const int band = place / (BAND * tiles_n), within = place % (BAND * tiles_n);
  const int rows = min(BAND, tiles_m - band * BAND);
  tile_m = band * BAND + within % rows;
  tile_n = within / rows;
}

template <int WT, typename TO, bool GATED>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                         const void* __restrict__ bias, int bias_is_float,
                                                         TO* __restrict__ out, int M, int N, int K, int k_split) {
  constexpr int TILE = 64 * WT;          // rows of each operand in the workgroup's tile
  constexpr int PIECES = TILE * 4 / 256;  // 16-byte pieces of an operand's step each thread moves
  extern __shared__ __attribute__((aligned(16))) bf16_t staged[];  // [2 buffers][w, x][TILE][TILE_STRIDE]
  auto staged_w = [&](int buffer) { return staged + (size_t)(buffer * 2) * TILE * TILE_STRIDE; };
  auto staged_x = [&](int buffer) { return staged + (size_t)(buffer * 2 + 1) * TILE * TILE_STRIDE; };
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wave_n = wave & 1, wave_m = wave >> 1;
  int tile_n, tile_m;
  tile_of_workgroup(blockIdx.x, (N + TILE - 1) / TILE, (M + TILE - 1) / TILE, tile_n, tile_m);
  const int n0 = tile_n * TILE, m0 = tile_m * TILE;
  const int k_first = blockIdx.z * k_split;
  const int r32 = lane & 31, half = lane >> 5;

  const bf16_t* w_src[PIECES];
  const bf16_t* x_src[PIECES];
  bool w_live[PIECES], x_live[PIECES];
#pragma unroll
  for (int i = 0; i < PIECES; ++i) {
    const int piece = threadIdx.x + i * 256, row = piece >> 2, part = piece & 3;
    w_live[i] = n0 + row < N;
    x_live[i] = m0 + row < M;
    w_src[i] = w + (size_t)min(n0 + row, N - 1) * K + k_first + part * 8;
    x_src[i] = x + (size_t)min(m0 + row, M - 1) * K + k_first + part * 8;
  }
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8 w_piece[PIECES], x_piece[PIECES];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      w_piece[i] = w_live[i] ? load8(w_src[i] + k0) : zero;
      x_piece[i] = x_live[i] ? load8(x_src[i] + k0) : zero;
    }
  };
  auto stage = [&](int buffer) {
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      const int piece = threadIdx.x + i * 256, row = piece >> 2, part = piece & 3;
      *(bf16x8*)(staged_w(buffer) + row * TILE_STRIDE + part * 8) = w_piece[i];
      *(bf16x8*)(staged_x(buffer) + row * TILE_STRIDE + part * 8) = x_piece[i];
    }
  };

  f32x16 acc[WT][WT];  // [tile of weight rows][tile of x rows]
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int steps = k_split / TILE_K;
  fetch(0);
  stage(0);
  for (int step = 0; step < steps; ++step) {
    const int buffer = step & 1;
    __syncthreads();
    if (step + 1 < steps) fetch((step + 1) * TILE_K);
    const bf16_t* from_w = staged_w(buffer) + (size_t)(wave_n * 32 * WT + r32) * TILE_STRIDE + half * 8;
    const bf16_t* from_x = staged_x(buffer) + (size_t)(wave_m * 32 * WT + r32) * TILE_STRIDE + half * 8;
#pragma unroll
    for (int kk = 0; kk < TILE_K / 16; ++kk) {
      bf16x8 a[WT], b[WT];
#pragma unroll
      for (int i = 0; i < WT; ++i) {
        a[i] = *(const bf16x8*)(from_w + (size_t)i * 32 * TILE_STRIDE + kk * 16);
        b[i] = *(const bf16x8*)(from_x + (size_t)i * 32 * TILE_STRIDE + kk * 16);
      }
#pragma unroll
      for (int i = 0; i < WT; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (step + 1 < steps) stage(buffer ^ 1);  // read last in step - 1: everyone has passed this step's barrier since
  }

  __syncthreads();  // every wave has read the last stage: LDS is free for the way out
  store_tiles<WT, TO, GATED>(acc, (float*)staged + (size_t)wave * 32 * (32 * WT + 4), out, bias, bias_is_float,
                             blockIdx.z, M, N, n0 + wave_n * 32 * WT, m0 + wave_m * 32 * WT, lane);
}

template <int WT, typename TO, bool GATED>
static int launch_tiled(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int M, int N,
                        int K, int splits, hipStream_t stream) {
  constexpr int TILE = 64 * WT;
  const size_t stages = (size_t)4 * TILE * TILE_STRIDE * sizeof(bf16_t);
  const size_t way_out = (size_t)4 * 32 * (32 * WT + 4) * sizeof(float);  // store_tiles' rows of the four waves
  const size_t lds = stages > way_out ? stages : way_out;
  if (lds > 64 * 1024) {
    static bool asked = false;
    if (!asked) {
      if (hipFuncSetAttribute((const void*)gemm_tiled_kernel<WT, TO, GATED>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return ERR_BAD_ARGUMENT;
      asked = true;
    }
  }
  hipLaunchKernelGGL((gemm_tiled_kernel<WT, TO, GATED>), dim3(((N + TILE - 1) / TILE) * ((M + TILE - 1) / TILE), 1, splits),
                     dim3(256), lds, stream, (const bf16_t*)x, (const bf16_t*)w, bias, bias_is_float, (TO*)out, M, N, K,
                     K / splits);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- many rows, wide tiles
// gemm_wide: the tiled product with a 256 x 256 tile and both operands brought from global memory
// straight into LDS (global_load_lds_dwordx4: a wave's 64 lanes fill 1 KB of LDS in lane order, no
// registers in between).  K goes in steps of 32 through four stages of 32 KB, so the loads of three
// steps are under way while one is multiplied: a load takes longer to come back than a step's
// products take, and with one wave a SIMD nobody else hides it.
// A staged row is 64 bytes = 4 pieces of 16; piece p of row r lies in slot p ^ f(r), f mixing bits
// 1 to 3 of r, so that the lanes that read one piece of consecutive rows for an MFMA operand hit
// different banks, while the writes stay in lane order.
// Each of the four waves (2 x 2) owns 4 x 4 tiles of v_mfma_f32_32x32x16_bf16: 256 accumulators.
// The reads of LDS are written as instructions, with their waits: left to the compiler, every read
// of LDS waits for all loads into LDS that are under way, whichever stage they fill.
// One barrier a step, between its two halves: after it the next step's stage has landed for all
// waves, and all waves have read the previous one, which the step after next may be written over.
#define WIDE_TILE 256
#define WIDE_K 32
#define WIDE_STAGES 4
#define WIDE_OPERAND_BYTES (WIDE_TILE * WIDE_K * 2)     // one staged operand: 16 KB
#define WIDE_STAGE_BYTES (2 * WIDE_OPERAND_BYTES)        // w, then x

__device__ __forceinline__ int wide_swizzle(int row) { return (((row >> 1) ^ (row >> 3)) & 1) | (((row >> 2) & 1) << 1); }

// The wave's share of one operand's step: pieces (wave * 4 + i) * 64 + lane of 1024, four instructions.
__device__ __forceinline__ void wide_stage(const bf16_t* const (&src)[4], int k_offset, bf16_t* staged_operand, int wave) {
#pragma unroll
  for (int i = 0; i < 4; ++i)
    __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(src[i] + k_offset),
                                     (void __attribute__((address_space(3)))*)(staged_operand + (size_t)(wave * 4 + i) * 512),
                                     16, 0, 0);
}

// Loads into LDS that may still be under way: `stages` of them (8 instructions each), no more.
__device__ __forceinline__ void wide_wait_loads(int stages) {
  if (stages >= 2) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  else if (stages == 1) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// One 16-byte read of LDS for an MFMA operand: row tile I of the wave's four (32 rows = 2048 bytes
// apart) at `at`.  The eight reads of a half step (w and x tiles in turn) are dealt out between its
// products rather than put in front of them: a read that finds LDS busy holds up the wave, which
// is the only one on its SIMD, and should do so while a product runs.
template <int I>
__device__ __forceinline__ void wide_read(bf16x8& operand, unsigned at) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(operand) : "v"(at), "n"(I * 2048) : "memory");
}
// The reads come back in the order they were asked for.  The operands pass through the statement
// so that nothing that uses them is moved in front of it.
#define WIDE_ARRIVED(a, b)                                                                                     \
  asm volatile("s_waitcnt lgkmcnt(0)"                                                                          \
               : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]) \
               :: "memory")
// Two products of the current half step (tiles 2 P and 2 P + 1 of the sixteen, w tile = P / 2),
// then one read for the half step after it.
#define WIDE_PAIR(P, a_now, b_now, a_then, b_then, at_w, at_x)                                                      \
  acc[(P) / 2][((P) % 2) * 2] =                                                                                     \
      __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_now[(P) / 2], b_now[((P) % 2) * 2], acc[(P) / 2][((P) % 2) * 2], 0, 0, 0); \
  acc[(P) / 2][((P) % 2) * 2 + 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(                                        \
      a_now[(P) / 2], b_now[((P) % 2) * 2 + 1], acc[(P) / 2][((P) % 2) * 2 + 1], 0, 0, 0);                           \
  __builtin_amdgcn_sched_barrier(0);                                                                                \
  if ((P) % 2 == 0) wide_read<(P) / 2>(a_then[(P) / 2], at_w);                                                      \
  else wide_read<(P) / 2>(b_then[(P) / 2], at_x);                                                                   \
  __builtin_amdgcn_sched_barrier(0)

template <typename TO, bool GATED>
__global__ __launch_bounds__(256) void gemm_wide_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                        const void* __restrict__ bias, int bias_is_float,
                                                        TO* __restrict__ out, int M, int N, int K, int k_split) {
  extern __shared__ __attribute__((aligned(16))) bf16_t staged[];  // [4 stages][w, x][256 rows][32]
  constexpr int STAGE = WIDE_STAGE_BYTES / 2, OPERAND = WIDE_OPERAND_BYTES / 2;  // in elements
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int wave_n = wave & 1, wave_m = wave >> 1;
  int tile_n, tile_m;
  tile_of_workgroup(blockIdx.x, (N + WIDE_TILE - 1) / WIDE_TILE, (M + WIDE_TILE - 1) / WIDE_TILE, tile_n, tile_m);
  const int n0 = tile_n * WIDE_TILE, m0 = tile_m * WIDE_TILE;
  const int k_first = blockIdx.z * k_split;
  const int r32 = lane & 31, half = lane >> 5;

  // where this lane's pieces of a step come from: piece -> (row, slot), the slot holds part slot ^ f(row)
  const bf16_t* w_src[4];
  const bf16_t* x_src[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int piece = (wave * 4 + i) * 64 + lane;
    const int row = piece >> 2, part = (piece & 3) ^ wide_swizzle(row);
    w_src[i] = w + (size_t)min(n0 + row, N - 1) * K + k_first + part * 8;
    x_src[i] = x + (size_t)min(m0 + row, M - 1) * K + k_first + part * 8;
  }
  auto load_stage = [&](int step) {
    bf16_t* to = staged + (size_t)(step % WIDE_STAGES) * STAGE;
    wide_stage(w_src, step * WIDE_K, to, wave);
    wide_stage(x_src, step * WIDE_K, to + OPERAND, wave);
  };
  // where this lane reads its operands: rows r32 + 32 i of the wave's 128, part 2 * kk + half
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) bf16_t*)staged;
  const int swizzle = wide_swizzle(r32);
  const unsigned row_w = lds_base + (unsigned)(wave_n * 128 + r32) * (WIDE_K * 2);
  const unsigned row_x = lds_base + WIDE_OPERAND_BYTES + (unsigned)(wave_m * 128 + r32) * (WIDE_K * 2);
  const unsigned slot0 = (unsigned)((half ^ swizzle) * 16), slot1 = (unsigned)(((2 + half) ^ swizzle) * 16);

  f32x16 acc[4][4];  // [tile of weight rows][tile of x rows]
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int steps = k_split / WIDE_K;
  const int last = steps - 1;
#pragma unroll
  for (int step = 0; step < WIDE_STAGES - 1; ++step)
    if (step < steps) load_stage(step);
  wide_wait_loads(min(last, WIDE_STAGES - 2));  // stage 0 has landed
  __builtin_amdgcn_s_barrier();
  bf16x8 a0[4], b0[4], a1[4], b1[4];
  wide_read<0>(a0[0], row_w + slot0);
  wide_read<0>(b0[0], row_x + slot0);
  wide_read<1>(a0[1], row_w + slot0);
  wide_read<1>(b0[1], row_x + slot0);
  wide_read<2>(a0[2], row_w + slot0);
  wide_read<2>(b0[2], row_x + slot0);
  wide_read<3>(a0[3], row_w + slot0);
  wide_read<3>(b0[3], row_x + slot0);
  // A step with the loads of the step three ahead dealt out between its products (LOADS), or, for
  // the last three steps, without: two bodies, so that neither has a branch inside.
  auto one_step = [&](int step, auto with_loads) {
    constexpr bool LOADS = decltype(with_loads)::value;
    const unsigned stage_now = (unsigned)(step % WIDE_STAGES) * WIDE_STAGE_BYTES;
    const unsigned stage_next = (unsigned)((step + 1) % WIDE_STAGES) * WIDE_STAGE_BYTES;
    // the stage read in step - 1 is free: every wave finished with it before the barrier of that step
    bf16_t* to = staged + (size_t)((step + WIDE_STAGES - 1) % WIDE_STAGES) * STAGE;
    const int k_then = (step + WIDE_STAGES - 1) * WIDE_K;
    auto load_piece = [&](int i) {  // one of the wave's eight loads of the step three ahead
      if (!LOADS) return;
      const bf16_t* from = i < 4 ? w_src[i] : x_src[i - 4];
      __builtin_amdgcn_global_load_lds(
          (const void __attribute__((address_space(1)))*)(from + k_then),
          (void __attribute__((address_space(3)))*)(to + (i < 4 ? 0 : OPERAND) + (size_t)(wave * 4 + i % 4) * 512), 16,
          0, 0);
      __builtin_amdgcn_sched_barrier(0);
    };
    const unsigned at_w1 = row_w + stage_now + slot1, at_x1 = row_x + stage_now + slot1;
    WIDE_ARRIVED(a0, b0);
    WIDE_PAIR(0, a0, b0, a1, b1, at_w1, at_x1); load_piece(0);
    WIDE_PAIR(1, a0, b0, a1, b1, at_w1, at_x1); load_piece(1);
    WIDE_PAIR(2, a0, b0, a1, b1, at_w1, at_x1); load_piece(2);
    WIDE_PAIR(3, a0, b0, a1, b1, at_w1, at_x1); load_piece(3);
    WIDE_PAIR(4, a0, b0, a1, b1, at_w1, at_x1); load_piece(4);
    WIDE_PAIR(5, a0, b0, a1, b1, at_w1, at_x1); load_piece(5);
    WIDE_PAIR(6, a0, b0, a1, b1, at_w1, at_x1); load_piece(6);
    WIDE_PAIR(7, a0, b0, a1, b1, at_w1, at_x1); load_piece(7);
    WIDE_ARRIVED(a1, b1);  // and this wave no longer reads the current stage
    // stages up to min(step + 3, last) are on their way; step + 1 must have landed
    if (LOADS) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else wide_wait_loads(last - (step + 1));
    __builtin_amdgcn_s_barrier();
    const unsigned at_w0 = row_w + stage_next + slot0, at_x0 = row_x + stage_next + slot0;
    WIDE_PAIR(0, a1, b1, a0, b0, at_w0, at_x0);
    WIDE_PAIR(1, a1, b1, a0, b0, at_w0, at_x0);
    WIDE_PAIR(2, a1, b1, a0, b0, at_w0, at_x0);
    WIDE_PAIR(3, a1, b1, a0, b0, at_w0, at_x0);
    WIDE_PAIR(4, a1, b1, a0, b0, at_w0, at_x0);
    WIDE_PAIR(5, a1, b1, a0, b0, at_w0, at_x0);
    WIDE_PAIR(6, a1, b1, a0, b0, at_w0, at_x0);
    WIDE_PAIR(7, a1, b1, a0, b0, at_w0, at_x0);
  };
  // (after the last step the reads "for the next step" fetch a stage that holds nothing new: they
  // stay inside LDS and nobody uses them)
  int step = 0;
  for (; step + WIDE_STAGES - 1 < steps; ++step) one_step(step, std::true_type{});
  for (; step < steps; ++step) one_step(step, std::false_type{});
  WIDE_ARRIVED(a0, b0);
  __syncthreads();  // every wave has read the last stage: LDS is free for the way out
  store_tiles<4, TO, GATED>(acc, (float*)staged + (size_t)wave * 32 * (32 * 4 + 4), out, bias, bias_is_float,
                            blockIdx.z, M, N, n0 + wave_n * 128, m0 + wave_m * 128, lane);
}

template <typename TO, bool GATED>
static int launch_wide(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int M, int N,
                       int K, int splits, hipStream_t stream) {
  const size_t lds = (size_t)WIDE_STAGES * WIDE_STAGE_BYTES;  // 128 KB
  static bool asked = false;
  if (!asked) {
    if (hipFuncSetAttribute((const void*)gemm_wide_kernel<TO, GATED>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
      return ERR_BAD_ARGUMENT;
    asked = true;
  }
  hipLaunchKernelGGL((gemm_wide_kernel<TO, GATED>),
                     dim3(((N + WIDE_TILE - 1) / WIDE_TILE) * ((M + WIDE_TILE - 1) / WIDE_TILE), 1, splits), dim3(256), lds,
                     stream, (const bf16_t*)x, (const bf16_t*)w, bias, bias_is_float, (TO*)out, M, N, K, K / splits);
  return LAUNCH_STATUS();
}

template <typename TO, bool GATED>
static int pick_tiled(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int M, int N, int K,
                      int splits, hipStream_t stream) {
  // the wide tile when there are enough of them for most CUs (256) to get one
  const long wide_tiles = (long)((N + 255) / 256) * ((M + 255) / 256) * splits;
  if (wide_tiles >= 200 && (K / splits) % WIDE_K == 0)
    return launch_wide<TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
  return launch_tiled<2, TO, GATED>(x, w, bias, bias_is_float, out, M, N, K, splits, stream);
}

// x, w bfloat16; out bfloat16 or float32; any M and N, K a multiple of 32, an even N with `gated`.
// With splits > 1 (float32 out, not gated, K / splits a multiple of 32) `out` is [splits, M, N]
// partial sums, the bias in the first.
extern "C" int llmserve_gemm_tiled(const void* x, const void* w, const void* bias, int bias_is_float, void* out,
                                   int out_is_float, int gated, int M, int N, int K, int splits, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || K % TILE_K || (gated && N % 2) || splits < 1) return ERR_BAD_ARGUMENT;
  if (splits > 1 && (gated || !out_is_float || K % splits || (K / splits) % TILE_K)) return ERR_BAD_ARGUMENT;
  if (gated)
    return out_is_float ? pick_tiled<float, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream)
                        : pick_tiled<bf16_t, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream);
  return out_is_float ? pick_tiled<float, false>(x, w, bias, bias_is_float, out, M, N, K, splits, stream)
                      : pick_tiled<bf16_t, false>(x, w, bias, bias_is_float, out, M, N, K, 1, stream);
}

// x, w bfloat16; out bfloat16 or float32.  Needs 1 <= M <= 64, K a multiple of 32, and with
// `gated` an even N.  Any N.  With splits > 1 (float32 out, not gated, K / splits a multiple of
// 32) `out` is [splits, M, N]: slice s holds the sums over the s-th part of K (the bias in slice 0),
// and whoever reads it adds the slices in order.
extern "C" int llmserve_gemm_skinny(const void* x, const void* w, const void* bias, int bias_is_float, void* out,
                                    int out_is_float, int gated, int M, int N, int K, int splits,
                                    hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || K % STEP || (gated && N % 2) || splits < 1) return ERR_BAD_ARGUMENT;
  if (splits > 1 && (gated || !out_is_float || K % splits || (K / splits) % STEP)) return ERR_BAD_ARGUMENT;
  if (M <= 16 && (K / splits) % (STEP * GROUP) == 0) {
    // several weight tiles a wave where a wave has many groups of K to walk (or x is all 16 rows) and
    // enough workgroups are left (measured at the 1.5B and 7B sizes)
    const int per_wave = K / splits / (STEP * GROUP) / 4;
    const long tiles = (N + 15) / 16;
    const long by_four = (tiles + 3) / 4 * splits, by_two = (tiles + 1) / 2 * splits;  // workgroups
    const int share = (per_wave >= 8 && by_four >= 128 && (M > 2 || tiles <= 1024)) || (tiles >= 4096 && M >= 4) ? 4
                      : (per_wave >= 4 || M > 8 || (tiles >= 4096 && M >= 4)) && by_two * 4 >= TARGET_WAVES ? 2
                                                                                                            : 1;
    // Two tiles or one: through LDS (gemm_stream), unless many rows of x meet a long walk over K.
    if (share != 4 && !(share == 2 && M > 8 && per_wave >= 4)) {
      if (gated)
        return out_is_float ? pick_stream<float, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream)
                            : pick_stream<bf16_t, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream);
      return out_is_float ? pick_stream<float, false>(x, w, bias, bias_is_float, out, M, N, K, splits, stream)
                          : pick_stream<bf16_t, false>(x, w, bias, bias_is_float, out, M, N, K, 1, stream);
    }
#define PAIR_CASE(NT)                                                                                              \
  if (share == NT) {                                                                                               \
    if (gated)                                                                                                     \
      return out_is_float ? launch_pair<NT, float, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream)       \
                          : launch_pair<NT, bf16_t, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream);     \
    return out_is_float ? launch_pair<NT, float, false>(x, w, bias, bias_is_float, out, M, N, K, splits, stream)   \
                        : launch_pair<NT, bf16_t, false>(x, w, bias, bias_is_float, out, M, N, K, 1, stream);      \
  }
    PAIR_CASE(2)
    PAIR_CASE(4)
#undef PAIR_CASE
  }
  if (M > 16 && !gated && K % splits == 0 && (K / splits) % (STEP * GROUP) == 0 && (long)N * K <= (1L << 22)) {
    // A small weight at 17 to 64 rows: two or four tiles of x beside one weight tile a workgroup, through
    // LDS.  In a captured chain over different weights, the 1.5B sizes' qkv and o: 4.8 and 4.0 us at 17
    // rows, 5.0 and 4.5 at 32, 6.0 and 5.6 at 48, 6.7 and 6.2 at 64 (the library 7.1-7.7 throughout, the
    // kernel below 5.9 and 4.8 at 17 rows, 6.8 and 5.5 at 32).  Larger weights stay with the library.
    // With K cut in two (float32 partial sums) o takes 3.5 us at 17 rows, 3.7 at 32, 4.6 at 64 (the kernel
    // below, in three parts: 4.9, 5.6, 8.0).
    const int g = M <= 32 && splits == 1 ? 2 : 1;
    return out_is_float ? pick_stream<float, false>(x, w, bias, bias_is_float, out, M, N, K, splits, stream, 1, g)
                        : pick_stream<bf16_t, false>(x, w, bias, bias_is_float, out, M, N, K, 1, stream, 1, g);
  }
  if (gated)
    return out_is_float ? pick_waves<float, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream)
                        : pick_waves<bf16_t, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream);
  return out_is_float ? pick_waves<float, false>(x, w, bias, bias_is_float, out, M, N, K, splits, stream)
                      : pick_waves<bf16_t, false>(x, w, bias, bias_is_float, out, M, N, K, 1, stream);
}
