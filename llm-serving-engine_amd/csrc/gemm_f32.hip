// float32 products on the matrix cores: out[M, N] = x[M, K] . w[N, K]^T (+ bias), every operand,
// product and sum in 32 bits (v_mfma_f32_16x16x4_f32 and v_mfma_f32_32x32x2_f32 multiply and add
// float32 as they stand; no reduced-precision matrix mode, no packed forms).  This is the true 32-bit
// path of every product in the model (the reference runs its float32 products through its BLAS,
// model.py:60-66 via nn.Linear); gemm_generic.hip remains for operands of mixed types and for a K
// that is no multiple of 4.
//
// gemm_f32_stream (M <= 64, decoding): the product is a stream of the weight matrix from HBM.  A
// workgroup owns 16 weight rows and its waves split K between them; lane (r, g) keeps groups of four
// 16-byte loads of weight row r in flight, k = 16 s + 4 g .. + 3 of every 16-wide step s.  An MFMA
// takes a 16 x 4 piece of the weights as its A operand (lane (r, g) gives A[r][g]) and 4 x 16 of x^T as
// B; which four k an instruction covers is free as long as A and B agree, so instruction j of a step
// takes element j of each lane's load: k = 16 s + 4 g + j.  The waves' partial tiles are added through
// LDS in wave order, so a row's bits depend on the shape of the weight only, never on the batch.
//
// gemm_f32_tiled (any M, prompt portions): 128 weight rows x 128 rows of x a workgroup, four waves as
// 2 x 2, each 2 x 2 tiles of v_mfma_f32_32x32x2_f32; K in steps of 16 through two LDS buffers, the next
// step's 16-byte pieces requested from global memory before the current step is multiplied.  A staged
// row is 16 floats padded to 20, so that the 16-byte reads of an operand spread over all banks.
//
// With `gated`, weight rows alternate gate_j, up_j and the epilogue writes silu(gate) * up (reference
// model.py:188) to out[M, N / 2].  With `splits` > 1, K is cut over workgroups and `out` is
// [splits, M, N] partial sums (bias in the first) that the reader adds in order.
#include "common.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define STREAM_GROUP 4  // 16-byte loads of a weight row a lane has in flight: 64 k

__device__ __forceinline__ f32x4 load4(const float* p) { return *(const f32x4*)p; }

__device__ __forceinline__ float silu(float gate) { return gate / (1.f + expf(-gate)); }

// MT: 16-row tiles of x (up to 16 MT rows): every weight operand meets MT operands of x, which each wave
// reads for itself (M / 16 of what it reads of the weights, from L2).
template <int WAVES, int MT, bool GATED>
__global__ __launch_bounds__(WAVES * 64) void gemm_f32_stream_kernel(const float* __restrict__ x,
                                                                     const float* __restrict__ w,
                                                                     const float* __restrict__ bias,
                                                                     float* __restrict__ out, int M, int N, int K,
                                                                     int k_split) {
  extern __shared__ float partial[];  // [WAVES][MT][64 lanes][4]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int n = min((int)blockIdx.x * 16 + r, N - 1);
  const int k_first = blockIdx.y * k_split;
  const int k_count = min(k_split, K - k_first);  // the last slice may be shorter
  const float* w_row = w + (size_t)n * K + k_first + g * 4;
  bool x_live[MT];
  const float* x_row[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    x_live[t] = t * 16 + r < M;
    x_row[t] = x + (size_t)min(t * 16 + r, M - 1) * K + k_first + g * 4;
  }
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = zero;

  const int groups = k_count / (16 * STREAM_GROUP);
  f32x4 a[STREAM_GROUP], a_next[STREAM_GROUP];
  int group = wave;
  if (group < groups) {
#pragma unroll
    for (int u = 0; u < STREAM_GROUP; ++u) a[u] = load4(w_row + (group * STREAM_GROUP + u) * 16);
  }
  while (group < groups) {
    const int next = group + WAVES;
    // this group's x is asked for before the next group's weights: loads come back in the order
    // they were asked for, and the products below wait for x
    f32x4 b[MT][STREAM_GROUP];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int u = 0; u < STREAM_GROUP; ++u) b[t][u] = x_live[t] ? load4(x_row[t] + (group * STREAM_GROUP + u) * 16) : zero;
    asm volatile("" ::: "memory");
    if (next < groups) {
#pragma unroll
      for (int u = 0; u < STREAM_GROUP; ++u) a_next[u] = load4(w_row + (next * STREAM_GROUP + u) * 16);
    }
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int u = 0; u < STREAM_GROUP; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u][j], b[t][u][j], acc[t], 0, 0, 0);
#pragma unroll
    for (int u = 0; u < STREAM_GROUP; ++u) a[u] = a_next[u];
    group = next;
  }
  // the steps left over when the slice is no multiple of 64; the last may be cut (K is a multiple of 4)
  for (int step = groups * STREAM_GROUP + wave; step * 16 < k_count; step += WAVES) {
    const bool inside = step * 16 + g * 4 < k_count;
    const f32x4 a_tail = inside ? load4(w_row + step * 16) : zero;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const f32x4 b_tail = inside && x_live[t] ? load4(x_row[t] + step * 16) : zero;
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_tail[j], b_tail[j], acc[t], 0, 0, 0);
    }
  }

#pragma unroll
  for (int t = 0; t < MT; ++t) *(f32x4*)(partial + ((wave * MT + t) * 64 + lane) * 4) = acc[t];
  __syncthreads();
  if (wave >= MT) return;
  // wave t finishes tile t of x.  D[n][m]: the lane holds token m = 16 t + r and rows n0 + 4 g .. + 3
  const int t = wave;
  f32x4 total = zero;
  for (int v = 0; v < WAVES; ++v) total += *(const f32x4*)(partial + ((v * MT + t) * 64 + lane) * 4);
  const int m = t * 16 + r;
  const int n_first = blockIdx.x * 16 + g * 4;
  if (m >= M) return;
  if (bias && blockIdx.y == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) total[i] += bias[min(n_first + i, N - 1)];
  }
  if (GATED) {
    float* dst = out + (size_t)m * (N / 2) + n_first / 2;
#pragma unroll
    for (int i = 0; i < 2; ++i)
      if (n_first + 2 * i + 1 < N) dst[i] = silu(total[2 * i]) * total[2 * i + 1];
  } else {
    float* dst = out + ((size_t)blockIdx.y * M + m) * N + n_first;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n_first + i < N) dst[i] = total[i];
  }
}

template <int WAVES, int MT, bool GATED>
static int launch_stream(const float* x, const float* w, const float* bias, float* out, int M, int N, int K, int splits,
                         int k_split, hipStream_t stream) {
  const size_t lds = (size_t)WAVES * MT * 64 * 4 * sizeof(float);
  hipLaunchKernelGGL((gemm_f32_stream_kernel<WAVES, MT, GATED>), dim3((N + 15) / 16, splits), dim3(WAVES * 64), lds,
                     stream, x, w, bias, out, M, N, K, k_split);
  return LAUNCH_STATUS();
}

template <int WAVES, bool GATED>
static int pick_tiles(const float* x, const float* w, const float* bias, float* out, int M, int N, int K, int splits,
                      int k_split, hipStream_t stream) {
  if (M <= 16) return launch_stream<WAVES, 1, GATED>(x, w, bias, out, M, N, K, splits, k_split, stream);
  if (M <= 32) return launch_stream<WAVES, 2, GATED>(x, w, bias, out, M, N, K, splits, k_split, stream);
  return launch_stream<WAVES, 4, GATED>(x, w, bias, out, M, N, K, splits, k_split, stream);
}

template <bool GATED>
static int pick_stream(const float* x, const float* w, const float* bias, float* out, int M, int N, int K, int splits,
                       hipStream_t stream) {
  // a slice of K is a multiple of 64 (whole groups) except the last
  const int k_split = splits == 1 ? K : ((K + splits - 1) / splits + 63) / 64 * 64;
  if ((size_t)k_split * (splits - 1) >= (size_t)K) return ERR_BAD_ARGUMENT;  // a slice would be empty
  // enough waves to cover the chip (about 2,048), but no more than there are groups of K
  const int tiles = (N + 15) / 16 * splits, groups = max(1, k_split / (16 * STREAM_GROUP));
  int waves = 4;
  while (waves < 16 && waves * tiles < 2048 && waves * 2 <= groups) waves *= 2;
  if (waves == 4) return pick_tiles<4, GATED>(x, w, bias, out, M, N, K, splits, k_split, stream);
  if (waves == 8) return pick_tiles<8, GATED>(x, w, bias, out, M, N, K, splits, k_split, stream);
  return pick_tiles<16, GATED>(x, w, bias, out, M, N, K, splits, k_split, stream);
}

// ---------------------------------------------------------------------------- many rows

#define TILE 128      // weight rows and rows of x a workgroup
#define TILE_K 16     // k a step
#define ROW_PAD 20    // floats a staged row takes: 16 and 4 of padding

// The tile (n, m) that a workgroup takes.  The chip hands workgroups to its eight chiplets in turn
// (workgroup i to chiplet i % 8), each with an L2 of its own: where the tiles divide by eight, chiplet c
// takes a contiguous run of them, counted down the rows of x first, so that what runs on a chiplet at
// one time shares its operands through that L2.
__device__ __forceinline__ int tile_of_workgroup(int id, int total) {
  return total % 8 == 0 ? (id % 8) * (total / 8) + id / 8 : id;
}

template <bool GATED>
__global__ __launch_bounds__(256) void gemm_f32_tiled_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                             const float* __restrict__ bias, float* __restrict__ out,
                                                             int M, int N, int K, int k_split, int tiles_m,
                                                             int tiles_n) {
  __shared__ __attribute__((aligned(16))) float ws[2][TILE * ROW_PAD];
  __shared__ __attribute__((aligned(16))) float xs[2][TILE * ROW_PAD];
  const int tile = tile_of_workgroup(blockIdx.x, tiles_m * tiles_n);
  const int tile_m = tile % tiles_m, tile_n = tile / tiles_m;
  const int n0 = tile_n * TILE, m0 = tile_m * TILE;
  const int k_first = blockIdx.y * k_split;
  const int k_end = min(K, k_first + k_split);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n_wave = (wave & 1) * 64, m_wave = (wave >> 1) * 64;
  const int i = lane & 31, half = lane >> 5;

  // what this thread brings of a step: piece `piece` (4 k) of rows `row` and `row + 64` of each operand
  const int row = threadIdx.x >> 2, piece = threadIdx.x & 3;
  const float* w_from[2];
  const float* x_from[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    w_from[h] = w + (size_t)min(n0 + row + 64 * h, N - 1) * K + piece * 4;
    x_from[h] = x + (size_t)min(m0 + row + 64 * h, M - 1) * K + piece * 4;
  }
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  f32x16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;

  f32x4 w_in[2], x_in[2];
  auto fetch = [&](int k0) {
    const bool inside = k0 + piece * 4 < k_end;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      w_in[h] = inside ? load4(w_from[h] + k0) : zero;
      x_in[h] = inside ? load4(x_from[h] + k0) : zero;
    }
  };
  auto stage = [&](int buffer) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      *(f32x4*)(ws[buffer] + (row + 64 * h) * ROW_PAD + piece * 4) = w_in[h];
      *(f32x4*)(xs[buffer] + (row + 64 * h) * ROW_PAD + piece * 4) = x_in[h];
    }
  };

  fetch(k_first);
  stage(0);
  __syncthreads();
  int buffer = 0;
  for (int k0 = k_first; k0 < k_end; k0 += TILE_K) {
    const bool more = k0 + TILE_K < k_end;
    if (more) fetch(k0 + TILE_K);
    // lane (i, half) holds k = 8 half .. + 7 of row i of each of its tiles; instruction s takes element s
    f32x4 a_low[2], a_high[2], b_low[2], b_high[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const float* a_at = ws[buffer] + (n_wave + 32 * t + i) * ROW_PAD + 8 * half;
      const float* b_at = xs[buffer] + (m_wave + 32 * t + i) * ROW_PAD + 8 * half;
      a_low[t] = *(const f32x4*)a_at;
      a_high[t] = *(const f32x4*)(a_at + 4);
      b_low[t] = *(const f32x4*)b_at;
      b_high[t] = *(const f32x4*)(b_at + 4);
    }
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_low[a][s], b_low[b][s], acc[a][b], 0, 0, 0);
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_high[a][s], b_high[b][s], acc[a][b], 0, 0, 0);
    if (more) stage(buffer ^ 1);
    __syncthreads();
    buffer ^= 1;
  }

  // D[n][m] of a 32 x 32 tile: the lane holds column m = i and rows n = 8 q + 4 half + e, q = 0 .. 3, e = 0 .. 3
  const bool with_bias = bias && blockIdx.y == 0;
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const int m = m0 + m_wave + 32 * b + i;
    if (m >= M) continue;
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + n_wave + 32 * a + 8 * q + 4 * half;
        if (n >= N) continue;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = acc[a][b][4 * q + e];
          if (with_bias) v[e] += bias[min(n + e, N - 1)];
        }
        if (GATED) {
          float* dst = out + (size_t)m * (N / 2) + n / 2;
          if (n + 1 < N) dst[0] = silu(v[0]) * v[1];
          if (n + 3 < N) dst[1] = silu(v[2]) * v[3];
        } else {
          float* dst = out + ((size_t)blockIdx.y * M + m) * N + n;
          if (n + 3 < N && (N & 3) == 0) {
            *(f32x4*)dst = (f32x4){v[0], v[1], v[2], v[3]};
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + e < N) dst[e] = v[e];
          }
        }
      }
    }
  }
}

template <bool GATED>
static int launch_tiled(const float* x, const float* w, const float* bias, float* out, int M, int N, int K, int splits,
                        hipStream_t stream) {
  const int k_split = splits == 1 ? K : ((K + splits - 1) / splits + TILE_K - 1) / TILE_K * TILE_K;
  if ((size_t)k_split * (splits - 1) >= (size_t)K) return ERR_BAD_ARGUMENT;
  const int tiles_m = (M + TILE - 1) / TILE, tiles_n = (N + TILE - 1) / TILE;
  hipLaunchKernelGGL((gemm_f32_tiled_kernel<GATED>), dim3(tiles_m * tiles_n, splits), dim3(256), 0, stream, x, w, bias,
                     out, M, N, K, k_split, tiles_m, tiles_n);
  return LAUNCH_STATUS();
}

// out [M, N] (or [splits, M, N] partial sums) = x [M, K] . w [N, K]^T (+ bias [N]); all float32, K a multiple
// of 4.  gated: w's rows alternate gate and up (N even), out is [M, N / 2] = silu(gate) * up, no splits.
// Up to 64 rows of x go to the weight-streaming kernel, more to the tiled one.
extern "C" int llmserve_gemm_f32(const float* x, const float* w, const float* bias, float* out, int gated, int M, int N,
                                 int K, int splits, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || K % 4 || splits < 1 || (gated && (splits != 1 || N % 2))) return ERR_BAD_ARGUMENT;
  if (M <= 64)
    return gated ? pick_stream<true>(x, w, bias, out, M, N, K, splits, stream)
                 : pick_stream<false>(x, w, bias, out, M, N, K, splits, stream);
  return gated ? launch_tiled<true>(x, w, bias, out, M, N, K, splits, stream)
               : launch_tiled<false>(x, w, bias, out, M, N, K, splits, stream);
}
