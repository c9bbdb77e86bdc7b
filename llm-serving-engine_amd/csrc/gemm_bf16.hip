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
    if (next < groups) {
#pragma unroll
      for (int u = 0; u < GROUP; ++u) a_next[u] = load8_stream(w_row + (next * GROUP + u) * STEP);
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      bf16x8 b[GROUP];
#pragma unroll
      for (int u = 0; u < GROUP; ++u) b[u] = x_live[t] ? load8(x_row[t] + (group * GROUP + u) * STEP) : zero;
#pragma unroll
      for (int u = 0; u < GROUP; ++u) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b[u], acc[t], 0, 0, 0);
    }
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
        for (int e = 0; e < 4; ++e) gated[e] = value[2 * e] / (1.f + expf(-value[2 * e])) * value[2 * e + 1];
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
  const int n0 = blockIdx.x * TILE, m0 = blockIdx.y * TILE;
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
  hipLaunchKernelGGL((gemm_tiled_kernel<WT, TO, GATED>), dim3((N + TILE - 1) / TILE, (M + TILE - 1) / TILE, splits),
                     dim3(256), lds, stream, (const bf16_t*)x, (const bf16_t*)w, bias, bias_is_float, (TO*)out, M, N, K,
                     K / splits);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- many rows, wide tiles
// gemm_wide: the tiled product with a 256 x 256 tile, steps of 64 over K, and both operands brought
// from global memory straight into LDS (global_load_lds_dwordx4: a wave's 64 lanes fill 1 KB of LDS
// in lane order, no registers in between), two stages: the next step's 64 KB are under way while
// the current step is multiplied.  A staged row is 128 bytes = 8 pieces of 16; piece p of row r lies
// in slot p ^ (r & 7), so that the eight lanes that read one piece of eight consecutive rows for an
// MFMA operand hit eight different slots (no bank conflict), while the writes stay in lane order.
// Each of the four waves (2 x 2) owns 4 x 4 tiles of v_mfma_f32_32x32x16_bf16: 256 accumulators.
#define WIDE_TILE 256
#define WIDE_K 64

__device__ __forceinline__ void wide_stage(const bf16_t* __restrict__ from, int rows_total, int row0, int ld, int k0,
                                           bf16_t* staged, int wave, int lane) {
  // 256 rows x 8 pieces = 2048 pieces of 16 bytes; wave w, instruction i fills pieces (w * 8 + i) * 64 + lane
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int piece = (wave * 8 + i) * 64 + lane;
    const int row = piece >> 3, slot = piece & 7;
    const int part = slot ^ (row & 7);
    const bf16_t* src = from + (size_t)min(row0 + row, rows_total - 1) * ld + k0 + part * 8;
    __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)src,
                                     (void __attribute__((address_space(3)))*)(staged + (size_t)(wave * 8 + i) * 512),
                                     16, 0, 0);
  }
}

template <typename TO, bool GATED>
__global__ __launch_bounds__(256) void gemm_wide_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                        const void* __restrict__ bias, int bias_is_float,
                                                        TO* __restrict__ out, int M, int N, int K, int k_split) {
  extern __shared__ __attribute__((aligned(16))) bf16_t staged[];  // [2 stages][w, x][256 rows][64]
  constexpr int OPERAND = WIDE_TILE * WIDE_K;  // elements of one staged operand
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int wave_n = wave & 1, wave_m = wave >> 1;
  const int n0 = blockIdx.x * WIDE_TILE, m0 = blockIdx.y * WIDE_TILE;
  const int k_first = blockIdx.z * k_split;
  const int r32 = lane & 31, half = lane >> 5;

  f32x16 acc[4][4];  // [tile of weight rows][tile of x rows]
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int steps = k_split / WIDE_K;
  wide_stage(w, N, n0, K, k_first, staged, wave, lane);
  wide_stage(x, M, m0, K, k_first, staged + OPERAND, wave, lane);
  for (int step = 0; step < steps; ++step) {
    bf16_t* now = staged + (size_t)(step & 1) * 2 * OPERAND;
    if (step + 1 < steps) {
      bf16_t* next = staged + (size_t)((step + 1) & 1) * 2 * OPERAND;
      wide_stage(w, N, n0, K, k_first + (step + 1) * WIDE_K, next, wave, lane);
      wide_stage(x, M, m0, K, k_first + (step + 1) * WIDE_K, next + OPERAND, wave, lane);
      __builtin_amdgcn_s_waitcnt(0x4F70);  // vmcnt(16): this step's pieces have landed, the next step's 16 may be out
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    }
    __syncthreads();
    const bf16_t* from_w = now + (size_t)(wave_n * 128 + r32) * WIDE_K;
    const bf16_t* from_x = now + OPERAND + (size_t)(wave_m * 128 + r32) * WIDE_K;
    // this lane's piece of a row in sub-step kk: part kk * 2 + half, in slot part ^ (row & 7); rows r32 + 32 i
    // keep r32 & 7.  The operands of sub-step kk + 1 are read from LDS while sub-step kk is multiplied.
    bf16x8 a[2][4], b[2][4];
    auto read_operands = [&](int kk, bf16x8 (&a_now)[4], bf16x8 (&b_now)[4]) {
      const int slot = ((kk * 2 + half) ^ (r32 & 7)) * 8;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a_now[i] = *(const bf16x8*)(from_w + (size_t)i * 32 * WIDE_K + slot);
        b_now[i] = *(const bf16x8*)(from_x + (size_t)i * 32 * WIDE_K + slot);
      }
    };
    read_operands(0, a[0], b[0]);
#pragma unroll
    for (int kk = 0; kk < WIDE_K / 16; ++kk) {
      if (kk + 1 < WIDE_K / 16) read_operands(kk + 1, a[(kk + 1) & 1], b[(kk + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);  // the reads stay in front of this sub-step's products: one wave a SIMD, nobody else hides their latency
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[kk & 1][i], b[kk & 1][j], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();  // everyone has read this stage: the step after next may be written over it
  }

  store_tiles<4, TO, GATED>(acc, (float*)staged + (size_t)wave * 32 * (32 * 4 + 4), out, bias, bias_is_float,
                            blockIdx.z, M, N, n0 + wave_n * 128, m0 + wave_m * 128, lane);
}

template <typename TO, bool GATED>
static int launch_wide(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int M, int N,
                       int K, int splits, hipStream_t stream) {
  const size_t lds = (size_t)2 * 2 * WIDE_TILE * WIDE_K * sizeof(bf16_t);  // 128 KB
  static bool asked = false;
  if (!asked) {
    if (hipFuncSetAttribute((const void*)gemm_wide_kernel<TO, GATED>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
      return ERR_BAD_ARGUMENT;
    asked = true;
  }
  hipLaunchKernelGGL((gemm_wide_kernel<TO, GATED>),
                     dim3((N + WIDE_TILE - 1) / WIDE_TILE, (M + WIDE_TILE - 1) / WIDE_TILE, splits), dim3(256), lds,
                     stream, (const bf16_t*)x, (const bf16_t*)w, bias, bias_is_float, (TO*)out, M, N, K, K / splits);
  return LAUNCH_STATUS();
}

// As llmserve_gemm_tiled, with K (and K / splits) a multiple of 64.
extern "C" int llmserve_gemm_wide(const void* x, const void* w, const void* bias, int bias_is_float, void* out,
                                  int out_is_float, int gated, int M, int N, int K, int splits, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || K % WIDE_K || (gated && N % 2) || splits < 1) return ERR_BAD_ARGUMENT;
  if (splits > 1 && (gated || !out_is_float || K % splits || (K / splits) % WIDE_K)) return ERR_BAD_ARGUMENT;
  if (gated)
    return out_is_float ? launch_wide<float, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream)
                        : launch_wide<bf16_t, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream);
  return out_is_float ? launch_wide<float, false>(x, w, bias, bias_is_float, out, M, N, K, splits, stream)
                      : launch_wide<bf16_t, false>(x, w, bias, bias_is_float, out, M, N, K, 1, stream);
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
  if (gated)
    return out_is_float ? pick_waves<float, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream)
                        : pick_waves<bf16_t, true>(x, w, bias, bias_is_float, out, M, N, K, 1, stream);
  return out_is_float ? pick_waves<float, false>(x, w, bias, bias_is_float, out, M, N, K, splits, stream)
                      : pick_waves<bf16_t, false>(x, w, bias, bias_is_float, out, M, N, K, 1, stream);
}
