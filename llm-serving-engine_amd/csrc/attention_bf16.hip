// Paged grouped-query attention on the matrix cores, bfloat16 pages, float32 softmax.
// Compiled once per head size (-DHEAD_DIM=..., a multiple of 16).
//
// One kernel serves prompt portions and single decoded tokens.  The unit of work is a tile
// of up to 16 "columns": the (token, query head) pairs of a few consecutive tokens of one
// request that share one kv head.  A wave computes, for steps of 32 cached keys,
//   S^T[key][column] = K[key][:] . Q[column][:]          v_mfma_f32_16x16x32_bf16, A = K rows
//   P = exp(S * scale - running max), masked per column to the keys (p - window, p]
//   O^T[d][column] += V^T[d][key] * P^T[key][column]      A = rows of the transposed V page
// so each lane owns one column: its running maximum, its sum and four rows of every 16-row
// tile of O^T.  Value pages are stored transposed ([page, kv_head, dim, offset]) so that the
// keys, the contraction index of the second product, are contiguous for the A operand; the
// two 16-key halves of a step are interleaved in groups of four keys so that the layout S
// comes out in is already the layout P goes in with, without a shuffle.
// The four waves of a workgroup take the steps of the tile's key range in turn and merge
// their partial results through LDS; with `splits` > 1 several workgroups share a key range
// and a second kernel merges them (for few long requests).  A wave may carry several column
// tiles (COLUMN_TILES) through the same keys, which divides the cache traffic of a long
// prompt portion by as much.
// When every request of the step brings one token (FUSED), the kernel also does what comes
// before and after it in a decode step: it rotates the queries in registers, the workgroup
// that owns the newest key rotates that key and stores key and value in their page first.
#include "common.h"

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<multiple of 16>"
#endif
#if HEAD_DIM % 16 != 0 || HEAD_DIM < 16 || HEAD_DIM > 256
#error "HEAD_DIM must be a multiple of 16 between 16 and 256"
#endif

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int D = HEAD_DIM;
constexpr int D_TILES = D / 16;
constexpr bool WIDE = (D % 32 == 0);          // 32-wide MFMA steps over the head dimension
constexpr int QK_STEPS = WIDE ? D / 32 : D / 16;
constexpr int KEYS = 32;                      // keys per step

struct QkOperand {                            // one lane's share of a row for one MFMA step
#if HEAD_DIM % 32 == 0
  bf16x8 v;
#else
  s16x4 v;
#endif
};

__device__ __forceinline__ QkOperand load_qk(const bf16_t* row, int step, int q) {
  QkOperand r;
#if HEAD_DIM % 32 == 0
  r.v = *(const bf16x8*)(row + step * 32 + q * 8);
#else
  r.v = *(const s16x4*)(row + step * 16 + q * 4);
#endif
  return r;
}

__device__ __forceinline__ f32x4 mfma_qk(const QkOperand& a, const QkOperand& b, f32x4 c) {
#if HEAD_DIM % 32 == 0
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, c, 0, 0, 0);
#else
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, b.v, c, 0, 0, 0);
#endif
}

// work[tile] = {request index in the step, first token row, tokens in the tile, unused}
// pairing: 0 none, 1 adjacent pairs (2j, 2j+1), 2 half pairs (j, j + D/2)
__device__ __forceinline__ void rotate_pair(float& a, float& b, float2 cos_sin) {
  const float x = a * cos_sin.x - b * cos_sin.y, y = b * cos_sin.x + a * cos_sin.y;
  a = x;
  b = y;
}

struct FusedDecode {          // what the kernel needs to rotate and store; unused unless FUSED
  const float2* table;        // [rows][D / 2] (cos, sin) of each token's angles, or null
  int pairing;
  const int* slots;           // [rows] page * page_size + offset of each token, negative: store nothing
};

template <int COLUMN_TILES, bool FUSED, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void attention_tiles_kernel(
    const bf16_t* __restrict__ qkv, int row_width, bf16_t* __restrict__ out, float* __restrict__ partial_acc,
    float* __restrict__ partial_ml, bf16_t* __restrict__ keys,
    bf16_t* __restrict__ values, const int* __restrict__ block_tables, int table_width,
    const int* __restrict__ positions, const int* __restrict__ work, int heads, int kv_heads, int tokens_per_tile,
    int page_size, float scale, int window, int splits, FusedDecode fused) {
  extern __shared__ float lds[];  // [WAVES][16 columns][D + 2]
  const int group = heads / kv_heads;
  const int kv_head = blockIdx.y % kv_heads, head_tile = blockIdx.y / kv_heads;
  const int heads_here = min(group - head_tile * 16, 16);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, q = lane >> 4;
  // the work list runs from early to late tokens; late ones walk more keys, so they start first
  const int* item = work + (size_t)(gridDim.x - 1 - blockIdx.x) * 4;
  const int request = item[0], row0 = item[1], tokens = item[2];
  const int position0 = positions[row0];
  const int last_key = position0 + tokens - 1;
  const int first_key = window > 0 ? max(0, position0 - window + 1) : 0;
  const int* table = block_tables + (size_t)request * table_width;

  // this lane's column in each of its column tiles
  int column_position[COLUMN_TILES], column_first[COLUMN_TILES];
  bool column_live[COLUMN_TILES];
  QkOperand query[COLUMN_TILES][QK_STEPS];
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t) {
    const int token = t * tokens_per_tile + c / heads_here;
    column_live[t] = token < tokens && c / heads_here < tokens_per_tile;
    const int safe = min(token, tokens - 1);
    const int head = kv_head * group + head_tile * 16 + c % heads_here;
    column_position[t] = column_live[t] ? position0 + safe : -1;
    column_first[t] = window > 0 ? column_position[t] - window + 1 : 0;
    const bf16_t* q_row = qkv + (size_t)(row0 + safe) * row_width + (size_t)head * D;
#pragma unroll
    for (int s = 0; s < QK_STEPS; ++s) query[t][s] = load_qk(q_row, s, q);
#if HEAD_DIM % 32 == 0
    if (FUSED && fused.pairing != 0) {  // the queries come unrotated: rotate them here, in float32
      const float2* angles = fused.table + (size_t)(row0 + safe) * (D / 2);
      if (fused.pairing == 1) {
#pragma unroll
        for (int s = 0; s < QK_STEPS; ++s)
#pragma unroll
          for (int pair = 0; pair < 4; ++pair) {
            float a = (float)query[t][s].v[2 * pair], b = (float)query[t][s].v[2 * pair + 1];
            rotate_pair(a, b, angles[(s * 32 + q * 8) / 2 + pair]);
            query[t][s].v[2 * pair] = (bf16_t)a;
            query[t][s].v[2 * pair + 1] = (bf16_t)b;
          }
      } else {  // the partner of dim d is d + D/2: the same lane, QK_STEPS / 2 steps on (D % 64 == 0)
#pragma unroll
        for (int s = 0; s < QK_STEPS / 2; ++s)
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            float a = (float)query[t][s].v[i], b = (float)query[t][s + QK_STEPS / 2].v[i];
            rotate_pair(a, b, angles[s * 32 + q * 8 + i]);
            query[t][s].v[i] = (bf16_t)a;
            query[t][s + QK_STEPS / 2].v[i] = (bf16_t)b;
          }
      }
    }
#endif
  }

  float running_max[COLUMN_TILES], running_sum[COLUMN_TILES];
  f32x4 acc[COLUMN_TILES][D_TILES];
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t) {
    running_max[t] = -INFINITY;
    running_sum[t] = 0.f;
#pragma unroll
    for (int d = 0; d < D_TILES; ++d) acc[t][d] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

  const int step_first = first_key / KEYS, step_last = last_key / KEYS;
  const int per_split = (step_last - step_first + 1 + splits - 1) / splits;
  const int step_begin = step_first + blockIdx.z * per_split;
  const int step_end = min(step_last + 1, step_begin + per_split);
  const size_t page_stride = (size_t)kv_heads * page_size * D;
  const size_t head_offset = (size_t)kv_head * page_size * D;

  if (FUSED && step_last >= step_begin && step_last < step_end) {
    // this workgroup reads the newest key: it stores it first (one token per tile when FUSED; with
    // more than 16 query heads per kv head several workgroups store the same values)
    const int slot = fused.slots[row0];
    if (slot >= 0 && wave == 0) {
      const bf16_t* k_row = qkv + (size_t)row0 * row_width + (size_t)(heads + kv_head) * D;
      const bf16_t* v_row = k_row + (size_t)kv_heads * D;
      bf16_t* k_page = keys + (size_t)(slot / page_size) * page_stride + head_offset + (size_t)(slot % page_size) * D;
      bf16_t* v_page = values + (size_t)(slot / page_size) * page_stride + head_offset + slot % page_size;
      const float2* angles = fused.table + (size_t)row0 * (D / 2);
      for (int j = lane; j < D / 2; j += WAVE) {
        const int ia = fused.pairing == 2 ? j : 2 * j, ib = fused.pairing == 2 ? j + D / 2 : 2 * j + 1;
        float a = (float)k_row[ia], b = (float)k_row[ib];
        if (fused.pairing != 0) rotate_pair(a, b, angles[j]);
        k_page[ia] = (bf16_t)a;
        k_page[ib] = (bf16_t)b;
      }
      for (int d = lane; d < D; d += WAVE) v_page[(size_t)d * page_size] = v_row[d];
      __threadfence_block();  // read again below by this workgroup only
    }
    __syncthreads();
  }

  // One step's loads: the K rows of the two 16-key halves (lane (c, q) loads key c of each half,
  // its q-th slice of the row) and the V^T rows (lane (c, q) loads, for row d = 16 * tile + c, keys
  // 4q .. 4q+3 of each half).  Keys outside [first_key, last_key] are read from a key inside it
  // (their weights are zero), so no page is touched that the request does not hold.
  struct StepPages { int k_lo, k_hi, v_lo, v_hi; };
  struct StepLoads {
    QkOperand k_lo[QK_STEPS], k_hi[QK_STEPS];
    bf16x4 v_lo[D_TILES], v_hi[D_TILES];
  };
  const int low_limit = first_key & ~3, high_limit = last_key & ~3;
  auto key_of = [&](int step, int half) { return min(max(step * KEYS + 16 * half + c, first_key), last_key); };
  auto start_of = [&](int step, int half) { return min(max(step * KEYS + 16 * half + 4 * q, low_limit), high_limit); };
  auto pages_of = [&](int step) {
    return StepPages{table[key_of(step, 0) / page_size], table[key_of(step, 1) / page_size],
                     table[start_of(step, 0) / page_size], table[start_of(step, 1) / page_size]};
  };
  auto fetch = [&](int step, const StepPages& pages, StepLoads& L) {
    const bf16_t* row_lo = keys + (size_t)pages.k_lo * page_stride + head_offset + (size_t)(key_of(step, 0) % page_size) * D;
    const bf16_t* row_hi = keys + (size_t)pages.k_hi * page_stride + head_offset + (size_t)(key_of(step, 1) % page_size) * D;
#pragma unroll
    for (int s = 0; s < QK_STEPS; ++s) {
      L.k_lo[s] = load_qk(row_lo, s, q);
      L.k_hi[s] = load_qk(row_hi, s, q);
    }
    const bf16_t* base_lo = values + (size_t)pages.v_lo * page_stride + head_offset + start_of(step, 0) % page_size;
    const bf16_t* base_hi = values + (size_t)pages.v_hi * page_stride + head_offset + start_of(step, 1) % page_size;
#pragma unroll
    for (int d = 0; d < D_TILES; ++d) {
      L.v_lo[d] = *(const bf16x4*)(base_lo + (size_t)(d * 16 + c) * page_size);
      L.v_hi[d] = *(const bf16x4*)(base_hi + (size_t)(d * 16 + c) * page_size);
    }
  };
  auto compute = [&](int step, StepLoads& L) {
    const int key0 = step * KEYS;
    if (key0 + KEYS - 1 > last_key) {  // slots after the last key were never written: keep them out of 0 * x
      const int start_lo = start_of(step, 0), start_hi = start_of(step, 1);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool dead_lo = start_lo + i > last_key, dead_hi = start_hi + i > last_key;  // the slots really read
#pragma unroll
        for (int d = 0; d < D_TILES; ++d) {
          if (dead_lo) L.v_lo[d][i] = (bf16_t)0.f;
          if (dead_hi) L.v_hi[d][i] = (bf16_t)0.f;
        }
      }
    }
#pragma unroll
    for (int t = 0; t < COLUMN_TILES; ++t) {
      f32x4 s_lo = {0.f, 0.f, 0.f, 0.f}, s_hi = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < QK_STEPS; ++s) {
        s_lo = mfma_qk(L.k_lo[s], query[t][s], s_lo);
        s_hi = mfma_qk(L.k_hi[s], query[t][s], s_hi);
      }
      // lane holds, for its column, keys key0 + 4q + i (lo) and key0 + 16 + 4q + i (hi)
      float score[8];
      float tile_max = -INFINITY;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int key = key0 + (i < 4 ? 4 * q + i : 16 + 4 * q + (i - 4));
        const bool seen = key <= column_position[t] && key >= column_first[t];
        score[i] = seen ? (i < 4 ? s_lo[i] : s_hi[i - 4]) * scale : -INFINITY;
        tile_max = fmaxf(tile_max, score[i]);
      }
      tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, WAVE));
      tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, WAVE));
      const float next_max = fmaxf(running_max[t], tile_max);
      float correction = 1.f;
      bf16x8 weights;
      float added = 0.f;
      if (next_max == -INFINITY) {  // nothing seen yet by this column
#pragma unroll
        for (int i = 0; i < 8; ++i) weights[i] = (bf16_t)0.f;
      } else {
        correction = __expf(running_max[t] - next_max);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float p = __expf(score[i] - next_max);  // exp(-inf) = 0 for masked keys
          added += p;
          weights[i] = (bf16_t)p;
        }
      }
      running_sum[t] = running_sum[t] * correction + added;
      running_max[t] = next_max;
#pragma unroll
      for (int d = 0; d < D_TILES; ++d) {
        bf16x8 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[i] = L.v_lo[d][i];
          v[4 + i] = L.v_hi[d][i];
        }
        acc[t][d] *= correction;
        acc[t][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, weights, acc[t][d], 0, 0, 0);
      }
    }
  };

  // (Issuing a step's loads one step ahead was measured and does not pay: a step's arithmetic is
  // short beside the latency of its loads, which scatter over the pool's pages; what hides that
  // latency is many waves, each with a short walk.)
  for (int step = step_begin + wave; step < step_end; step += WAVES) {
    StepLoads loads;
    fetch(step, pages_of(step), loads);
    compute(step, loads);
  }

  // merge the waves, one column tile at a time: each wave leaves, per column, D sums, its
  // maximum and its sum of weights
  constexpr int STRIDE = D + 2;
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t) {
    float sum = running_sum[t];
    sum += __shfl_xor(sum, 16, WAVE);
    sum += __shfl_xor(sum, 32, WAVE);
    float* mine = lds + ((size_t)wave * 16 + c) * STRIDE;
#pragma unroll
    for (int d = 0; d < D_TILES; ++d)
#pragma unroll
      for (int i = 0; i < 4; ++i) mine[d * 16 + 4 * q + i] = acc[t][d][i];
    if (q == 0) {
      mine[D] = running_max[t];
      mine[D + 1] = sum;
    }
    __syncthreads();
    for (int index = threadIdx.x; index < 16 * (D / 4); index += WAVES * 64) {
      const int column = index / (D / 4), d4 = (index % (D / 4)) * 4;
      const int token = t * tokens_per_tile + column / heads_here;
      if (token >= tokens || column / heads_here >= tokens_per_tile) continue;
      float best = -INFINITY;
      for (int w = 0; w < WAVES; ++w) best = fmaxf(best, lds[((size_t)w * 16 + column) * STRIDE + D]);
      float total = 0.f;
      f32x4 merged = {0.f, 0.f, 0.f, 0.f};
      for (int w = 0; w < WAVES; ++w) {
        const float* theirs = lds + ((size_t)w * 16 + column) * STRIDE;
        const float factor = theirs[D] == -INFINITY ? 0.f : __expf(theirs[D] - best);
        total += theirs[D + 1] * factor;
#pragma unroll
        for (int i = 0; i < 4; ++i) merged[i] += theirs[d4 + i] * factor;
      }
      const int head = kv_head * group + head_tile * 16 + column % heads_here;
      const size_t row = (size_t)row0 + token;
      if (splits == 1) {
        bf16_t* dst = out + (row * heads + head) * D + d4;
        const float inverse = total > 0.f ? 1.f / total : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[i] = (bf16_t)(merged[i] * inverse);
      } else {
        const size_t slot = (row * heads + head) * splits + blockIdx.z;
        float* dst = partial_acc + slot * D + d4;
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[i] = merged[i];
        if (d4 == 0) {
          partial_ml[slot * 2] = best;
          partial_ml[slot * 2 + 1] = total;
        }
      }
    }
    __syncthreads();
  }
}

// Merges the key splits of one (token, head): out = sum_s acc_s * exp(m_s - m) / sum_s l_s *
// exp(m_s - m), in split order.  A second kernel rather than "the last workgroup merges": a
// workgroup that reads what others wrote needs the other chiplets' L2 written back first, and
// that costs more than this launch.
__global__ void attention_merge_kernel(const float* __restrict__ partial_acc, const float* __restrict__ partial_ml,
                                       bf16_t* __restrict__ out, int splits) {
  const size_t pair = blockIdx.x;  // row * heads + head
  const float* ml = partial_ml + pair * splits * 2;
  float best = -INFINITY;
  for (int s = 0; s < splits; ++s) best = fmaxf(best, ml[2 * s]);
  float total = 0.f;
  for (int s = 0; s < splits; ++s) total += ml[2 * s] == -INFINITY ? 0.f : ml[2 * s + 1] * __expf(ml[2 * s] - best);
  const float inverse = total > 0.f ? 1.f / total : 0.f;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float sum = 0.f;
    for (int s = 0; s < splits; ++s)
      if (ml[2 * s] != -INFINITY) sum += partial_acc[(pair * splits + s) * D + d] * __expf(ml[2 * s] - best);
    out[pair * D + d] = (bf16_t)(sum * inverse);
  }
}

template <int COLUMN_TILES, bool FUSED, int WAVES>
static int launch_tiles(const void* qkv, int row_width, void* out, float* partial_acc, float* partial_ml,
                        void* keys, void* values, const int* block_tables, int table_width,
                        const int* positions, const int* work, int tiles, int heads, int kv_heads,
                        int tokens_per_tile, int page_size, float scale, int window, int splits, FusedDecode fused,
                        hipStream_t stream) {
  const int group = heads / kv_heads;
  const int head_tiles = (group + 15) / 16;
  const size_t shared = (size_t)WAVES * 16 * (D + 2) * sizeof(float);
  if (shared > 64 * 1024) {  // more dynamic LDS than a kernel gets by default: ask for it once
    static bool asked = false;
    if (!asked) {
      if (hipFuncSetAttribute((const void*)attention_tiles_kernel<COLUMN_TILES, FUSED, WAVES>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)shared) != hipSuccess)
        return ERR_BAD_ARGUMENT;
      asked = true;
    }
  }
  hipLaunchKernelGGL((attention_tiles_kernel<COLUMN_TILES, FUSED, WAVES>), dim3(tiles, kv_heads * head_tiles, splits),
                     dim3(WAVES * 64), shared, stream, (const bf16_t*)qkv, row_width, (bf16_t*)out, partial_acc,
                     partial_ml, (bf16_t*)keys, (bf16_t*)values, block_tables, table_width, positions, work,
                     heads, kv_heads, tokens_per_tile, page_size, scale, window, splits, fused);
  return LAUNCH_STATUS();
}

extern "C" int llmserve_attention_head_dim() { return D; }


// Whether the fused decode form can rotate with this pairing at this head size.
extern "C" int llmserve_attention_can_fuse(int pairing) {
  if (pairing == 0) return 1;
  if (D % 32 != 0) return 0;
  return pairing == 1 || (pairing == 2 && D % 64 == 0);
}

// `work` holds `tiles` items of four ints; a tile covers `column_tiles * tokens_per_tile`
// tokens at most, where tokens_per_tile = max(1, 16 / (heads / kv_heads)).  page_size must
// be a multiple of 4.  With splits > 1, partial_acc is float32 [rows * heads * splits * D],
// partial_ml [rows * heads * splits * 2] (rows being the step's token count), and every row
// of the step must lie in one of the tiles: a second kernel merges the splits of all rows.
// With `fuse` every tile holds one token, qkv is as the projection left it, and the kernel
// rotates (table of cos and sin per row, pairing) and stores the token's key and value at slots[row] itself.
extern "C" int llmserve_attention_tiles(const void* qkv, int row_width, void* out, float* partial_acc,
                                        float* partial_ml, void* keys, void* values,
                                        const int* block_tables, int table_width, const int* positions,
                                        const int* work, int tiles, int column_tiles, int rows, int heads,
                                        int kv_heads, int page_size, float scale, int window, int splits, int fuse,
                                        const float* table, int pairing, const int* slots,
                                        hipStream_t stream) {
  if (tiles <= 0) return 0;
  if (heads % kv_heads || page_size % 4 || splits < 1 || (splits > 1 && (!partial_acc || !partial_ml)))
    return ERR_BAD_ARGUMENT;
  const int group = heads / kv_heads;
  const int tokens_per_tile = group >= 16 ? 1 : 16 / group;
  FusedDecode fused = {(const float2*)table, pairing, slots};
  int status;
  if (fuse) {
    if (column_tiles != 1 || !slots || !llmserve_attention_can_fuse(pairing) || (pairing != 0 && !table))
      return ERR_BAD_ARGUMENT;
    status = launch_tiles<1, true, 4>(qkv, row_width, out, partial_acc, partial_ml, keys, values, block_tables,
                                        table_width, positions, work, tiles, heads, kv_heads, tokens_per_tile,
                                        page_size, scale, window, splits, fused, stream);
  } else if (column_tiles == 1) {
    status = launch_tiles<1, false, 4>(qkv, row_width, out, partial_acc, partial_ml, keys, values, block_tables,
                                    table_width, positions, work, tiles, heads, kv_heads, tokens_per_tile, page_size,
                                    scale, window, splits, fused, stream);
  } else if (column_tiles == 4) {
    status = launch_tiles<4, false, 4>(qkv, row_width, out, partial_acc, partial_ml, keys, values, block_tables,
                                    table_width, positions, work, tiles, heads, kv_heads, tokens_per_tile, page_size,
                                    scale, window, splits, fused, stream);
  } else {
    return ERR_BAD_ARGUMENT;
  }
  if (status != 0 || splits == 1) return status;
  hipLaunchKernelGGL(attention_merge_kernel, dim3(rows * heads), dim3(64), 0, stream, partial_acc, partial_ml,
                     (bf16_t*)out, splits);
  return LAUNCH_STATUS();
}
