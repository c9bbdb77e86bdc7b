// Paged grouped-query attention in true float32 on the matrix cores (v_mfma_f32_16x16x4_f32 multiplies
// and adds float32 as they stand), float32 pages.  Compiled once per head size (-DHEAD_DIM=..., a
// multiple of 16).  It is the 32-bit path's attention for prompt portions and decoded tokens alike
// (reference model.py:140-175 computes the same recurrence page by page); attention_generic.hip
// remains for head sizes that are no multiple of 16 and pages that are no multiple of 4.
// Two things may change a score before the softmax, for position encodings and models that want them
// (the reference has neither): `soft_cap` > 0 squashes it to cap * tanh(score / cap), and `slopes` (one
// per query head) then adds -slope * (query position - key position).
//
// The unit of work is an item: up to 16 * COLUMN_TILES "columns", the (token, query head) pairs of
// consecutive tokens of one request that share one kv head, running through the tokens head by head so
// that a tile is full whatever the number of heads.  A workgroup takes an item and a kv head; its four
// waves take the steps of 16 cached keys in turn.  In a step a wave computes
//   S^T[key][column] = K[key][:] . Q[column][:]        A = K rows: lane (i, g) loads d = 16 s + 4 g .. + 3
//   P = exp2(S - the column's running maximum), masked per column to the keys (p - window, p]
//   O^T[d][column] += V^T[d][key] * P^T[key][column]    A = rows of the transposed V page
// A lane holds S for keys 4 g .. 4 g + 3 of column i, which is what the second product wants of P as
// its B operand, so nothing is exchanged between lanes but each column's maximum.  Every page is
// looked up once a step by the lane that reads it, and each step's keys and values pass through all
// the columns of the item, all query heads of the kv head among them.  The waves' results are merged
// through LDS in wave order; with `splits` > 1 several workgroups share an item's keys, leave
// (maximum, sum, unnormalised result) per column, and a second kernel merges them.
#include "common.h"

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<multiple of 16>"
#endif
#if HEAD_DIM % 16 != 0 || HEAD_DIM < 16 || HEAD_DIM > 256
#error "HEAD_DIM must be a multiple of 16 between 16 and 256"
#endif

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int D = HEAD_DIM;
constexpr int D_STEPS = D / 16;  // 16-wide steps over the head dimension, and 16-row tiles of O^T
constexpr int KEYS = 16;         // keys a step
constexpr int WAVES = 4;

__device__ __forceinline__ f32x4 load4(const float* p) { return *(const f32x4*)p; }

// work[item] = {request index in the step, first token row, first head of that token, columns}
// CHANGED: the scores carry a soft cap or a distance bias (a variant of its own, so that the plain one pays nothing)
template <int COLUMN_TILES, bool CHANGED>
__global__ __launch_bounds__(WAVES * 64) void attention_f32_kernel(
    const float* __restrict__ qkv, int row_width, float* __restrict__ out, float* __restrict__ partial_acc,
    float* __restrict__ partial_ml, const float* __restrict__ keys, const float* __restrict__ values,
    const int* __restrict__ block_tables, int table_width, const int* __restrict__ positions,
    const int* __restrict__ work, int heads, int kv_heads, int page_size, float scale_log2, int window, int splits,
    int columns_total, const float* __restrict__ slopes, float soft_cap) {
  __shared__ float wave_max[WAVES][COLUMN_TILES][16];
  __shared__ float wave_sum[WAVES][COLUMN_TILES][16];
  __shared__ __attribute__((aligned(16))) float merged[COLUMN_TILES][D_STEPS][64][4];
  const int* item = work + 4 * (gridDim.x - 1 - blockIdx.x);  // the list's last items walk the most keys: they start first
  const int request = item[0], first_row = item[1], first_head = item[2], columns = item[3];
  if (columns <= 0) return;  // an item that only pads a captured step's list
  const int kv_head = blockIdx.y, split = blockIdx.z;
  const int group = heads / kv_heads;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int i = lane & 15, g = lane >> 4;
  const int* table = block_tables + (size_t)request * table_width;

  // this lane's column in each tile: its token, head, and the keys it sees, [first, position]
  int position[COLUMN_TILES], first[COLUMN_TILES], token_row[COLUMN_TILES], head[COLUMN_TILES];
  [[maybe_unused]] float slope[COLUMN_TILES];  // of the column's head, in units of log2
  f32x4 query[COLUMN_TILES][D_STEPS];
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t) {
    const int c = t * 16 + i;
    const bool live = c < columns;
    const int flat = first_head + min(c, columns - 1);
    token_row[t] = first_row + flat / group;
    head[t] = kv_head * group + flat % group;
    position[t] = live ? positions[token_row[t]] : -1;
    first[t] = window > 0 ? max(0, position[t] - window + 1) : 0;
    if (CHANGED) slope[t] = slopes ? slopes[head[t]] * 1.4426950408889634f : 0.f;
    const float* q = qkv + (size_t)token_row[t] * row_width + head[t] * D + 4 * g;
#pragma unroll
    for (int s = 0; s < D_STEPS; ++s) {
      query[t][s] = load4(q + 16 * s);
#pragma unroll
      for (int e = 0; e < 4; ++e) query[t][s][e] *= scale_log2;
    }
  }
  // the item's keys: from the first that its first token sees to its last token's own
  const int last_flat = first_head + columns - 1;
  const int end = positions[first_row + last_flat / group] + 1;
  const int first_position = positions[first_row];
  const int begin = window > 0 ? max(0, first_position - window + 1) : 0;
  // steps of 16 keys, aligned to 16; the splits share them in contiguous runs, the waves take a run's in turn
  const int step_first = begin / KEYS, step_end = (end + KEYS - 1) / KEYS;
  const int per_split = (step_end - step_first + splits - 1) / splits;
  const int my_first = step_first + split * per_split, my_end = min(step_end, my_first + per_split);

  float running_max[COLUMN_TILES], running_sum[COLUMN_TILES];
  f32x4 acc[COLUMN_TILES][D_STEPS];
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t) {
    running_max[t] = -INFINITY;
    running_sum[t] = 0.f;
#pragma unroll
    for (int s = 0; s < D_STEPS; ++s) acc[t][s] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  const size_t page_elements = (size_t)page_size * D;
  const int piece_stride = page_size * KEY_PIECE;  // between the pieces of a key (common.h: key_element)

  // Which key a lane reads for the first product (key0 + i) and which four for the second (key0 + 4 g .. + 3, one
  // page: pages are multiples of 4).  A key outside the item's range is masked, and its page may have been given
  // back: the nearest inside is read instead.  The pages of a wave's next step are looked up a step ahead.
  auto key_of = [&](int step) { return max(min(step * KEYS + i, end - 1), begin); };
  auto value_key_of = [&](int step) { return max(min(step * KEYS + 4 * g, (end - 1) & ~3), begin & ~3); };
  int next_key_page = 0, next_value_page = 0;
  if (my_first + wave < my_end) {
    next_key_page = table[key_of(my_first + wave) / page_size];
    next_value_page = table[value_key_of(my_first + wave) / page_size];
  }
  for (int step = my_first + wave; step < my_end; step += WAVES) {
    const int key0 = step * KEYS;
    // K: lane (i, g) reads d = 16 s + 4 g .. + 3 of its key
    const int key_mine = key_of(step);
    const int key_page = next_key_page;
    const float* k_at = keys + ((size_t)key_page * kv_heads + kv_head) * page_elements +
                        (size_t)(key_mine % page_size) * KEY_PIECE + (g >> 1) * piece_stride + (g & 1) * 4;
    f32x4 k[D_STEPS];
#pragma unroll
    for (int s = 0; s < D_STEPS; ++s) k[s] = load4(k_at + (size_t)(2 * s) * piece_stride);
    // V^T: lane (i, g) reads its four keys of row d = 16 s + i
    const int value_key = value_key_of(step);
    const int value_page = next_value_page;
    if (step + WAVES < my_end) {
      next_key_page = table[key_of(step + WAVES) / page_size];
      next_value_page = table[value_key_of(step + WAVES) / page_size];
    }
    // (its four keys are half a piece of eight keys, or lie in the one piece of a page that is no multiple of eight)
    const float* v_at = values + ((size_t)value_page * kv_heads + kv_head) * page_elements +
                        value_element(i, value_key % page_size, page_size, D);
    const int value_width = value_piece_width(page_size);
    f32x4 v[D_STEPS];
#pragma unroll
    for (int s = 0; s < D_STEPS; ++s) v[s] = load4(v_at + (size_t)(16 * s) * value_width);

    f32x4 p[COLUMN_TILES];
#pragma unroll
    for (int t = 0; t < COLUMN_TILES; ++t) {
      f32x4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < D_STEPS; ++s)
#pragma unroll
        for (int e = 0; e < 4; ++e) s4 = __builtin_amdgcn_mfma_f32_16x16x4f32(k[s][e], query[t][s][e], s4, 0, 0, 0);
      // the lane holds column i, keys key0 + 4 g + e
      float best = -INFINITY;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int key = key0 + 4 * g + e;
        const bool seen = key <= position[t] && key >= first[t];
        if (CHANGED) {  // scores are kept in units of log2: the cap is applied to the score itself
          if (soft_cap > 0.f) s4[e] = soft_cap * 1.4426950408889634f * tanhf(s4[e] * 0.6931471805599453f / soft_cap);
          s4[e] -= slope[t] * (float)(position[t] - key);
        }
        s4[e] = seen ? s4[e] : -INFINITY;
        best = fmaxf(best, s4[e]);
      }
      best = fmaxf(best, __shfl_xor(best, 16, WAVE));
      best = fmaxf(best, __shfl_xor(best, 32, WAVE));
      const float next_max = fmaxf(running_max[t], best);
      // a column that has seen no key yet keeps its empty state (exp2(-inf - -inf) is no number)
      const float correction = next_max == -INFINITY ? 1.f : exp2f(running_max[t] - next_max);
      float added = 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        p[t][e] = s4[e] == -INFINITY ? 0.f : exp2f(s4[e] - next_max);
        added += p[t][e];
      }
      running_sum[t] = running_sum[t] * correction + added;  // this lane's keys only; the lanes of a column add up at the end
      running_max[t] = next_max;
#pragma unroll
      for (int s = 0; s < D_STEPS; ++s)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[t][s][e] *= correction;
    }
    // values of slots beyond the item's last key may be anything, also no number: they count as zero, and so
    // does what a lane read in place of keys outside the item's range
    const bool values_mine = value_key == key0 + 4 * g;
#pragma unroll
    for (int s = 0; s < D_STEPS; ++s)
#pragma unroll
      for (int e = 0; e < 4; ++e) v[s][e] = values_mine && value_key + e < end ? v[s][e] : 0.f;
#pragma unroll
    for (int t = 0; t < COLUMN_TILES; ++t)
#pragma unroll
      for (int s = 0; s < D_STEPS; ++s)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[t][s] = __builtin_amdgcn_mfma_f32_16x16x4f32(v[s][e], p[t][e], acc[t][s], 0, 0, 0);
  }

  // each column's sum over the four lanes that hold it
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t) {
    running_sum[t] += __shfl_xor(running_sum[t], 16, WAVE);
    running_sum[t] += __shfl_xor(running_sum[t], 32, WAVE);
    if (g == 0) {
      wave_max[wave][t][i] = running_max[t];
      wave_sum[wave][t][i] = running_sum[t];
    }
  }
  __syncthreads();
  float total_max[COLUMN_TILES], total_sum[COLUMN_TILES];
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t) {
    float best = -INFINITY;
    for (int w = 0; w < WAVES; ++w) best = fmaxf(best, wave_max[w][t][i]);
    float sum = 0.f;
    for (int w = 0; w < WAVES; ++w)
      sum += wave_max[w][t][i] == -INFINITY ? 0.f : wave_sum[w][t][i] * exp2f(wave_max[w][t][i] - best);
    total_max[t] = best;
    total_sum[t] = sum;
    const float mine = running_max[t] == -INFINITY ? 0.f : exp2f(running_max[t] - best);
#pragma unroll
    for (int s = 0; s < D_STEPS; ++s)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[t][s][e] *= mine;
  }
  // the waves add their results in wave order
  for (int w = 0; w < WAVES; ++w) {
    if (wave == w) {
#pragma unroll
      for (int t = 0; t < COLUMN_TILES; ++t)
#pragma unroll
        for (int s = 0; s < D_STEPS; ++s) {
          f32x4* at = (f32x4*)merged[t][s][lane];
          *at = w == 0 ? acc[t][s] : *at + acc[t][s];
        }
    }
    __syncthreads();
  }
  // O^T[d][column]: lane (i, g) holds column i and d = 16 s + 4 g .. + 3; wave w writes the tiles s = w, w + 4, ..
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t) {
    if (t * 16 + i >= columns) continue;
    const size_t column = (size_t)token_row[t] * heads + head[t];
    for (int s = wave; s < D_STEPS; s += WAVES) {
      f32x4 result = *(const f32x4*)merged[t][s][lane];
      if (splits == 1) {
        const float scale = total_sum[t] > 0.f ? 1.f / total_sum[t] : 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) result[e] *= scale;
        *(f32x4*)(out + column * D + 16 * s + 4 * g) = result;
      } else {
        *(f32x4*)(partial_acc + ((size_t)split * columns_total + column) * D + 16 * s + 4 * g) = result;
      }
    }
    if (splits > 1 && wave == 0 && g == 0) {
      float* ml = partial_ml + ((size_t)split * columns_total + column) * 2;
      ml[0] = total_max[t];
      ml[1] = total_sum[t];
    }
  }
}

// out[column][:] = sum_s acc_s 2^(m_s - m) / sum_s l_s 2^(m_s - m) over the splits of a column, m the largest m_s.
// A thread a dimension, at most 64 splits: in every wave lane s asks for split s's maximum and sum (one trip to memory
// for all of them; a loop over the splits made one after the other), the wave agrees on the largest and on the total,
// and every thread then adds up its dimension over the splits, in split order, asking for up to thirty-two of their
// partial sums at a time.
#define MERGE_SPLITS_MAX 64
constexpr int MERGE_THREADS = (D + 63) / 64 * 64;

template <int AT_ONCE>
__device__ __forceinline__ float merge_some(const float* acc, size_t split_stride, int first, int splits, float weight) {
  float part[AT_ONCE];
#pragma unroll
  for (int i = 0; i < AT_ONCE; ++i) part[i] = acc[(size_t)min(first + i, splits - 1) * split_stride];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < AT_ONCE; ++i) {
    const float w = __shfl(weight, min(first + i, MERGE_SPLITS_MAX - 1), 64);
    if (first + i < splits && w != 0.f) sum += part[i] * w;
  }
  return sum;
}

__global__ __launch_bounds__(MERGE_THREADS) void attention_f32_merge_kernel(float* __restrict__ out,
                                                                           const float* __restrict__ partial_acc,
                                                                           const float* __restrict__ partial_ml,
                                                                           int splits, int columns_total) {
  const size_t column = blockIdx.x;
  const int lane = threadIdx.x & 63, d = threadIdx.x;
  const float2 mine = lane < splits ? *(const float2*)(partial_ml + ((size_t)lane * columns_total + column) * 2)
                                    : make_float2(-INFINITY, 0.f);
  const float best = wave_max(mine.x);
  const float weight = mine.x == -INFINITY ? 0.f : exp2f(mine.x - best);  // a split that saw no key counts nothing
  const float total = wave_sum(mine.y * weight);                          // (lanes beyond the splits add 0)
  const float inverse = total > 0.f ? 1.f / total : 0.f;
  const float* acc = partial_acc + column * D + min(d, D - 1);
  const size_t split_stride = (size_t)columns_total * D;
  float sum = 0.f;
  int first = 0;
  for (; splits - first > 8; first += 32) sum += merge_some<32>(acc, split_stride, first, splits, weight);
  if (first < splits) sum += merge_some<8>(acc, split_stride, first, splits, weight);
  if (d < D) out[column * D + d] = sum * inverse;
}

// qkv [tokens, row_width] float32 with the queries in front (heads * D), out [tokens, heads * D]; key pages in
// pieces ([page, kv_head, D / 8, offset, 8]), value pages transposed in pieces of eight keys ([page, kv_head,
// page_size / 8, D, 8]; common.h: value_element); work [items, 4].
// column_tiles 1 or 2; page_size a multiple of 4; slopes float32 [heads] or null, soft_cap 0 for none.  With splits > 1: partial_acc float32 [splits, tokens * heads, D]
// and partial_ml [splits, tokens * heads, 2]; every column of the step must belong to an item.
extern "C" int llmserve_attention_f32(const float* qkv, int row_width, float* out, float* partial_acc, float* partial_ml,
                                      const float* keys, const float* values, const int* block_tables, int table_width,
                                      const int* positions, const int* work, int items, int column_tiles, int tokens,
                                      int heads, int kv_heads, int page_size, float scale, int window, int splits,
                                      const float* slopes, float soft_cap, hipStream_t stream) {
  if (items <= 0 || tokens <= 0) return 0;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || page_size <= 0 || page_size % 4 || splits < 1 ||
      splits > MERGE_SPLITS_MAX || (column_tiles != 1 && column_tiles != 2) || (splits > 1 && (!partial_acc || !partial_ml)))
    return ERR_BAD_ARGUMENT;
  const float scale_log2 = scale * 1.4426950408889634f;
  const int columns_total = tokens * heads;
  dim3 grid(items, kv_heads, splits);
  const bool changed = slopes != nullptr || soft_cap > 0.f;
#define LAUNCH_ATTENTION_F32(TILES, CHANGED)                                                                          \
  hipLaunchKernelGGL((attention_f32_kernel<TILES, CHANGED>), grid, dim3(WAVES * 64), 0, stream, qkv, row_width, out,   \
                     partial_acc, partial_ml, keys, values, block_tables, table_width, positions, work, heads,        \
                     kv_heads, page_size, scale_log2, window, splits, columns_total, slopes, soft_cap)
  if (column_tiles == 1 && !changed) LAUNCH_ATTENTION_F32(1, false);
  else if (column_tiles == 1) LAUNCH_ATTENTION_F32(1, true);
  else if (!changed) LAUNCH_ATTENTION_F32(2, false);
  else LAUNCH_ATTENTION_F32(2, true);
#undef LAUNCH_ATTENTION_F32
  int status = LAUNCH_STATUS();
  if (status != 0 || splits == 1) return status;
  hipLaunchKernelGGL(attention_f32_merge_kernel, dim3(columns_total), dim3(MERGE_THREADS), 0, stream, out, partial_acc, partial_ml,
                     splits, columns_total);
  return LAUNCH_STATUS();
}
