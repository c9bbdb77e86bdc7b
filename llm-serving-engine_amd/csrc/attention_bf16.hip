// Paged grouped-query attention on the matrix cores, bfloat16 pages, float32 softmax.
// Compiled once per head size (-DHEAD_DIM=..., a multiple of 16).
//
// One kernel serves prompt portions and single decoded tokens.  The unit of work is a tile
// of up to 16 "columns": the (token, query head) pairs of a few consecutive tokens of one
// request that share one kv head.  A wave computes, for steps of 32 cached keys,
//   S^T[key][column] = K[key][:] . Q[column][:]          v_mfma_f32_16x16x32_bf16, A = K rows
//   P = exp(S * scale - the column's reference maximum), masked per column to the keys (p - window, p]
//   O^T[d][column] += V^T[d][key] * P^T[key][column]      A = rows of the transposed V page
// so each lane owns one column: its running maximum, its sum and four rows of every 16-row
// tile of O^T.  Value pages are stored transposed, in pieces of eight keys ([page, kv_head, offset / 8,
// dim, 8]; common.h: value_element), so that the keys, the contraction index of the second product, are
// contiguous for the A operand and neighbouring lanes, which hold neighbouring rows, read neighbouring bytes; key pages
// are stored in pieces of eight elements, a piece of all the page's keys side by side ([page,
// kv_head, dim / 8, offset, 8]), so that neighbouring lanes, which hold the same piece of
// neighbouring keys, read neighbouring bytes (common.h: key_element); the
// keys of a step are dealt to the rows of the first product in groups of four so that the
// layout S comes out in is already the layout P goes in with, without a shuffle.
// The four waves of a workgroup take the steps of the tile's key range in turn and merge
// their partial results through LDS; with `splits` > 1 several workgroups share a key range
// and a second kernel merges them (for few long requests).  A wave may carry several column
// tiles (COLUMN_TILES) through the same keys, which divides the cache traffic of a long
// prompt portion by as much.
// When every request of the step brings one token (FUSED), the kernel also does what comes
// before and after it in a decode step: it rotates the queries in registers, the workgroup
// that owns the newest key rotates that key and stores key and value in their page first.
// CHANGED: a score is changed before the softmax, for encodings and models that want it (the
// reference has neither): `soft_cap` > 0 squashes it to cap * tanh(score / cap), and `slopes` (one
// per query head) then takes slope * (query position - key position) off it.
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
constexpr float RESCALE_STEP = 8.f;           // log2 units a column's maximum may run ahead of its reference

struct QkOperand {                            // one lane's share of a row for one MFMA step
#if HEAD_DIM % 32 == 0
  bf16x8 v;
#else
  s16x4 v;
#endif
};

// `key`: where the key's first piece lies in its page; the pieces are `piece_stride` elements apart
// (common.h: key_element; KEY_PIECE for a row that is in one piece, as a query's is).  A lane's share of MFMA step `step` is piece 4 step + q, or, with 16-wide
// steps, half q % 2 of piece 2 step + q / 2.
__device__ __forceinline__ QkOperand load_qk(const bf16_t* key, unsigned piece_stride, int step, int q) {
  QkOperand r;
#if HEAD_DIM % 32 == 0
  r.v = *(const bf16x8*)(key + (unsigned)(step * 4 + q) * piece_stride);
#else
  r.v = *(const s16x4*)(key + (unsigned)(step * 2 + (q >> 1)) * piece_stride + (q & 1) * 4);
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

// work[tile] = {request index in the step, first token row, first head, columns}: see ColumnMap
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
  int unmerged;               // key splits are left for the reader to merge: each split's result is divided by its own
                              // sum of weights and stored as bfloat16 where partial_acc points, [rows][heads][splits][D]
  int by_item;                // the splits' partial results are kept by work item (item * tokens_per_tile + token)
                              // instead of by the step's row: for the few short requests of a step of long portions
};

struct ScoreChange {          // unused unless CHANGED
  const float* slopes;        // [heads], or null
  float soft_cap;             // 0: none
};

// One step's operands as a lane holds them: its slices of the K rows of the two 16-row tiles and,
// for every 16-row tile of V^T, eight consecutive keys of its row.
struct StepLoads {
  QkOperand k_lo[QK_STEPS], k_hi[QK_STEPS];
  bf16x8 v[D_TILES];
};

// Which (token, query head) a column of a work item is.  With up to 16 query heads a kv head the
// columns run through the item's tokens head by head, beginning at `first_head` of its first token,
// so that every column tile is full whatever the number of heads; with more than 16 a workgroup
// takes 16 heads (or what is left) and a column tile is one token.
struct ColumnMap {
  int heads_here, first_head, columns;
  bool packed;
  // (a column's number is below 256 and there are at most 16 heads here: the quotient by a multiplication, exact for
  // numbers below 65,536 / heads_here; a division proper costs forty instructions, several times a workgroup)
  unsigned reciprocal = 65536u / (unsigned)heads_here + 1u;
  __device__ __forceinline__ int over_heads(int flat) const { return (int)(((unsigned)flat * reciprocal) >> 16); }
  __device__ __forceinline__ void of(int tile, int c, int& token, int& head, bool& live) const {
    if (packed) {
      const int flat = first_head + tile * 16 + c;
      token = over_heads(flat);
      head = flat - token * heads_here;
      live = tile * 16 + c < columns;
    } else {
      token = tile;
      head = min(c, heads_here - 1);
      live = tile < columns && c < heads_here;
    }
  }
  __device__ __forceinline__ int tokens() const { return packed ? over_heads(first_head + columns - 1) + 1 : columns; }
};

// What a lane keeps for its column in each of its column tiles.
template <int COLUMN_TILES>
struct Columns {
  int position[COLUMN_TILES], first[COLUMN_TILES];  // the keys the column sees: [first, position]
  QkOperand query[COLUMN_TILES][QK_STEPS];
  float slope[COLUMN_TILES];  // of the column's head, in units of log2 a key; set and read only where scores are changed
  float running_max[COLUMN_TILES], running_sum[COLUMN_TILES];
  f32x4 acc[COLUMN_TILES][D_TILES];
};

// First product of a step, for all column tiles: after it the K rows are no longer needed.
template <int COLUMN_TILES>
__device__ __forceinline__ void scores_of(const Columns<COLUMN_TILES>& columns, const StepLoads& L, f32x4* s_lo,
                                          f32x4* s_hi) {
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t) {
    s_lo[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    s_hi[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < QK_STEPS; ++s) {
      s_lo[t] = mfma_qk(L.k_lo[s], columns.query[t][s], s_lo[t]);
      s_hi[t] = mfma_qk(L.k_hi[s], columns.query[t][s], s_hi[t]);
    }
  }
}

// Softmax weights and second product of a step.  Scores are kept in units of log2 (scale * log2 e is
// folded into one multiply-add, weights are exp2 of differences to the column's reference).  The
// reference is the column's maximum at some earlier step; it moves only when a score exceeds it by
// more than RESCALE_STEP, so weights reach 2^RESCALE_STEP at most, the accumulators are rescaled
// rarely, and the common step needs no exchange between the four lanes of a column: each checks its
// own eight scores.  `interior`: every column of the wave sees all 32 keys of the step (no masks).
// `v_start`: the first of the eight keys this lane's V values were really read from; values of keys
// after `last_key` (slots never written) are kept out of 0 * x.
// CHANGED: `soft_cap` > 0 squashes a score to cap * tanh(score * scale / cap), as 1 - 2 / (1 + e^(2 score * scale / cap))
// (right at both ends: e^x = inf gives 1, 0 gives -1), and the column's slope times the key's distance comes off it.
template <int COLUMN_TILES, bool CHANGED = false>
__device__ __forceinline__ void weigh_and_add(Columns<COLUMN_TILES>& columns, StepLoads& L, const f32x4* s_lo,
                                              const f32x4* s_hi, int key0, int q, bool interior, int last_key,
                                              int v_start, float scale_log2, float soft_cap = 0.f) {
  bf16x8 weights[COLUMN_TILES];
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t) {
    // lane holds, for its column, keys key0 + 8q + i
    const bool unset = columns.running_max[t] == -INFINITY;  // nothing seen yet by this column
    const float reference = unset ? 0.f : columns.running_max[t];
    float x[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = fmaf(i < 4 ? s_lo[t][i] : s_hi[t][i - 4], scale_log2, -reference);
    if constexpr (CHANGED) {
      if (soft_cap > 0.f) {
        const float cap_log2 = soft_cap * 1.44269504088896f, doubled = 2.f * scale_log2 / soft_cap;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float e = __builtin_amdgcn_exp2f((i < 4 ? s_lo[t][i] : s_hi[t][i - 4]) * doubled);
          x[i] = fmaf(cap_log2, 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + e), -reference);
        }
      }
      const float distance = (float)(columns.position[t] - (key0 + 8 * q));  // of the lane's first key
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] -= columns.slope[t] * (distance - (float)i);
    }
    if (!interior) {
      // key0 + 8q + i outside [first, position], counted from the lane's first key (nothing to add per key)
      const int last_seen = columns.position[t] - (key0 + 8 * q), first_seen = columns.first[t] - (key0 + 8 * q);
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (i > last_seen || i < first_seen) x[i] = -INFINITY;
    }
    // (the largest of three in one instruction, written out: through fmaxf the compiler first passes every
    // score through a v_max with itself, thirteen instructions for eight scores where four do)
    float highest;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(highest) : "v"(x[0]), "v"(x[1]), "v"(x[2]));
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(highest) : "v"(highest), "v"(x[3]), "v"(x[4]));
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(highest) : "v"(highest), "v"(x[5]), "v"(x[6]));
    asm("v_max_f32 %0, %1, %2" : "=v"(highest) : "v"(highest), "v"(x[7]));
    if (__any(highest > (unset ? -INFINITY : RESCALE_STEP))) {
      float column_highest = fmaxf(highest, __shfl_xor(highest, 16, WAVE));
      column_highest = fmaxf(column_highest, __shfl_xor(column_highest, 32, WAVE));
      if (column_highest > (unset ? -INFINITY : RESCALE_STEP)) {  // the same answer in the four lanes of a column
        const float correction = unset ? 0.f : __builtin_amdgcn_exp2f(-column_highest);
        columns.running_max[t] = reference + column_highest;
        columns.running_sum[t] *= correction;
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] -= column_highest;
#pragma unroll
        for (int d = 0; d < D_TILES; ++d) columns.acc[t][d] *= correction;
      }
    }
    float added = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float p = __builtin_amdgcn_exp2f(x[i]);  // exp2(-inf) = 0 for keys the column does not see
      added += p;
      weights[t][i] = (bf16_t)p;
    }
    columns.running_sum[t] += added;
  }
  if (key0 + KEYS - 1 > last_key) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (v_start + i > last_key) {
#pragma unroll
        for (int d = 0; d < D_TILES; ++d) L.v[d][i] = (bf16_t)0.f;
      }
  }
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t)
#pragma unroll
    for (int d = 0; d < D_TILES; ++d)
      columns.acc[t][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(L.v[d], weights[t], columns.acc[t][d], 0, 0, 0);
}

template <int COLUMN_TILES, bool FUSED, int WAVES, bool CHANGED = false>
__global__ __launch_bounds__(WAVES * 64, (COLUMN_TILES > 2 || HEAD_DIM > 192 || WAVES > 4) ? 1 : 2) void attention_tiles_kernel(
    const bf16_t* __restrict__ qkv, int row_width, bf16_t* __restrict__ out, float* __restrict__ partial_acc,
    float* __restrict__ partial_ml, bf16_t* __restrict__ keys,
    bf16_t* __restrict__ values, const int* __restrict__ block_tables, int table_width,
    const int* __restrict__ positions, const int* __restrict__ work, int heads, int kv_heads, int tokens_per_tile,
    int page_size, int page_shift, float scale, int window, int splits, FusedDecode fused, ScoreChange change) {
  static_assert(!(FUSED && CHANGED), "the fused decode form takes plain scores only");
  extern __shared__ float lds[];  // [WAVES][16 columns][D + 4]
  if (FUSED)  // a short kernel: fetch all arguments in one go rather than each before its first use
    asm volatile("" ::"s"(row_width), "s"(table_width), "s"(heads), "s"(kv_heads), "s"(page_size), "s"(page_shift),
                 "s"(scale), "s"(window), "s"(splits), "s"(fused.pairing));
  const int group = heads / kv_heads;
  const int kv_head = blockIdx.y % kv_heads, head_tile = blockIdx.y / kv_heads;
  const int heads_here = min(group - head_tile * 16, 16);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // the same in all lanes: kept in a scalar register
  const int c = lane & 15, q = lane >> 4;
  // the work list runs from early to late tokens; late ones walk more keys, so they start first
  // (when FUSED every request brings one token: tile i is request i and row i, nothing to look up)
  const int* item = work + (size_t)(gridDim.x - 1 - blockIdx.x) * 4;
  // an item of no columns pads a work list to the length a captured step was recorded with: nothing to do
  if (!FUSED && item[3] <= 0) return;
  const int request = FUSED ? (int)blockIdx.x : item[0], row0 = FUSED ? (int)blockIdx.x : item[1];
  const ColumnMap map = {heads_here, FUSED ? 0 : item[2], FUSED ? (group <= 16 ? heads_here : 1) : item[3], group <= 16};
  const int tokens = map.tokens();
  const int position0 = positions[row0];
  const int* table = block_tables + (size_t)request * table_width;
  // FUSED: a step of single tokens is short, and what it takes is mostly the time its loads need to come
  // back.  So everything the start of the kernel needs is asked for here at once, before anything is
  // used: the pieces of the token's key and value row (one wave will store them; which one depends on the
  // position, so all ask), the angles, and the pages of this wave's first step, looked up as if that
  // step lay wholly inside the context (if it does not, they are looked up again below).
  constexpr int PAIR_PIECES = (D / 2 + WAVE - 1) / WAVE, VALUE_PIECES = (D + WAVE - 1) / WAVE;
  [[maybe_unused]] bf16_t new_a[PAIR_PIECES], new_b[PAIR_PIECES], new_v[VALUE_PIECES];
  [[maybe_unused]] float2 new_angle[PAIR_PIECES];
  [[maybe_unused]] int new_slot = -1;
  [[maybe_unused]] int early_k = -1, early_k_hi = -1, early_v = -1;
  const bool early_pages = FUSED && window <= 0 && splits == 1 && (wave * KEYS + KEYS - 1) / page_size < table_width;
  // (heads up to 128 wide leave the registers for a wave's second step to be asked for together with its first)
  constexpr bool TWO_STEPS = FUSED && HEAD_DIM <= 128;
  [[maybe_unused]] int second_k = -1, second_k_hi = -1, second_v = -1;
  const bool second_pages = TWO_STEPS && early_pages && ((wave + WAVES) * KEYS + KEYS - 1) / page_size < table_width;
  if (FUSED) {
    const bf16_t* k_row = qkv + (size_t)row0 * row_width + (size_t)(heads + kv_head) * D;
    const bf16_t* v_row = k_row + (size_t)kv_heads * D;
    // (the slot is the same for all lanes; asked for as if it were not, or the compiler waits for it right
    // here to move it into a scalar register)
    int no_offset;
    asm volatile("v_mov_b32 %0, 0" : "=v"(no_offset));
    new_slot = fused.slots[row0 + no_offset];
#pragma unroll
    for (int i = 0; i < PAIR_PIECES; ++i) {
      const int j = min(lane + i * WAVE, D / 2 - 1);
      new_a[i] = k_row[fused.pairing == 2 ? j : 2 * j];
      new_b[i] = k_row[fused.pairing == 2 ? j + D / 2 : 2 * j + 1];
      if (fused.pairing != 0) new_angle[i] = fused.table[(size_t)row0 * (D / 2) + j];
    }
#pragma unroll
    for (int i = 0; i < VALUE_PIECES; ++i) new_v[i] = v_row[min(lane + i * WAVE, D - 1)];
    if (early_pages) {
      const int key = wave * KEYS + 8 * (c >> 2) + (c & 3);
      early_k = table[key / page_size];
      early_k_hi = table[(key + 4) / page_size];
      early_v = table[(wave * KEYS + 8 * q) / page_size];
    }
    if (second_pages) {
      const int key = (wave + WAVES) * KEYS + 8 * (c >> 2) + (c & 3);
      second_k = table[key / page_size];
      second_k_hi = table[(key + 4) / page_size];
      second_v = table[((wave + WAVES) * KEYS + 8 * q) / page_size];
    }
  }
  const int last_key = position0 + tokens - 1;
  const int first_key = window > 0 ? max(0, position0 - window + 1) : 0;

  // this lane's column in each of its column tiles
  Columns<COLUMN_TILES> columns;
  bool column_live[COLUMN_TILES];
  auto& column_position = columns.position;
  auto& column_first = columns.first;
  auto& query = columns.query;
  auto& running_max = columns.running_max;
  auto& running_sum = columns.running_sum;
  auto& acc = columns.acc;
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t) {
    int token, head_here;
    map.of(t, c, token, head_here, column_live[t]);
    const int safe = min(token, tokens - 1);
    const int head = kv_head * group + head_tile * 16 + head_here;
    column_position[t] = column_live[t] ? position0 + safe : -1;
    column_first[t] = window > 0 ? column_position[t] - window + 1 : 0;
    if constexpr (CHANGED) columns.slope[t] = change.slopes ? change.slopes[head] * 1.44269504088896f : 0.f;
    const bf16_t* q_row = qkv + (size_t)(row0 + safe) * row_width + (size_t)head * D;
#pragma unroll
    for (int s = 0; s < QK_STEPS; ++s) query[t][s] = load_qk(q_row, KEY_PIECE, s, q);  // a query's row is in one piece
#if HEAD_DIM % 32 == 0
    if (FUSED && fused.pairing != 0) {  // the queries come unrotated: rotate them here, in float32
      const float2* angles = fused.table + (size_t)(row0 + safe) * (D / 2);
      // All angles are asked for before the first is used, and without a branch on the pairing (the
      // compiler would otherwise wait for the queries before it asks).  Adjacent pairs: lane q rotates
      // pairs 4q .. 4q+3 of every 16; halves: elements 8q .. 8q+7 of every 32 with their partners D/2 on.
      float2 angle[QK_STEPS * 4];
      const bool adjacent = fused.pairing == 1;
#pragma unroll
      for (int n = 0; n < QK_STEPS * 4; ++n)
        angle[n] = angles[adjacent ? (n / 4) * 16 + q * 4 + n % 4 : (n / 8) * 32 + q * 8 + n % 8];
      // the position is wanted in a scalar register from here on: ask now, not at its first use
      asm volatile("" ::"s"(position0));
      if (adjacent) {
#pragma unroll
        for (int s = 0; s < QK_STEPS; ++s)
#pragma unroll
          for (int pair = 0; pair < 4; ++pair) {
            float a = (float)query[t][s].v[2 * pair], b = (float)query[t][s].v[2 * pair + 1];
            rotate_pair(a, b, angle[s * 4 + pair]);
            query[t][s].v[2 * pair] = (bf16_t)a;
            query[t][s].v[2 * pair + 1] = (bf16_t)b;
          }
      } else {  // the partner of dim d is d + D/2: the same lane, QK_STEPS / 2 steps on (D % 64 == 0)
#pragma unroll
        for (int s = 0; s < QK_STEPS / 2; ++s)
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            float a = (float)query[t][s].v[i], b = (float)query[t][s + QK_STEPS / 2].v[i];
            rotate_pair(a, b, angle[s * 8 + i]);
            query[t][s].v[i] = (bf16_t)a;
            query[t][s + QK_STEPS / 2].v[i] = (bf16_t)b;
          }
      }
    }
#endif
  }

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
  const unsigned page_stride = (unsigned)kv_heads * page_size * D;  // elements of one page: checked to fit by the host
  const unsigned head_offset = (unsigned)kv_head * page_size * D;

  // FUSED: the wave that will read the newest key stores it (and the value) first; no other wave of the
  // workgroup reads it
  // (one token per tile when FUSED; with more than 16 query heads per kv head several workgroups store
  // the same values)
  const bool stores_token = FUSED && step_last >= step_begin && step_last < step_end &&
                            wave == (step_last - step_begin) % WAVES;
  if (stores_token && new_slot >= 0) {
    // element e of the key: piece e / 8 of the slot's offset, pieces page_size * 8 elements apart
    bf16_t* k_page = keys + (size_t)(new_slot / page_size) * page_stride + head_offset + (size_t)(new_slot % page_size) * KEY_PIECE;
    const unsigned piece_stride = (unsigned)page_size * KEY_PIECE;
    auto k_at = [&](int e) -> bf16_t& { return k_page[(unsigned)(e / KEY_PIECE) * piece_stride + e % KEY_PIECE]; };
    bf16_t* v_page = values + (size_t)(new_slot / page_size) * page_stride + head_offset +
                     (size_t)(new_slot % page_size / VALUE_PIECE) * (D * VALUE_PIECE) + new_slot % page_size % VALUE_PIECE;
#pragma unroll
    for (int i = 0; i < PAIR_PIECES; ++i) {
      const int j = lane + i * WAVE;
      if (j < D / 2) {
        float a = (float)new_a[i], b = (float)new_b[i];
        if (fused.pairing != 0) rotate_pair(a, b, new_angle[i]);
        k_at(fused.pairing == 2 ? j : 2 * j) = (bf16_t)a;
        k_at(fused.pairing == 2 ? j + D / 2 : 2 * j + 1) = (bf16_t)b;
      }
    }
#pragma unroll
    for (int i = 0; i < VALUE_PIECES; ++i) {
      const int d = lane + i * WAVE;
      if (d < D) v_page[(size_t)d * VALUE_PIECE] = new_v[i];  // (pages are multiples of eight keys here: common.h, value_element)
    }
    // Other lanes of this wave read these bytes back below.  A wave's accesses to memory are carried
    // out in the order it issues them, so nothing has to be waited for; the fence keeps the compiler
    // from moving the loads up.
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
  }

  // One step's loads.  The 32 keys of a step are dealt to the two 16-row tiles of the first product
  // so that a lane ends up with the scores of eight consecutive keys: row r of the "lo" tile is key
  // 8 * (r / 4) + r % 4 of the step, of the "hi" tile four keys further, and lane (c, q), which gets
  // rows 4q .. 4q+3 of both, holds keys 8q .. 8q+7.  That is the order the second product wants its
  // weights in, and its other operand is then one 16-byte piece of a row of the transposed V page
  // (row d = 16 * tile + c, keys 8q .. 8q+7; a page holds a multiple of 8 keys).  Keys outside
  // [first_key, last_key] are read from a key inside it (their weights are zero), so no page is
  // touched that the request does not hold.
  const int row_key = 8 * (c >> 2) + (c & 3);  // this lane's K row within a step (lo tile; hi: + 4)
  const int low_limit = first_key & ~7, high_limit = last_key & ~7;
  // Where a step's rows lie: the page numbers come from the block table (a load of their own,
  // requested two steps ahead so that the loads of the rows never wait for it), the offsets
  // within the pages are arithmetic.
  struct StepPages { int k, k_hi, v; };
  struct StepKeys { int k, k_hi, v; };
  auto keys_of = [&](int step) {  // the keys this lane reads in a step
    const int key0 = step * KEYS;
    StepKeys at = {key0 + row_key, key0 + row_key + 4, key0 + 8 * q};
    if (key0 < first_key || key0 + KEYS - 1 > last_key) {
      at.k = min(max(at.k, first_key), last_key);
      at.k_hi = min(max(at.k_hi, first_key), last_key);
      at.v = min(max(at.v, low_limit), high_limit);
    }
    return at;
  };
  auto page_index = [&](int key) { return page_shift >= 0 ? key >> page_shift : key / page_size; };
  auto pages_of = [&](int step) {
    const StepKeys at = keys_of(step);
    return StepPages{table[page_index(at.k)], table[page_index(at.k_hi)], table[page_index(at.v)]};
  };
  auto fetch_keys = [&](int step, const StepPages& P, StepLoads& L) {
    const StepKeys at = keys_of(step);
    const int offset = at.k - page_index(at.k) * page_size, offset_hi = at.k_hi - page_index(at.k_hi) * page_size;
    const bf16_t* key_lo = keys + (size_t)(unsigned)P.k * page_stride + (head_offset + (unsigned)offset * KEY_PIECE);
    const bf16_t* key_hi = keys + (size_t)(unsigned)P.k_hi * page_stride + (head_offset + (unsigned)offset_hi * KEY_PIECE);
    const unsigned piece_stride = (unsigned)page_size * KEY_PIECE;
#pragma unroll
    for (int s = 0; s < QK_STEPS; ++s) {
      L.k_lo[s] = load_qk(key_lo, piece_stride, s, q);
      L.k_hi[s] = load_qk(key_hi, piece_stride, s, q);
    }
  };
  auto fetch_values = [&](int step, const StepPages& P, StepLoads& L) {
    const StepKeys at = keys_of(step);
    // the lane's eight keys are one piece of the page: [page_size / 8][D][8], the rows of a piece side by side
    const bf16_t* base = values + (size_t)(unsigned)P.v * page_stride +
                         (head_offset + (unsigned)(at.v - page_index(at.v) * page_size) * (unsigned)D);
#pragma unroll
    for (int d = 0; d < D_TILES; ++d) L.v[d] = *(const bf16x8*)(base + (unsigned)(d * 16 + c) * VALUE_PIECE);
  };

  const float scale_log2 = scale * 1.44269504088896f;

  // A wave's next step is requested into the registers of the current one as soon as they are
  // free: the K rows after the first product, the V rows after the second; the page numbers of a
  // step are looked up a step before its rows are requested.
  if (step_begin + wave < step_end) {
    const int step0 = step_begin + wave;
    StepLoads loads;
    StepPages pages = early_pages && step0 < step_last ? StepPages{early_k, early_k_hi, early_v} : pages_of(step0);
    fetch_keys(step0, pages, loads);
    fetch_values(step0, pages, loads);
    if constexpr (TWO_STEPS) {
      // A step of single tokens is a few trips to memory in a row, and a wave has two or three steps to
      // walk: its second step's K and V are asked for together with the first's, into registers of their
      // own, and each of the two sets is filled again as soon as its step has been multiplied.
      auto multiply = [&](int step, StepLoads& L) {
        f32x4 s_lo[COLUMN_TILES], s_hi[COLUMN_TILES];
        scores_of(columns, L, s_lo, s_hi);
        const int key0 = step * KEYS;
        const bool interior = key0 + KEYS - 1 <= position0 && (window <= 0 || key0 >= last_key - window + 1);
        weigh_and_add(columns, L, s_lo, s_hi, key0, q, interior, last_key,
                      min(max(key0 + 8 * q, low_limit), high_limit), scale_log2);
      };
      StepLoads ahead;
      const int step1 = step0 + WAVES;
      if (step1 < step_end) {
        const StepPages pages1 =
            second_pages && step1 < step_last ? StepPages{second_k, second_k_hi, second_v} : pages_of(step1);
        fetch_keys(step1, pages1, ahead);
        fetch_values(step1, pages1, ahead);
      }
      StepPages pages_even = pages, pages_odd = pages;  // of the steps that will fill `loads` and `ahead` again
      if (step0 + 2 * WAVES < step_end) pages_even = pages_of(step0 + 2 * WAVES);
      if (step0 + 3 * WAVES < step_end) pages_odd = pages_of(step0 + 3 * WAVES);
      for (int step = step0; step < step_end; step += 2 * WAVES) {
        multiply(step, loads);
        if (step + 2 * WAVES < step_end) {
          fetch_keys(step + 2 * WAVES, pages_even, loads);
          fetch_values(step + 2 * WAVES, pages_even, loads);
          if (step + 4 * WAVES < step_end) pages_even = pages_of(step + 4 * WAVES);
        }
        if (step + WAVES < step_end) {
          multiply(step + WAVES, ahead);
          if (step + 3 * WAVES < step_end) {
            fetch_keys(step + 3 * WAVES, pages_odd, ahead);
            fetch_values(step + 3 * WAVES, pages_odd, ahead);
            if (step + 5 * WAVES < step_end) pages_odd = pages_of(step + 5 * WAVES);
          }
        }
      }
    } else {
    if (step0 + WAVES < step_end) pages = pages_of(step0 + WAVES);
    for (int step = step0; step < step_end; step += WAVES) {
      const bool more = step + WAVES < step_end;
      f32x4 s_lo[COLUMN_TILES], s_hi[COLUMN_TILES];
      scores_of(columns, loads, s_lo, s_hi);
      if (more) fetch_keys(step + WAVES, pages, loads);
      const int key0 = step * KEYS;
      const bool interior = key0 + KEYS - 1 <= position0 && (window <= 0 || key0 >= last_key - window + 1);
      weigh_and_add<COLUMN_TILES, CHANGED>(columns, loads, s_lo, s_hi, key0, q, interior, last_key,
                                           min(max(key0 + 8 * q, low_limit), high_limit), scale_log2, change.soft_cap);
      if (more) fetch_values(step + WAVES, pages, loads);
      if (step + 2 * WAVES < step_end) pages = pages_of(step + 2 * WAVES);
    }
    }
  }

  // merge the waves, one column tile at a time: each wave leaves, per column, D sums, its
  // maximum and its sum of weights
  // (a column's row is D sums, then its maximum and its sum of weights; rows 16 bytes apart in the banks, so that a
  // lane's four sums of a tile go and come as one 16-byte piece)
  constexpr int STRIDE = D + 4;
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t) {
    float sum = running_sum[t];
    sum += __shfl_xor(sum, 16, WAVE);
    sum += __shfl_xor(sum, 32, WAVE);
    float* mine = lds + ((size_t)wave * 16 + c) * STRIDE;
#pragma unroll
    for (int d = 0; d < D_TILES; ++d) *(f32x4*)(mine + d * 16 + 4 * q) = acc[t][d];
    if (q == 0) *(float2*)(mine + D) = make_float2(running_max[t], sum);
    __syncthreads();
    for (int index = threadIdx.x; index < 16 * (D / 4); index += WAVES * 64) {
      const int column = index / (D / 4), d4 = (index % (D / 4)) * 4;
      int token, head_here;
      bool live;
      map.of(t, column, token, head_here, live);
      if (!live) continue;
      float2 theirs_ml[WAVES];
      f32x4 theirs_acc[WAVES];
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        const float* theirs = lds + ((size_t)w * 16 + column) * STRIDE;
        theirs_ml[w] = *(const float2*)(theirs + D);
        theirs_acc[w] = *(const f32x4*)(theirs + d4);
      }
      float best = -INFINITY;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) best = fmaxf(best, theirs_ml[w].x);
      float total = 0.f;
      f32x4 merged = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        const float factor = theirs_ml[w].x == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(theirs_ml[w].x - best);
        total += theirs_ml[w].y * factor;
        merged += theirs_acc[w] * factor;
      }
      const int head = kv_head * group + head_tile * 16 + head_here;
      const size_t row = (size_t)row0 + token;
      if (splits == 1) {
        const float inverse = total > 0.f ? 1.f / total : 0.f;
        const bf16x4 rounded = {(bf16_t)(merged[0] * inverse), (bf16_t)(merged[1] * inverse), (bf16_t)(merged[2] * inverse),
                                (bf16_t)(merged[3] * inverse)};
        *(bf16x4*)(out + (row * heads + head) * D + d4) = rounded;
      } else {
        const size_t kept_as = fused.by_item ? (size_t)(gridDim.x - 1 - blockIdx.x) * tokens_per_tile + token : row;
        const size_t slot = (kept_as * heads + head) * splits + blockIdx.z;
        if (fused.unmerged) {
          // for the product that merges: [head][split][piece of 8][16 rows][8], the rows of a piece side by
          // side, so that the four lanes of its loads that hold four rows' share of a piece read 64 bytes
          // in a row (the step has at most 16 rows)
          const size_t of_split = (size_t)head * splits + blockIdx.z;
          bf16_t* dst = (bf16_t*)partial_acc + ((of_split * (D / 8) + d4 / 8) * 16 + row) * 8 + d4 % 8;
          const float inverse = total > 0.f ? 1.f / total : 0.f;
          const bf16x4 rounded = {(bf16_t)(merged[0] * inverse), (bf16_t)(merged[1] * inverse), (bf16_t)(merged[2] * inverse),
                                  (bf16_t)(merged[3] * inverse)};
          *(bf16x4*)dst = rounded;
          if (d4 == 0) *(float2*)(partial_ml + (of_split * 16 + row) * 2) = make_float2(best, total);
        } else {
          *(f32x4*)(partial_acc + slot * D + d4) = merged;
          if (d4 == 0) *(float2*)(partial_ml + slot * 2) = make_float2(best, total);
        }
      }
    }
    __syncthreads();
  }
}

// Merges the key splits of one (token, head): out = sum_s acc_s * 2^(m_s - m) / sum_s l_s *
// 2^(m_s - m), in split order (the maxima are kept in units of log2).  A second kernel rather than "the last workgroup merges": a
// workgroup that reads what others wrote needs the other chiplets' L2 written back first, and
// that costs more than this launch.
// A thread a dimension, at most 64 splits: in every wave lane s asks for split s's maximum and sum (one trip to
// memory for all of them, where a loop over the splits made one after the other: nine splits took
// 14.6 us, thirty-three 41), the wave agrees on the largest and on the total, and every thread then adds up
// its dimension over the splits, whose partial sums it asks for up to thirty-two at a time (one wave that took two
// dimensions a lane and eight splits at a time made six trips in a row for twenty-four splits; attention and merge
// together, us a layer: one request over 8,192 keys in 64 splits 16.5 -> 11.4, four over 16,384 in 48 30.0 -> 26.9,
// eight over 30,000 in 12 52.7 -> 50.5).
#define MERGE_SPLITS_MAX 64
constexpr int MERGE_THREADS = (D + WAVE - 1) / WAVE * WAVE;

template <int AT_ONCE>
__device__ __forceinline__ float merge_some(const float* acc, int first, int splits, float weight) {
  float part[AT_ONCE];
#pragma unroll
  for (int i = 0; i < AT_ONCE; ++i) part[i] = acc[(size_t)min(first + i, splits - 1) * D];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < AT_ONCE; ++i) {
    const float w = __shfl(weight, min(first + i, MERGE_SPLITS_MAX - 1), WAVE);
    if (first + i < splits && w != 0.f) sum += part[i] * w;
  }
  return sum;
}

// out[d] = sum_s acc_s[d] w_s / sum_s l_s w_s of the splits whose maxima and sums lie at `ml` and partial sums at
// `acc`, for the dimensions threadIdx.x, threadIdx.x + blockDim.x, ...; every lane of every wave must call it (the
// weights pass between lanes)
__device__ __forceinline__ void merge_splits(const float* ml, const float* acc, int splits, bf16_t* out) {
  const int lane = threadIdx.x & (WAVE - 1);
  const float2 mine = lane < splits ? *(const float2*)(ml + (size_t)lane * 2) : make_float2(-INFINITY, 0.f);
  const float best = wave_max(mine.x);
  const float weight = mine.x == -INFINITY ? 0.f : exp2f(mine.x - best);  // a split that saw no key counts nothing
  const float total = wave_sum(mine.y * weight);                          // (lanes beyond the splits add 0)
  const float inverse = total > 0.f ? 1.f / total : 0.f;
  for (int d0 = 0; d0 < D; d0 += blockDim.x) {  // (the same trips for all lanes: those beyond D read D - 1 and store nothing)
    const int d = d0 + threadIdx.x;
    const float* mine_acc = acc + min(d, D - 1);
    float sum = 0.f;
    int first = 0;
    for (; splits - first > 8; first += 32) sum += merge_some<32>(mine_acc, first, splits, weight);
    if (first < splits) sum += merge_some<8>(mine_acc, first, splits, weight);
    if (d < D) out[d] = (bf16_t)(sum * inverse);
  }
}

// (a workgroup of one thread a dimension where the (token, head) pairs are few and the trips count, of one wave where
// they are many: a prompt portion's 24,576 pairs in four splits 12 us against 15)
__global__ __launch_bounds__(MERGE_THREADS) void attention_merge_kernel(const float* __restrict__ partial_acc,
                                                                        const float* __restrict__ partial_ml,
                                                                        bf16_t* __restrict__ out, int splits) {
  const size_t pair = blockIdx.x;  // row * heads + head
  merge_splits(partial_ml + pair * splits * 2, partial_acc + pair * splits * D, splits, out + pair * D);
}

// The same for partial results that are kept by work item: workgroup (item, head) merges the item's tokens one
// after the other (a few), and writes to the rows that the item names.
__global__ __launch_bounds__(MERGE_THREADS) void attention_merge_items_kernel(const float* __restrict__ partial_acc,
                                                                              const float* __restrict__ partial_ml,
                                                                              bf16_t* __restrict__ out,
                                                                              const int* __restrict__ work, int splits,
                                                                              int heads, int group, int tokens_per_tile) {
  const int* item = work + (size_t)blockIdx.x * 4;
  const int tokens = group <= 16 ? (item[2] + item[3] + group - 1) / group : item[3];
  const int head = blockIdx.y;
  for (int token = 0; token < tokens; ++token) {
    const size_t kept_as = ((size_t)blockIdx.x * tokens_per_tile + token) * heads + head;
    const size_t pair = ((size_t)item[1] + token) * heads + head;
    merge_splits(partial_ml + kept_as * splits * 2, partial_acc + kept_as * splits * D, splits, out + pair * D);
  }
}

static int launch_merge(float* partial_acc, float* partial_ml, void* out, int splits, size_t pairs, hipStream_t stream) {
  hipLaunchKernelGGL(attention_merge_kernel, dim3((unsigned)pairs), dim3(pairs >= 4096 ? WAVE : MERGE_THREADS), 0, stream,
                     partial_acc, partial_ml, (bf16_t*)out, splits);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- prompt portions, D = 128
// For portions of many tokens the kernel above reads every key once per few tokens, and what bounds it
// then is the path from the caches into the registers (every wave asks for its own 16 KB a step).  This
// one shares each step's K and V among the four waves of a workgroup through LDS.  A workgroup takes up
// to 4 * COLUMN_TILES column tiles of a request (128 (token, head) pairs with two tiles: 21 tokens at six
// query heads a kv head); every wave owns its own column tiles and walks all of their keys itself (no
// key split inside the workgroup, nothing to merge).  A step's 32 K rows and 128 x 32 V^T block (16 KB)
// go from memory straight into LDS (global_load_lds_dwordx4: each lane names its own 16 bytes of memory,
// and the 64 lanes of an instruction fill 1 KB of LDS in lane order), sixteen such instructions a step,
// four from each wave, a pair of steps ahead of their use, into one of four stages.  Who asks for what is
// chosen so that LDS holds the operands as the products read them, a whole wave 1 KB in a row:
//   K: chunks 2j and 2j+1 (1 KB each) = pieces 4j .. 4j+3 (eight elements each) of the 16 rows of the "lo"
//      and of the "hi" tile of the first product (for lane (c, q) piece 4j + q of row c)
//   V: chunk t (1 KB) = tile t of V^T: for lane (c, q) the keys 8q .. 8q+7 of row 16 t + c.
// The loads are written in assembly: the compiler knows that such a load writes LDS but not where, and
// makes every later read of LDS wait for all of them, so they could not run ahead.  Here the waits are
// counted by hand (the loop holds no other vector memory instruction): before the barrier that ends a
// pair of steps, every wave waits for the loads it asked for at the pair's beginning.
#if HEAD_DIM == 128
constexpr int PORTION_STAGE_BYTES = 2 * KEYS * D * 2;  // K rows, then V^T rows
constexpr int PORTION_STAGES = 4;

// (the instruction takes its place in LDS from M0; the register is given back as it was, the compiler is not told of it)
__device__ __forceinline__ void load_to_lds(const bf16_t* from, unsigned to) {
  unsigned kept;
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, off\n\ts_mov_b32 m0, %0"
               : "=&s"(kept)
               : "s"(to), "v"(from)
               : "memory");
}

template <int COLUMN_TILES>
__global__ __launch_bounds__(256, 2) void attention_portions_kernel(
    const bf16_t* __restrict__ qkv, int row_width, bf16_t* __restrict__ out, float* __restrict__ partial_acc,
    float* __restrict__ partial_ml, const bf16_t* __restrict__ keys,
    const bf16_t* __restrict__ values, const int* __restrict__ block_tables, int table_width,
    const int* __restrict__ positions, const int* __restrict__ work, int heads, int kv_heads, int tokens_per_tile,
    int page_size, int page_shift, float scale, int window, int splits) {
  __shared__ __attribute__((aligned(1024))) char stages[PORTION_STAGES * PORTION_STAGE_BYTES];
  const int group = heads / kv_heads;
  const int kv_head = blockIdx.y % kv_heads, head_tile = blockIdx.y / kv_heads;
  const int heads_here = min(group - head_tile * 16, 16);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, q = lane >> 4;
  const int* item = work + (size_t)(gridDim.x - 1 - blockIdx.x) * 4;  // late tokens walk more keys: they start first
  const int request = __builtin_amdgcn_readfirstlane(item[0]), row_first = __builtin_amdgcn_readfirstlane(item[1]);
  const ColumnMap all = {heads_here, __builtin_amdgcn_readfirstlane(item[2]), __builtin_amdgcn_readfirstlane(item[3]),
                         group <= 16};
  const int tokens_all = all.tokens();
  const int position_first = __builtin_amdgcn_readfirstlane(positions[row_first]);
  // the workgroup's keys, and this wave's: its COLUMN_TILES column tiles of the item's columns
  const int last_key_all = position_first + tokens_all - 1;
  const int first_key_all = window > 0 ? max(0, position_first - window + 1) : 0;
  const int skipped = wave * COLUMN_TILES * (all.packed ? 16 : 1);  // columns (packed) or tokens before this wave's
  const int mine_first = all.packed ? all.over_heads(all.first_head + skipped) : skipped;  // its first token, within the item
  const ColumnMap map = {heads_here, all.packed ? all.first_head + skipped - mine_first * heads_here : 0,
                         max(0, min(all.columns - skipped, COLUMN_TILES * (all.packed ? 16 : 1))), all.packed};
  const int tokens = map.columns > 0 ? map.tokens() : 0;  // 0: nothing of its own
  const int row0 = row_first + mine_first, position0 = position_first + mine_first;
  const int last_key = position0 + tokens - 1;
  const int first_key = window > 0 ? max(0, position0 - window + 1) : 0;
  const int* table = block_tables + (size_t)request * table_width;

  Columns<COLUMN_TILES> columns;
  bool column_live[COLUMN_TILES];
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t) {
    int token, head_here;
    map.of(t, c, token, head_here, column_live[t]);
    const int safe = max(0, min(token, tokens - 1));
    const int head = kv_head * group + head_tile * 16 + head_here;
    columns.position[t] = column_live[t] ? position0 + safe : -1;
    columns.first[t] = window > 0 ? columns.position[t] - window + 1 : 0;
    const bf16_t* q_row = qkv + (size_t)(min(row0, row_first + tokens_all - 1) + safe) * row_width + (size_t)head * D;
#pragma unroll
    for (int s = 0; s < QK_STEPS; ++s) columns.query[t][s] = load_qk(q_row, KEY_PIECE, s, q);  // a query's row is in one piece
    columns.running_max[t] = -INFINITY;
    columns.running_sum[t] = 0.f;
#pragma unroll
    for (int d = 0; d < D_TILES; ++d) columns.acc[t][d] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  // The queries were asked for with ordinary loads, which the compiler counts: made to wait for them here, it
  // knows them arrived; left to wait at their first use, inside the walk, it would wait there for everything
  // that is under way, the loads into LDS included.
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t)
#pragma unroll
    for (int s = 0; s < QK_STEPS; ++s) asm volatile("" ::"v"(columns.query[t][s].v));

  // the item's steps, of which this workgroup walks one of `splits` runs (blockIdx.z; possibly none)
  const int step_first_item = first_key_all / KEYS, step_last_item = last_key_all / KEYS;
  const int per_split = (step_last_item - step_first_item + splits) / splits;
  const int step_first_all = step_first_item + (int)blockIdx.z * per_split;
  const int step_last_all = min(step_last_item, step_first_all + per_split - 1);
  const int step_first = first_key / KEYS, step_last = tokens > 0 ? last_key / KEYS : -1;
  const unsigned page_stride = (unsigned)kv_heads * page_size * D;
  const unsigned head_offset = (unsigned)kv_head * page_size * D;

  // Pages hold 16 keys, or a power of two beyond (the entry point refuses others): a step lies in two pages or in
  // one.  Their numbers come through scalar loads, asked for a step before the step's rows are; the entries looked
  // at are kept within the blocks that hold the item's keys, so that a step that reaches beyond them (the last
  // one, the first under a window, the steps asked for past the end) reads rows of a page the request holds:
  // rows of other keys than it wants, all of which the mask weighs with zero.
  struct StepPages { int first, second; };
  const int first_block = first_key_all >> page_shift, last_block = last_key_all >> page_shift;
  const int second_page = page_shift == 4 ? 1 : 0;
  auto pages_of_step = [&](int step) {
    const int block = (step * KEYS) >> page_shift;
    return StepPages{table[min(max(block, first_block), last_block)],
                     table[min(max(block + second_page, first_block), last_block)]};
  };
  // What this lane asks for in every step: of K the piece 4 wave + lane / 16 of row lane % 16 of the "lo" tile
  // (key 8 (row / 4) + row % 4 of the step) and of the same row of the "hi" tile (four keys on: 64 bytes on in
  // the page); of V^T the keys 8 (lane / 16) .. + 7 of rows 32 wave + lane % 16 and sixteen further (256 bytes on).
  // So an address is the page's number times the bytes of a page on top of what is fixed for the lane and, with
  // pages of more than 32 keys, for the step.
  const int row_key = 8 * (c >> 2) + (c & 3);
  const unsigned k_piece = 4 * wave + q;
  const unsigned v_row = 32 * wave + c;
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) void*)stages;
  const unsigned in_page = (unsigned)page_size - 1;
  const char* k_lane = (const char*)(keys + (head_offset + (k_piece * page_size + ((unsigned)row_key & in_page)) * KEY_PIECE));
  const char* v_lane = (const char*)(values + (head_offset + ((8u * q) & in_page) * D + v_row * VALUE_PIECE));
  const unsigned page_bytes = page_stride * 2;
  const bool k_upper = c >= 8, v_upper = q >= 2;  // which of a step's two pages of 16 keys
  auto fill_step = [&](int step, const StepPages& pages, int stage) {
    const unsigned to = __builtin_amdgcn_readfirstlane(lds_base + (unsigned)stage * PORTION_STAGE_BYTES + (unsigned)wave * 2048);
    const unsigned of_step = (unsigned)(step * KEYS) & in_page;  // (0 unless a page holds several steps)
    const char* k_from = k_lane + (size_t)(unsigned)(k_upper ? pages.second : pages.first) * page_bytes + of_step * (KEY_PIECE * 2);
    const char* v_from = v_lane + (size_t)(unsigned)(v_upper ? pages.second : pages.first) * page_bytes + of_step * (D * 2);
    load_to_lds((const bf16_t*)k_from, to);
    load_to_lds((const bf16_t*)(k_from + 4 * KEY_PIECE * 2), to + 1024);
    load_to_lds((const bf16_t*)v_from, to + KEYS * D * 2);
    load_to_lds((const bf16_t*)(v_from + 16 * VALUE_PIECE * 2), to + KEYS * D * 2 + 1024);
  };
  // Two steps a barrier: the four stages are two pairs, one being read while the other is filled.  At the end of
  // a pair of steps every wave has read its stages and waits for what it asked for at the pair's beginning; after
  // the barrier that holds for all waves.
  auto end_of_pair = [&]() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

  const float scale_log2 = scale * 1.44269504088896f;
  const unsigned read_k = lane * 16, read_v = KEYS * D * 2 + lane * 16;  // this lane's bytes within a stage
  auto walk_step = [&](int step, int stage) {
    if (step >= step_first && step <= min(step_last, step_last_all)) {
      const char* from = stages + stage * PORTION_STAGE_BYTES;
      StepLoads loads;
#pragma unroll
      for (int s = 0; s < QK_STEPS; ++s) {
        loads.k_lo[s].v = *(const bf16x8*)(from + read_k + s * 2048);
        loads.k_hi[s].v = *(const bf16x8*)(from + read_k + s * 2048 + 1024);
      }
#pragma unroll
      for (int d = 0; d < D_TILES; ++d) loads.v[d] = *(const bf16x8*)(from + read_v + d * 1024);
      f32x4 s_lo[COLUMN_TILES], s_hi[COLUMN_TILES];
      scores_of(columns, loads, s_lo, s_hi);
      const int key0 = step * KEYS;
      const bool interior = key0 >= first_key_all && key0 + KEYS - 1 <= position0 && (window <= 0 || key0 >= last_key - window + 1);
      // (which keys' values the lane really read: those of a block that the item's keys lie in)
      const int value_block = min(max((key0 + 8 * q) >> page_shift, first_block), last_block);
      const int value_key = (value_block << page_shift) + ((key0 + 8 * q) & (int)in_page);
      weigh_and_add(columns, loads, s_lo, s_hi, key0, q, interior, last_key_all, value_key, scale_log2);
    }
  };
  fill_step(step_first_all, pages_of_step(step_first_all), 0);
  fill_step(step_first_all + 1, pages_of_step(step_first_all + 1), 1);
  StepPages next_even = pages_of_step(step_first_all + 2), next_odd = pages_of_step(step_first_all + 3);
  end_of_pair();
  int pair = 0;
  for (int step = step_first_all; step <= step_last_all; step += 2) {
    // (page numbers for the pair after next: used an iteration from now, nothing waits for them here)
    const StepPages after_even = pages_of_step(step + 4), after_odd = pages_of_step(step + 5);
    // (steps past the last ask for rows of the last block)
    fill_step(step + 2, next_even, 2 - 2 * pair);
    fill_step(step + 3, next_odd, 3 - 2 * pair);
    walk_step(step, 2 * pair);
    walk_step(step + 1, 2 * pair + 1);
    end_of_pair();
    next_even = after_even;
    next_odd = after_odd;
    pair = 1 - pair;
  }
  // LDS is used once more below: nothing may still be on its way into it
  asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");

  // each wave's columns leave through LDS of its own (16 columns x 128 floats) as whole rows: of `out`,
  // divided by the sum of weights, or (splits > 1) of the split's partial sums as they are, with the column's
  // reference maximum and sum of weights beside them, for the kernel that merges
  constexpr int STRIDE = D + 4;  // (a row of 128 floats would put all sixteen columns into the same banks)
  float* mine = (float*)stages + (size_t)wave * 16 * STRIDE;
  float2* mine_ml = (float2*)((float*)stages + 4 * 16 * STRIDE) + wave * 16;
#pragma unroll
  for (int t = 0; t < COLUMN_TILES; ++t) {
    float sum = columns.running_sum[t];
    sum += __shfl_xor(sum, 16, WAVE);
    sum += __shfl_xor(sum, 32, WAVE);
    const float inverse = splits > 1 ? 1.f : sum > 0.f ? 1.f / sum : 0.f;
#pragma unroll
    for (int d = 0; d < D_TILES; ++d)
      *(f32x4*)(mine + (size_t)c * STRIDE + d * 16 + 4 * q) = columns.acc[t][d] * inverse;
    if (splits > 1 && q == 0) mine_ml[c] = make_float2(columns.running_max[t], sum);
    // lane (column l / 4, quarter l % 4) writes 32 values of the column's row
    const int column = lane >> 2, quarter = lane & 3;
    int token, head_here;
    bool live;
    map.of(t, column, token, head_here, live);
    if (live) {
      const int head = kv_head * group + head_tile * 16 + head_here;
      const float* from = mine + (size_t)column * STRIDE + quarter * 32;
      if (splits > 1) {
        const size_t slot = ((size_t)(row0 + token) * heads + head) * splits + blockIdx.z;
        float* dst = partial_acc + slot * D + quarter * 32;
#pragma unroll
        for (int piece = 0; piece < 8; ++piece) *(f32x4*)(dst + piece * 4) = *(const f32x4*)(from + piece * 4);
        if (quarter == 0) *(float2*)(partial_ml + slot * 2) = mine_ml[column];
      } else {
        bf16_t* dst = out + ((size_t)(row0 + token) * heads + head) * D + quarter * 32;
#pragma unroll
        for (int piece = 0; piece < 4; ++piece) {
          const f32x4 lo = *(const f32x4*)(from + piece * 8);
          const f32x4 hi = *(const f32x4*)(from + piece * 8 + 4);
          bf16_t packed[8] = {(bf16_t)lo[0], (bf16_t)lo[1], (bf16_t)lo[2], (bf16_t)lo[3],
                              (bf16_t)hi[0], (bf16_t)hi[1], (bf16_t)hi[2], (bf16_t)hi[3]};
          *(uint4*)(dst + piece * 8) = *(const uint4*)packed;
        }
      }
    }
  }
}

// `work` holds `items` entries as for llmserve_attention_tiles; an item covers at most 4 * column_tiles
// column tiles (column_tiles 1 or 2), tokens_per_tile = max(1, 16 / (heads /
// kv_heads)).  page_size a power of two from 16 on.
extern "C" int llmserve_attention_portions(const void* qkv, int row_width, void* out, float* partial_acc,
                                           float* partial_ml, const void* keys,
                                           const void* values, const int* block_tables, int table_width,
                                           const int* positions, const int* work, int items, int column_tiles,
                                           int rows, int heads, int kv_heads, int page_size, float scale, int window,
                                           int splits, hipStream_t stream) {
  if (items <= 0) return 0;
  if (heads % kv_heads || page_size < 16 || (page_size & (page_size - 1)) != 0 || (column_tiles != 1 && column_tiles != 2))
    return ERR_BAD_ARGUMENT;
  if (splits < 1 || splits > MERGE_SPLITS_MAX || (splits > 1 && (!partial_acc || !partial_ml))) return ERR_BAD_ARGUMENT;
  if ((long)kv_heads * page_size * D >= (1L << 30)) return ERR_BAD_ARGUMENT;  // a page's bytes are counted in 32 bits
  const int group = heads / kv_heads;
  const int tokens_per_tile = group >= 16 ? 1 : 16 / group;
  const int page_shift = __builtin_ctz(page_size);
  const dim3 grid(items, kv_heads * ((group + 15) / 16), splits);
  if (column_tiles == 1)
    hipLaunchKernelGGL(attention_portions_kernel<1>, grid, dim3(256), 0, stream, (const bf16_t*)qkv, row_width,
                       (bf16_t*)out, partial_acc, partial_ml, (const bf16_t*)keys, (const bf16_t*)values, block_tables,
                       table_width, positions, work, heads, kv_heads, tokens_per_tile, page_size, page_shift, scale,
                       window, splits);
  else
    hipLaunchKernelGGL(attention_portions_kernel<2>, grid, dim3(256), 0, stream, (const bf16_t*)qkv, row_width,
                       (bf16_t*)out, partial_acc, partial_ml, (const bf16_t*)keys, (const bf16_t*)values, block_tables,
                       table_width, positions, work, heads, kv_heads, tokens_per_tile, page_size, page_shift, scale,
                       window, splits);
  const int status = LAUNCH_STATUS();
  if (status != 0 || splits == 1) return status;
  return launch_merge(partial_acc, partial_ml, out, splits, (size_t)rows * heads, stream);
}
#else
extern "C" int llmserve_attention_portions(const void*, int, void*, float*, float*, const void*, const void*, const int*,
                                           int, const int*, const int*, int, int, int, int, int, int, float, int, int,
                                           hipStream_t) {
  return ERR_BAD_ARGUMENT;  // built for head size 128 only
}
#endif

// waves of a workgroup of the fused decode form: eight walk a tile's keys where the registers allow it
#ifndef FUSED_WAVES
#define FUSED_WAVES (HEAD_DIM > 128 ? 4 : 8)
#endif
template <int COLUMN_TILES, bool FUSED, int WAVES, bool CHANGED = false>
static int launch_tiles(const void* qkv, int row_width, void* out, float* partial_acc, float* partial_ml,
                        void* keys, void* values, const int* block_tables, int table_width,
                        const int* positions, const int* work, int tiles, int heads, int kv_heads,
                        int tokens_per_tile, int page_size, float scale, int window, int splits, FusedDecode fused,
                        hipStream_t stream, ScoreChange change = {nullptr, 0.f}) {
  const int group = heads / kv_heads;
  const int page_shift = (page_size & (page_size - 1)) == 0 ? __builtin_ctz(page_size) : -1;
  const int head_tiles = (group + 15) / 16;
  const size_t shared = (size_t)WAVES * 16 * (D + 4) * sizeof(float);
  if (shared > 64 * 1024) {  // more dynamic LDS than a kernel gets by default: ask for it once
    static bool asked = false;
    if (!asked) {
      if (hipFuncSetAttribute((const void*)attention_tiles_kernel<COLUMN_TILES, FUSED, WAVES, CHANGED>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)shared) != hipSuccess)
        return ERR_BAD_ARGUMENT;
      asked = true;
    }
  }
  hipLaunchKernelGGL((attention_tiles_kernel<COLUMN_TILES, FUSED, WAVES, CHANGED>), dim3(tiles, kv_heads * head_tiles, splits),
                     dim3(WAVES * 64), shared, stream, (const bf16_t*)qkv, row_width, (bf16_t*)out, partial_acc,
                     partial_ml, (bf16_t*)keys, (bf16_t*)values, block_tables, table_width, positions, work,
                     heads, kv_heads, tokens_per_tile, page_size, page_shift, scale, window, splits, fused, change);
  return LAUNCH_STATUS();
}

extern "C" int llmserve_attention_head_dim() { return D; }


// Whether the fused decode form can rotate with this pairing at this head size.
extern "C" int llmserve_attention_can_fuse(int pairing) {
  if (pairing == 0) return 1;
  if (D % 32 != 0) return 0;
  return pairing == 1 || (pairing == 2 && D % 64 == 0);
}

// `work` holds `tiles` items of four ints {request index in the step, first token row, first head,
// columns}: with up to 16 query heads a kv head a run of at most `column_tiles` * 16 (token, head)
// pairs of the request, beginning at `first head` of the first token; with more, at most
// `column_tiles` tokens ("columns" counts tokens).  page_size must be a multiple of 8.  With splits > 1, partial_acc is float32 [rows * heads * splits * D],
// partial_ml [rows * heads * splits * 2] (rows being the step's token count), and every row
// of the step must lie in one of the tiles: a second kernel merges the splits of all rows.
// With `fuse` tile i is row i, the one token of request i (`work` is not read), qkv is as the projection left it, and the kernel
// rotates (table of cos and sin per row, pairing) and stores the token's key and value at slots[row] itself.
// `fuse` = 4 (column_tiles 1, splits > 1): the items are the few short requests of a step that also holds long portions;
// partial_acc [tiles * tokens_per_tile * heads * splits * D] and partial_ml are kept by item, and only the items' rows
// are merged and written.
// `fuse` + 2 leaves the key splits unmerged for a reader that merges them itself (gemm_merged; at most 16 rows):
// partial_acc is then bfloat16 [heads][splits][D / 8][16 rows][8], each split's result divided by its own sum of
// weights, and partial_ml [heads][splits][16 rows][2] holds each split's maximum (in units of log2) and sum of
// weights.
// `slopes` (float32 [heads], or null) and `soft_cap` (0 for none) change the scores before the softmax (see the head of
// this file); not together with `fuse` & 1.
extern "C" int llmserve_attention_tiles(const void* qkv, int row_width, void* out, float* partial_acc,
                                        float* partial_ml, void* keys, void* values,
                                        const int* block_tables, int table_width, const int* positions,
                                        const int* work, int tiles, int column_tiles, int rows, int heads,
                                        int kv_heads, int page_size, float scale, int window, int splits, int fuse,
                                        const float* table, int pairing, const int* slots, const float* slopes,
                                        float soft_cap, hipStream_t stream) {
  if (tiles <= 0) return 0;
  const bool changed = slopes != nullptr || soft_cap > 0.f;
  if (soft_cap < 0.f || (changed && (fuse & 1))) return ERR_BAD_ARGUMENT;
  const ScoreChange change = {slopes, soft_cap};
  if (heads % kv_heads || page_size % 8 || splits < 1 || splits > MERGE_SPLITS_MAX || (splits > 1 && (!partial_acc || !partial_ml)))
    return ERR_BAD_ARGUMENT;
  if ((long)kv_heads * page_size * D >= (1L << 31)) return ERR_BAD_ARGUMENT;  // a page's elements are counted in 32 bits
  const int group = heads / kv_heads;
  const int tokens_per_tile = group >= 16 ? 1 : 16 / group;
  const bool unmerged = (fuse & 2) != 0 && splits > 1;  // the splits stay as they are: whoever reads them merges them
  if (unmerged && rows > 16) return ERR_BAD_ARGUMENT;
  const bool by_item = (fuse & 4) != 0 && splits > 1;  // partial results by work item, merged for the items' rows only
  if (by_item && ((fuse & 3) != 0 || column_tiles != 1)) return ERR_BAD_ARGUMENT;
  fuse &= 1;
  FusedDecode fused = {(const float2*)table, pairing, slots, unmerged ? 1 : 0, by_item ? 1 : 0};
  int status;
  if (fuse) {
    if (column_tiles != 1 || tiles != rows || !slots || !llmserve_attention_can_fuse(pairing) || (pairing != 0 && !table))
      return ERR_BAD_ARGUMENT;
    status = launch_tiles<1, true, FUSED_WAVES>(qkv, row_width, out, partial_acc, partial_ml, keys, values, block_tables,
                                        table_width, positions, work, tiles, heads, kv_heads, tokens_per_tile,
                                        page_size, scale, window, splits, fused, stream);
  } else if (changed && column_tiles == 1) {
    status = launch_tiles<1, false, 4, true>(qkv, row_width, out, partial_acc, partial_ml, keys, values, block_tables,
                                          table_width, positions, work, tiles, heads, kv_heads, tokens_per_tile,
                                          page_size, scale, window, splits, fused, stream, change);
  } else if (changed && column_tiles == 2) {
    status = launch_tiles<2, false, 4, true>(qkv, row_width, out, partial_acc, partial_ml, keys, values, block_tables,
                                          table_width, positions, work, tiles, heads, kv_heads, tokens_per_tile,
                                          page_size, scale, window, splits, fused, stream, change);
  } else if (column_tiles == 1) {
    status = launch_tiles<1, false, 4>(qkv, row_width, out, partial_acc, partial_ml, keys, values, block_tables,
                                    table_width, positions, work, tiles, heads, kv_heads, tokens_per_tile, page_size,
                                    scale, window, splits, fused, stream);
  } else if (column_tiles == 2) {
    status = launch_tiles<2, false, 4>(qkv, row_width, out, partial_acc, partial_ml, keys, values, block_tables,
                                    table_width, positions, work, tiles, heads, kv_heads, tokens_per_tile, page_size,
                                    scale, window, splits, fused, stream);
  } else {
    return ERR_BAD_ARGUMENT;
  }
  if (status != 0 || splits == 1 || unmerged) return status;
  if (by_item) {
    hipLaunchKernelGGL(attention_merge_items_kernel, dim3(tiles, heads), dim3(MERGE_THREADS), 0, stream, partial_acc, partial_ml,
                       (bf16_t*)out, work, splits, heads, group, tokens_per_tile);
    return LAUNCH_STATUS();
  }
  return launch_merge(partial_acc, partial_ml, out, splits, (size_t)rows * heads, stream);
}
