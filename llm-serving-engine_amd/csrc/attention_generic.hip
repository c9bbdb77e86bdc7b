// Paged attention for any head size, in float32 arithmetic on float32 or bfloat16 pages.
// One block per (token, query head): the token's query attends to the cached keys of its
// request at positions (p - window, p], read through the request's block table, with an
// online softmax over tiles of 128 keys (reference model.py:140-175, the same recurrence per
// page).  It serves prompt portions and single decoded tokens alike: what differs between
// them is only how many tokens of a request are in the step.  This is the true 32-bit path
// and the path for head sizes without an MFMA kernel.
// Two things may change a score before the softmax, for position encodings and models that want
// them (the reference has neither): `soft_cap` > 0 squashes it to cap * tanh(score / cap), and
// `slopes` (one per query head) then adds -slope * (query position - key position), a bias that
// grows with distance.
#include "common.h"

#define KEYS_PER_TILE 128
#define MAX_DIM 512

template <typename T>
__global__ __launch_bounds__(KEYS_PER_TILE) void attention_generic_kernel(
    const T* __restrict__ qkv, int row_width, T* __restrict__ out, const T* __restrict__ keys,
    const T* __restrict__ values, const int* __restrict__ block_tables, int table_width,
    const int* __restrict__ token_sequence, const int* __restrict__ positions, int heads, int kv_heads, int dim,
    int page_size, float scale, int window, const float* __restrict__ slopes, float soft_cap) {
  __shared__ float query[MAX_DIM];
  __shared__ float weights[KEYS_PER_TILE];
  __shared__ float shared[17];
  const int token = blockIdx.x, head = blockIdx.y;
  const int kv_head = head / (heads / kv_heads);
  const int position = positions[token];
  const int* table = block_tables + (size_t)token_sequence[token] * table_width;
  const T* q = qkv + (size_t)token * row_width + head * dim;
  for (int d = threadIdx.x; d < dim; d += blockDim.x) query[d] = to_float(q[d]) * scale;
  __syncthreads();

  const int first = window > 0 ? max(0, position - window + 1) : 0;
  const float slope = slopes ? slopes[head] : 0.f;
  const int width = key_piece_width(dim);
  const int per_thread = (dim + KEYS_PER_TILE - 1) / KEYS_PER_TILE;  // output dims per thread, <= 4
  float acc[MAX_DIM / KEYS_PER_TILE] = {};
  float running_max = -INFINITY, running_sum = 0.f;

  for (int tile = first; tile <= position; tile += KEYS_PER_TILE) {
    const int key = tile + threadIdx.x;
    float score = -INFINITY;
    if (key <= position) {
      const int page = table[key / page_size];
      // the key's pieces lie page_size * width apart (common.h: key_element)
      const T* k = keys + ((size_t)page * kv_heads + kv_head) * page_size * dim + (size_t)(key % page_size) * width;
      float dot = 0.f;
      for (int piece = 0; piece < dim / width; ++piece) {
        const T* part = k + (size_t)piece * page_size * width;
        for (int e = 0; e < width; ++e) dot = fmaf(query[piece * width + e], to_float(part[e]), dot);
      }
      score = dot;
      if (soft_cap > 0.f) score = soft_cap * tanhf(score / soft_cap);
      score -= slope * (float)(position - key);
    }
    const float tile_max = block_max(score, shared);
    const float next_max = fmaxf(running_max, tile_max);
    const float correction = expf(running_max - next_max);  // 0 on the first tile
    const float weight = key <= position ? expf(score - next_max) : 0.f;
    weights[threadIdx.x] = weight;
    const float tile_sum = block_sum(weight, shared);  // also orders the writes to `weights`
    running_sum = running_sum * correction + tile_sum;
    running_max = next_max;
    const int in_tile = min(KEYS_PER_TILE, position - tile + 1);
    for (int i = 0; i < per_thread; ++i) {
      const int d = threadIdx.x + i * KEYS_PER_TILE;
      if (d >= dim) break;
      float sum = 0.f;
      for (int j = 0; j < in_tile; ++j) {
        const int at = tile + j;
        const int page = table[at / page_size];
        const T* v = values + ((size_t)page * kv_heads + kv_head) * page_size * dim;
        sum = fmaf(weights[j], to_float(v[value_element(d, at % page_size, page_size, dim)]), sum);  // common.h: value_element
      }
      acc[i] = acc[i] * correction + sum;
    }
    __syncthreads();
  }
  T* o = out + ((size_t)token * heads + head) * dim;
  for (int i = 0; i < per_thread; ++i) {
    const int d = threadIdx.x + i * KEYS_PER_TILE;
    if (d < dim) o[d] = from_float<T>(acc[i] / running_sum);
  }
}

extern "C" int llmserve_attention_generic(const void* qkv, int row_width, void* out, int is_float, const void* keys,
                                          const void* values, const int* block_tables, int table_width,
                                          const int* token_sequence, const int* positions, int tokens, int heads,
                                          int kv_heads, int dim, int page_size, float scale, int window,
                                          const float* slopes, float soft_cap, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (dim > MAX_DIM || dim <= 0 || heads % kv_heads || page_size <= 0) return ERR_BAD_ARGUMENT;
  dim3 grid(tokens, heads);
  if (is_float)
    hipLaunchKernelGGL(attention_generic_kernel<float>, grid, dim3(KEYS_PER_TILE), 0, stream, (const float*)qkv,
                       row_width, (float*)out, (const float*)keys, (const float*)values, block_tables, table_width,
                       token_sequence, positions, heads, kv_heads, dim, page_size, scale, window, slopes, soft_cap);
  else
    hipLaunchKernelGGL(attention_generic_kernel<bf16_t>, grid, dim3(KEYS_PER_TILE), 0, stream, (const bf16_t*)qkv,
                       row_width, (bf16_t*)out, (const bf16_t*)keys, (const bf16_t*)values, block_tables, table_width,
                       token_sequence, positions, heads, kv_heads, dim, page_size, scale, window, slopes, soft_cap);
  return LAUNCH_STATUS();
}
