// Embedding gather, residual add + RMSNorm, rotary position encoding with the cache
// write, SiLU * up, and row gather.  All arithmetic is float32; inputs and outputs are
// bfloat16 or float32 as the template says.
#include "common.h"

// ---------------------------------------------------------------------------- embedding
// out[t, :] = float(table[ids[t], :])        (reference model.py:293)
template <typename T>
__global__ void embedding_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                 float* __restrict__ out, int hidden) {
  const size_t row = (size_t)ids[blockIdx.x];
  const T* src = table + row * hidden;
  float* dst = out + (size_t)blockIdx.x * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(src[i]);
}

extern "C" int llmserve_embedding(const void* table, int table_is_float, const int* ids, float* out,
                                  int tokens, int hidden, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (table_is_float)
    hipLaunchKernelGGL(embedding_kernel<float>, dim3(tokens), dim3(256), 0, stream, (const float*)table, ids, out, hidden);
  else
    hipLaunchKernelGGL(embedding_kernel<bf16_t>, dim3(tokens), dim3(256), 0, stream, (const bf16_t*)table, ids, out, hidden);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- add + RMSNorm
// hidden[t] += delta[0][t] + delta[1][t] + ... (if delta); out[t] = hidden[t] *
// rsqrt(mean(hidden[t]^2) + eps) * weight   (reference model.py:20-23, :200-201).
// `delta` may come as `parts` partial sums [parts, rows, width] (a product split over K leaves
// them); they are added in order.  One block per row; the sum of squares is added in an order
// that depends only on the row length, so a row's result is the same in any batch.
template <typename TO>
__global__ void add_rms_norm_kernel(float* __restrict__ hidden, const float* __restrict__ delta, int parts,
                                    size_t part_stride, const void* __restrict__ weight, int weight_is_float,
                                    TO* __restrict__ out, int width, float eps) {
  __shared__ float shared[17];
  float* row = hidden + (size_t)blockIdx.x * width;
  const float* add = delta ? delta + (size_t)blockIdx.x * width : nullptr;
  float squares = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = row[i];
    if (add) {
      for (int p = 0; p < parts; ++p) v += add[p * part_stride + i];
      row[i] = v;
    }
    squares += v * v;
  }
  const float total = block_sum(squares, shared);
  const float scale = rsqrtf(total / (float)width + eps);
  TO* dst = out + (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x)
    dst[i] = from_float<TO>(row[i] * scale * load_as_float(weight, weight_is_float, i));
}

// The same for rows whose length is a multiple of 4, up to 16,384 floats: the row stays in
// registers between the two passes and moves in 16-byte pieces.  The block has a thread for every
// piece of a row of up to 4,096 floats (PIECES = 1; 2 or 4 pieces a thread beyond), so that all of
// a thread's loads (its piece of the row, of the weight and of every partial sum) are on their way
// before the first is used: on a short row the kernel takes as long as its loads need to come
// back, and a second piece per thread would be a second trip.  Piece j of a thread is quad
// min(threadIdx.x + j * blockDim.x, quads - 1): threads past the end read the last quad again and
// store nothing, so the loads need no branch.
template <int PARTS, int PIECES>
__device__ __forceinline__ void add_parts(float4 (&v)[PIECES], const float* from, size_t part_stride, int quads) {
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int i = min((int)(threadIdx.x + j * blockDim.x), quads - 1);
    float4 d[PARTS];
#pragma unroll
    for (int p = 0; p < PARTS; ++p) d[p] = ((const float4*)(from + (size_t)p * part_stride))[i];
#pragma unroll
    for (int p = 0; p < PARTS; ++p) {
      v[j].x += d[p].x; v[j].y += d[p].y; v[j].z += d[p].z; v[j].w += d[p].w;
    }
  }
}

template <int PIECES>
__device__ __forceinline__ void add_some_parts(float4 (&v)[PIECES], const float* from, int count, size_t part_stride,
                                               int quads) {
  switch (count) {
    case 1: add_parts<1, PIECES>(v, from, part_stride, quads); break;
    case 2: add_parts<2, PIECES>(v, from, part_stride, quads); break;
    case 3: add_parts<3, PIECES>(v, from, part_stride, quads); break;
    case 4: add_parts<4, PIECES>(v, from, part_stride, quads); break;
    case 5: add_parts<5, PIECES>(v, from, part_stride, quads); break;
    case 6: add_parts<6, PIECES>(v, from, part_stride, quads); break;
    case 7: add_parts<7, PIECES>(v, from, part_stride, quads); break;
    default: add_parts<8, PIECES>(v, from, part_stride, quads); break;
  }
}

__device__ __forceinline__ void store_four(float* dst, float a, float b, float c, float d) {
  *(float4*)dst = make_float4(a, b, c, d);
}
__device__ __forceinline__ void store_four(bf16_t* dst, float a, float b, float c, float d) {
  typedef bf16_t bf16x4 __attribute__((ext_vector_type(4)));
  *(bf16x4*)dst = (bf16x4){(bf16_t)a, (bf16_t)b, (bf16_t)c, (bf16_t)d};
}

template <typename TO, int PIECES>
__global__ __launch_bounds__(1024) void add_rms_norm_vector_kernel(float* __restrict__ hidden,
                                                                   const float* __restrict__ delta, int parts,
                                                                   size_t part_stride,
                                                                   const void* __restrict__ weight,
                                                                   int weight_is_float, TO* __restrict__ out,
                                                                   int width, float eps) {
  __shared__ float shared[17];
  const int quads = width / 4;
  float4* row = (float4*)(hidden + (size_t)blockIdx.x * width);
  const float* add = delta ? delta + (size_t)blockIdx.x * width : nullptr;
  float4 v[PIECES], wide[PIECES];
  uint2 narrow[PIECES];  // four bfloat16 weights as they lie in memory: converted after the loads
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int i = min((int)(threadIdx.x + j * blockDim.x), quads - 1);
    v[j] = row[i];
    if (weight_is_float)
      wide[j] = ((const float4*)weight)[i];
    else
      narrow[j] = ((const uint2*)weight)[i];
  }
  if (add) {
    // the parts are added in order, up to eight at a time: their loads are all requested before the
    // first is used (the first eight outside the loop, so that they need not wait for the row's piece)
    add_some_parts<PIECES>(v, add, min(parts, 8), part_stride, quads);
    for (int first = 8; first < parts; first += 8)
      add_some_parts<PIECES>(v, add + (size_t)first * part_stride, min(parts - first, 8), part_stride, quads);
  }
  float squares = 0.f;
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int i = threadIdx.x + j * blockDim.x;
    if (i < quads) {
      if (add) row[i] = v[j];
      squares += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
    }
  }
  const float total = block_sum(squares, shared);
  const float scale = rsqrtf(total / (float)width + eps);
  TO* dst = out + (size_t)blockIdx.x * width;
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int i = threadIdx.x + j * blockDim.x;
    if (i < quads) {
      float4 w = wide[j];
      if (!weight_is_float)  // a bfloat16 is the upper half of the float32 of the same value
        w = make_float4(__uint_as_float(narrow[j].x << 16), __uint_as_float(narrow[j].x & 0xffff0000u),
                        __uint_as_float(narrow[j].y << 16), __uint_as_float(narrow[j].y & 0xffff0000u));
      store_four(dst + 4 * i, v[j].x * scale * w.x, v[j].y * scale * w.y, v[j].z * scale * w.z, v[j].w * scale * w.w);
    }
  }
}

template <typename TO>
static void launch_add_rms_norm_vector(float* hidden, const float* delta, int parts, size_t part_stride,
                                       const void* weight, int weight_is_float, TO* out, int rows, int width,
                                       float eps, hipStream_t stream) {
  // a thread for every four floats of the row, in whole waves: the block size depends on the width alone
  const int quads = width / 4;
  const int pieces = quads <= 1024 ? 1 : quads <= 2048 ? 2 : 4;
  const int threads = ((quads + pieces - 1) / pieces + WAVE - 1) / WAVE * WAVE;
  if (pieces == 1)
    hipLaunchKernelGGL((add_rms_norm_vector_kernel<TO, 1>), dim3(rows), dim3(threads), 0, stream, hidden, delta, parts,
                       part_stride, weight, weight_is_float, out, width, eps);
  else if (pieces == 2)
    hipLaunchKernelGGL((add_rms_norm_vector_kernel<TO, 2>), dim3(rows), dim3(threads), 0, stream, hidden, delta, parts,
                       part_stride, weight, weight_is_float, out, width, eps);
  else
    hipLaunchKernelGGL((add_rms_norm_vector_kernel<TO, 4>), dim3(rows), dim3(threads), 0, stream, hidden, delta, parts,
                       part_stride, weight, weight_is_float, out, width, eps);
}

extern "C" int llmserve_add_rms_norm(float* hidden, const float* delta, int parts, const void* weight,
                                     int weight_is_float, void* out, int out_is_float, int rows, int width, float eps,
                                     hipStream_t stream) {
  if (rows <= 0) return 0;
  if (delta && parts < 1) return ERR_BAD_ARGUMENT;
  const size_t part_stride = (size_t)rows * width;
  if (width % 4 == 0 && width <= 1024 * 4 * 4) {
    if (out_is_float)
      launch_add_rms_norm_vector<float>(hidden, delta, parts, part_stride, weight, weight_is_float, (float*)out, rows,
                                        width, eps, stream);
    else
      launch_add_rms_norm_vector<bf16_t>(hidden, delta, parts, part_stride, weight, weight_is_float, (bf16_t*)out,
                                         rows, width, eps, stream);
    return LAUNCH_STATUS();
  }
  const int threads = width >= 2048 ? 512 : 256;
  if (out_is_float)
    hipLaunchKernelGGL(add_rms_norm_kernel<float>, dim3(rows), dim3(threads), 0, stream, hidden, delta, parts,
                       part_stride, weight, weight_is_float, (float*)out, width, eps);
  else
    hipLaunchKernelGGL(add_rms_norm_kernel<bf16_t>, dim3(rows), dim3(threads), 0, stream, hidden, delta, parts,
                       part_stride, weight, weight_is_float, (bf16_t*)out, width, eps);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- rotary + cache write
// table[t][j] = (cos, sin) of positions[t] * inverse[j], in float32 (reference model.py:29-33
// builds the same numbers for every position at start-up).  Every layer of a step rotates by the
// same angles, so they are computed once per step.
__global__ void rotary_table_kernel(const int* __restrict__ positions, const float* __restrict__ inverse,
                                    float2* __restrict__ table, int half) {
  const float position = (float)positions[blockIdx.x];
  for (int j = threadIdx.x; j < half; j += blockDim.x) {
    float sine, cosine;
    sincosf(position * inverse[j], &sine, &cosine);
    table[(size_t)blockIdx.x * half + j] = make_float2(cosine, sine);
  }
}

extern "C" int llmserve_rotary_table(const int* positions, const float* inverse, float* table, int tokens, int half,
                                     hipStream_t stream) {
  if (tokens <= 0) return 0;
  hipLaunchKernelGGL(rotary_table_kernel, dim3(tokens), dim3(64), 0, stream, positions, inverse, (float2*)table, half);
  return LAUNCH_STATUS();
}

// A token's row of qkv is [q heads | k heads | v heads], each head `dim` wide.  q and k heads
// are rotated in place by the token's angles (reference model.py:35-43): the pair (a, b)
// becomes (a cos - b sin, b cos + a sin), all in float32.
// pairing 0: none, 1: adjacent pairs (2j, 2j+1), 2: half pairs (j, j + dim/2).
// k (after rotation) and v are then written to the pages: slot = page * page_size + offset,
// key pages laid out [page, kv_head, dim / 8, offset, 8] (common.h: key_element), value pages
// transposed in pieces of eight keys, [page, kv_head, page_size / 8, dim, 8] (common.h: value_element;
// reference kv_cache.py:249-266 writes both as [page, offset, kv_head, dim]).
// slots may be null (nothing is stored); a negative slot skips the token.
template <typename T>
__global__ void rotate_and_store_kernel(T* __restrict__ qkv, const float2* __restrict__ table, int pairing, int heads,
                                        int kv_heads, int dim, T* __restrict__ keys, T* __restrict__ values,
                                        const int* __restrict__ slots, int page_size) {
  const int token = blockIdx.x;
  const int half = dim / 2;
  T* row = qkv + (size_t)token * (heads + 2 * kv_heads) * dim;
  if (pairing != 0) {
    const float2* angles = table + (size_t)token * half;
    const int pairs = (heads + kv_heads) * half;
    for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
      const int head = i / half, j = i % half;
      const float2 cs = angles[j];
      T* h = row + head * dim;
      const int ia = pairing == 1 ? 2 * j : j;
      const int ib = pairing == 1 ? 2 * j + 1 : j + half;
      const float a = to_float(h[ia]), b = to_float(h[ib]);
      h[ia] = from_float<T>(a * cs.x - b * cs.y);
      h[ib] = from_float<T>(b * cs.x + a * cs.y);
    }
  }
  if (slots == nullptr) return;
  const int slot = slots[token];
  if (slot < 0) return;
  __syncthreads();  // the rotated k is read back below by other threads
  const int page = slot / page_size, offset = slot % page_size;
  const T* k_row = row + heads * dim;
  const T* v_row = k_row + kv_heads * dim;
  for (int i = threadIdx.x; i < kv_heads * dim; i += blockDim.x) {
    const int head = i / dim, d = i % dim;
    const size_t block = ((size_t)page * kv_heads + head) * page_size * dim;
    keys[block + key_element(d, offset, page_size, dim)] = k_row[i];
    values[block + value_element(d, offset, page_size, dim)] = v_row[i];
  }
}

// The same for bfloat16 heads whose size is a multiple of 16, in 16-byte pieces: a thread takes 16
// elements of a q or k head (two pieces that hold eight pairs: with adjacent pairs elements 16p ..
// 16p + 15, with half pairs 8p .. 8p + 7 and their partners dim/2 on), rotates them, writes them
// back, and, for a k head, writes them to the page as well; further threads take eight elements of
// a v head each.  Threads are dealt to (token, piece) pairs without regard to blocks.
__global__ __launch_bounds__(256) void rotate_and_store_vector_kernel(
    bf16_t* __restrict__ qkv, const float2* __restrict__ table, int pairing, int heads, int kv_heads, int dim,
    bf16_t* __restrict__ keys, bf16_t* __restrict__ values, const int* __restrict__ slots, int page_size, int tokens) {
  typedef bf16_t bf16x8 __attribute__((ext_vector_type(8)));
  typedef bf16_t bf16x4 __attribute__((ext_vector_type(4)));
  const int per_head = dim / 16, half = dim / 2;
  const int rotated = (heads + kv_heads) * per_head;
  const size_t id = (size_t)blockIdx.x * 256 + threadIdx.x, rotating = (size_t)tokens * rotated;
  const int row_width = (heads + 2 * kv_heads) * dim;
  if (id >= rotating) {
    // The values.  A page keeps them transposed in pieces of eight keys (attention sums over keys), so a
    // token's value row is `dim` two-byte stores 16 bytes apart.  A thread therefore takes four dims of eight
    // tokens in a row: its loads are 8 bytes beside its neighbours', and where the eight tokens are one piece
    // of a page (a prompt's portion) it stores 16 bytes a dim, 64 bytes in a row.
    if (slots == nullptr) return;
    const int quads = dim / 4;
    const size_t unit = id - rotating;
    const int quad = (int)(unit % quads), head = (int)(unit / quads % kv_heads);
    const size_t octet = unit / quads / kv_heads;
    if (octet * 8 >= (size_t)tokens) return;
    const int first = (int)octet * 8, count = min(8, tokens - first);
    int slot[8];
    bf16x4 v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int token = first + min(i, count - 1);
      slot[i] = i < count ? slots[token] : -1;
      v[i] = *(const bf16x4*)(qkv + (size_t)token * row_width + (size_t)(heads + kv_heads + head) * dim + quad * 4);
    }
    bool together = count == 8 && slot[0] >= 0 && slot[0] % 8 == 0 && page_size % 8 == 0;
#pragma unroll
    for (int i = 1; i < 8; ++i) together = together && slot[i] == slot[0] + i;
    if (together) {
      bf16_t* v_page = values + ((size_t)(slot[0] / page_size) * kv_heads + head) * page_size * dim;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bf16x8 run = {v[0][e], v[1][e], v[2][e], v[3][e], v[4][e], v[5][e], v[6][e], v[7][e]};
        *(bf16x8*)(v_page + value_element(quad * 4 + e, slot[0] % page_size, page_size, dim)) = run;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (slot[i] < 0) continue;
        bf16_t* v_page = values + ((size_t)(slot[i] / page_size) * kv_heads + head) * page_size * dim;
#pragma unroll
        for (int e = 0; e < 4; ++e) v_page[value_element(quad * 4 + e, slot[i] % page_size, page_size, dim)] = v[i][e];
      }
    }
    return;
  }
  const int token = (int)(id / rotated), piece = (int)(id % rotated);
  bf16_t* row = qkv + (size_t)token * row_width;
  const int slot = slots ? slots[token] : -1;
  const int head = piece / per_head, p = piece % per_head;
  bf16_t* h = row + head * dim;
  const int ia = pairing == 2 ? 8 * p : 16 * p, ib = pairing == 2 ? 8 * p + half : 16 * p + 8;
  bf16x8 a = *(const bf16x8*)(h + ia), b = *(const bf16x8*)(h + ib);
  if (pairing != 0) {
    float2 cs[8];
    const float2* angles = table + (size_t)token * half + 8 * p;
#pragma unroll
    for (int i = 0; i < 8; ++i) cs[i] = angles[i];
    if (pairing == 2) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float x = (float)a[i], y = (float)b[i];
        a[i] = (bf16_t)(x * cs[i].x - y * cs[i].y);
        b[i] = (bf16_t)(y * cs[i].x + x * cs[i].y);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float x = (float)a[2 * i], y = (float)a[2 * i + 1];
        a[2 * i] = (bf16_t)(x * cs[i].x - y * cs[i].y);
        a[2 * i + 1] = (bf16_t)(y * cs[i].x + x * cs[i].y);
        const float u = (float)b[2 * i], v = (float)b[2 * i + 1];
        b[2 * i] = (bf16_t)(u * cs[4 + i].x - v * cs[4 + i].y);
        b[2 * i + 1] = (bf16_t)(v * cs[4 + i].x + u * cs[4 + i].y);
      }
    }
    *(bf16x8*)(h + ia) = a;
    *(bf16x8*)(h + ib) = b;
  }
  if (head >= heads && slot >= 0) {
    // pieces ia / 8 and ib / 8 of the key at this slot (dim is a multiple of 16 here)
    bf16_t* k_block = keys + ((size_t)(slot / page_size) * kv_heads + (head - heads)) * page_size * dim;
    const int offset = slot % page_size;
    *(bf16x8*)(k_block + ((size_t)(ia / KEY_PIECE) * page_size + offset) * KEY_PIECE) = a;
    *(bf16x8*)(k_block + ((size_t)(ib / KEY_PIECE) * page_size + offset) * KEY_PIECE) = b;
  }
}

extern "C" int llmserve_rotate_and_store(void* qkv, int is_float, const float* table, int pairing, int tokens,
                                         int heads, int kv_heads, int dim, void* keys, void* values,
                                         const int* slots, int page_size, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (dim % 2 || (pairing != 0 && table == nullptr) || pairing < 0 || pairing > 2) return ERR_BAD_ARGUMENT;
  if (!is_float && dim % 16 == 0) {
    // a thread for every 16 elements of a token's q and k heads, then one for every four dims of eight tokens' values
    const size_t threads = (size_t)tokens * (heads + kv_heads) * (dim / 16) +
                           (slots ? (size_t)((tokens + 7) / 8) * kv_heads * (dim / 4) : 0);
    hipLaunchKernelGGL(rotate_and_store_vector_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream,
                       (bf16_t*)qkv, (const float2*)table, pairing, heads, kv_heads, dim, (bf16_t*)keys,
                       (bf16_t*)values, slots, page_size, tokens);
    return LAUNCH_STATUS();
  }
  if (is_float)
    hipLaunchKernelGGL(rotate_and_store_kernel<float>, dim3(tokens), dim3(256), 0, stream, (float*)qkv,
                       (const float2*)table, pairing, heads, kv_heads, dim, (float*)keys, (float*)values, slots,
                       page_size);
  else
    hipLaunchKernelGGL(rotate_and_store_kernel<bf16_t>, dim3(tokens), dim3(256), 0, stream, (bf16_t*)qkv,
                       (const float2*)table, pairing, heads, kv_heads, dim, (bf16_t*)keys, (bf16_t*)values, slots,
                       page_size);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- act(gate) * up
// in: [rows, 2 * width] float32 or bfloat16 with gate_j at column 2j and up_j at column 2j + 1 (the
// product that made it had its weight rows interleaved); out: [rows, width].
// The activation is a parameter: 0 silu(z) = z * sigmoid(z) (reference model.py:188), 1 gelu (the exact one,
// z * Phi(z)), 2 gelu with tanh, 3 relu.  The products' fused epilogues know silu alone; a feed-forward with
// another gate activation runs its product plain and this kernel behind it.
#define ACT_SILU 0
#define ACT_GELU 1
#define ACT_GELU_TANH 2
#define ACT_RELU 3

__device__ __forceinline__ float gate_activation(int activation, float z) {
  switch (activation) {
    case ACT_GELU: return 0.5f * z * (1.f + erff(z * 0.70710678118654752f));
    case ACT_GELU_TANH: return 0.5f * z * (1.f + tanhf(0.79788456080286536f * (z + 0.044715f * z * z * z)));
    case ACT_RELU: return fmaxf(z, 0.f);
    default: return z / (1.f + expf(-z));
  }
}

template <typename TI, typename TO>
__global__ void gate_mul_kernel(const TI* __restrict__ in, TO* __restrict__ out, int width, int activation) {
  const TI* row = in + (size_t)blockIdx.x * 2 * width;
  TO* dst = out + (size_t)blockIdx.x * width;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < width; i += gridDim.y * blockDim.x) {
    const float gate = to_float(row[2 * i]), up = to_float(row[2 * i + 1]);
    dst[i] = from_float<TO>(gate_activation(activation, gate) * up);
  }
}

// SiLU for bfloat16 rows whose width is a multiple of 8: a thread takes eight outputs, 32 bytes in
// (two 16-byte loads, both on their way before the first is used) and 16 bytes out.
__global__ __launch_bounds__(256) void silu_mul_vector_kernel(const bf16_t* __restrict__ in, bf16_t* __restrict__ out,
                                                              size_t octets) {
  typedef bf16_t bf16x8 __attribute__((ext_vector_type(8)));
  const size_t at = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (at >= octets) return;
  const bf16x8 first = ((const bf16x8*)in)[2 * at], second = ((const bf16x8*)in)[2 * at + 1];
  bf16x8 result;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float gate = (float)first[2 * i], up = (float)first[2 * i + 1];
    result[i] = (bf16_t)(gate / (1.f + expf(-gate)) * up);
    const float gate2 = (float)second[2 * i], up2 = (float)second[2 * i + 1];
    result[4 + i] = (bf16_t)(gate2 / (1.f + expf(-gate2)) * up2);
  }
  ((bf16x8*)out)[at] = result;
}

extern "C" int llmserve_gate_mul(const void* in, int in_is_float, void* out, int out_is_float, int rows, int width,
                                 int activation, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (activation < ACT_SILU || activation > ACT_RELU) return ERR_BAD_ARGUMENT;
  if (activation == ACT_SILU && !in_is_float && !out_is_float && width % 8 == 0) {  // rows are contiguous: one run of octets
    const size_t octets = (size_t)rows * (width / 8);
    hipLaunchKernelGGL(silu_mul_vector_kernel, dim3((unsigned)((octets + 255) / 256)), dim3(256), 0, stream,
                       (const bf16_t*)in, (bf16_t*)out, octets);
    return LAUNCH_STATUS();
  }
  // a row is cut over several blocks when the rows alone would not fill the chip
  const int pieces = rows >= 1024 ? 1 : max(1, min((width + 255) / 256, 1024 / rows));
  const dim3 grid(rows, pieces), block(256);
  if (in_is_float && out_is_float)
    hipLaunchKernelGGL((gate_mul_kernel<float, float>), grid, block, 0, stream, (const float*)in, (float*)out, width, activation);
  else if (in_is_float)
    hipLaunchKernelGGL((gate_mul_kernel<float, bf16_t>), grid, block, 0, stream, (const float*)in, (bf16_t*)out, width, activation);
  else if (out_is_float)
    hipLaunchKernelGGL((gate_mul_kernel<bf16_t, float>), grid, block, 0, stream, (const bf16_t*)in, (float*)out, width, activation);
  else
    hipLaunchKernelGGL((gate_mul_kernel<bf16_t, bf16_t>), grid, block, 0, stream, (const bf16_t*)in, (bf16_t*)out, width, activation);
  return LAUNCH_STATUS();
}

extern "C" int llmserve_silu_mul(const void* in, int in_is_float, void* out, int out_is_float, int rows, int width,
                                 hipStream_t stream) {
  return llmserve_gate_mul(in, in_is_float, out, out_is_float, rows, width, ACT_SILU, stream);
}

// ---------------------------------------------------------------------------- gather rows
// out[r] = hidden[rows[r]] (+ delta[0][rows[r]] + delta[1][rows[r]] + ...)
__global__ void gather_rows_kernel(const float* __restrict__ hidden, const float* __restrict__ delta, int parts,
                                   size_t part_stride, const int* __restrict__ rows, float* __restrict__ out,
                                   int width) {
  const size_t src = (size_t)rows[blockIdx.x] * width;
  float* dst = out + (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = hidden[src + i];
    if (delta) {
      for (int first = 0; first < parts; first += 8) {  // eight loads in flight, added in order
        float d[8];
#pragma unroll
        for (int p = 0; p < 8; ++p) d[p] = first + p < parts ? delta[(size_t)(first + p) * part_stride + src + i] : 0.f;
#pragma unroll
        for (int p = 0; p < 8; ++p) v += d[p];
      }
    }
    dst[i] = v;
  }
}

extern "C" int llmserve_gather_rows(const float* hidden, const float* delta, int parts, int total_rows,
                                    const int* rows, float* out, int count, int width, hipStream_t stream) {
  if (count <= 0) return 0;
  hipLaunchKernelGGL(gather_rows_kernel, dim3(count), dim3(256), 0, stream, hidden, delta, parts,
                     (size_t)total_rows * width, rows, out, width);
  return LAUNCH_STATUS();
}
