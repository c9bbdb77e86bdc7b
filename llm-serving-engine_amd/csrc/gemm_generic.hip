// out[M, N] = x[M, K] . w[N, K]^T + bias[N], float32 multiply-add for any mix of float32
// and bfloat16 operands.  This is the true 32-bit path of every product in the model and the
// fallback for operand types the MFMA kernels do not take.  Each output element adds its K
// products in index order, whatever M is, so a row's result does not depend on the batch.
#include "common.h"

#define TILE 64
#define TILE_K 16

template <typename TX, typename TW, typename TO>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TX* __restrict__ x, const TW* __restrict__ w,
                                                           const void* __restrict__ bias, int bias_is_float,
                                                           TO* __restrict__ out, int M, int N, int K) {
  __shared__ float xs[TILE_K][TILE + 1];
  __shared__ float ws[TILE_K][TILE + 1];
  const int row0 = blockIdx.y * TILE, col0 = blockIdx.x * TILE;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;  // 16 x 16 threads, 4 x 4 outputs each
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += TILE_K) {
    // 64 rows x 16 k values of each operand: 1024 elements, 4 per thread
    for (int i = threadIdx.x; i < TILE * TILE_K; i += 256) {
      const int r = i / TILE_K, k = i % TILE_K;
      const bool in_k = k0 + k < K;
      xs[k][r] = (in_k && row0 + r < M) ? to_float(x[(size_t)(row0 + r) * K + k0 + k]) : 0.f;
      ws[k][r] = (in_k && col0 + r < N) ? to_float(w[(size_t)(col0 + r) * K + k0 + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TILE_K; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + ty * 4 + i;
    if (r >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = col0 + tx * 4 + j;
      if (c >= N) continue;
      float v = acc[i][j];
      if (bias) v += load_as_float(bias, bias_is_float, c);
      out[(size_t)r * N + c] = from_float<TO>(v);
    }
  }
}

template <typename TX, typename TW, typename TO>
static int launch(const void* x, const void* w, const void* bias, int bias_is_float, void* out, int M, int N, int K,
                  hipStream_t stream) {
  dim3 grid((N + TILE - 1) / TILE, (M + TILE - 1) / TILE);
  hipLaunchKernelGGL((gemm_generic_kernel<TX, TW, TO>), grid, dim3(256), 0, stream, (const TX*)x, (const TW*)w, bias,
                     bias_is_float, (TO*)out, M, N, K);
  return LAUNCH_STATUS();
}

template <typename TX, typename TW>
static int pick_out(int out_is_float, const void* x, const void* w, const void* bias, int bias_is_float, void* out,
                    int M, int N, int K, hipStream_t stream) {
  return out_is_float ? launch<TX, TW, float>(x, w, bias, bias_is_float, out, M, N, K, stream)
                      : launch<TX, TW, bf16_t>(x, w, bias, bias_is_float, out, M, N, K, stream);
}

extern "C" int llmserve_gemm_generic(const void* x, int x_is_float, const void* w, int w_is_float, const void* bias,
                                     int bias_is_float, void* out, int out_is_float, int M, int N, int K,
                                     hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) return ERR_BAD_ARGUMENT;
  if (x_is_float && w_is_float) return pick_out<float, float>(out_is_float, x, w, bias, bias_is_float, out, M, N, K, stream);
  if (x_is_float) return pick_out<float, bf16_t>(out_is_float, x, w, bias, bias_is_float, out, M, N, K, stream);
  if (w_is_float) return pick_out<bf16_t, float>(out_is_float, x, w, bias, bias_is_float, out, M, N, K, stream);
  return pick_out<bf16_t, bf16_t>(out_is_float, x, w, bias, bias_is_float, out, M, N, K, stream);
}
