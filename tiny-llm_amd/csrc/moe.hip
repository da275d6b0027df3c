// A mixture of small gated feed-forward layers whose experts are looked up in a table by token id (no
// router): every token uses `top` experts with equal weights.  The products here are rows against the
// weights of each row's own expert; the activation between them is the gated unit's kernel.
//
// A row's sums are formed in one fixed order (the lanes of a wave stride over the inner size, then a
// butterfly), whatever else the step holds.  Accumulation is float32 in both precisions.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / TL_WAVE;
constexpr int kCols = 64;                 // output columns a workgroup owns, kCols / kWaves a wave

__device__ __forceinline__ float dot_lanes(const float* __restrict__ a, const float* __restrict__ w, int K, int lane) {
  float acc = 0.f;
  if ((K & 3) == 0 && ((((uintptr_t)a) | ((uintptr_t)w)) & 15) == 0) {
    for (int k = lane * 4; k < K; k += TL_WAVE * 4) {
      const f32x4 x = *(const f32x4*)(a + k), y = *(const f32x4*)(w + k);
      acc = fmaf(x[0], y[0], acc);
      acc = fmaf(x[1], y[1], acc);
      acc = fmaf(x[2], y[2], acc);
      acc = fmaf(x[3], y[3], acc);
    }
  } else {
    for (int k = lane; k < K; k += TL_WAVE) acc = fmaf(a[k], w[k], acc);
  }
  return wave_sum(acc);
}

__device__ __forceinline__ float dot_lanes(const bf16_t* __restrict__ a, const bf16_t* __restrict__ w, int K, int lane) {
  float acc = 0.f;
  if ((K & 7) == 0 && ((((uintptr_t)a) | ((uintptr_t)w)) & 15) == 0) {
    for (int k = lane * 8; k < K; k += TL_WAVE * 8) {
      const bf16x8 x = *(const bf16x8*)(a + k), y = *(const bf16x8*)(w + k);
#pragma unroll
      for (int j = 0; j < 8; ++j) acc = fmaf((float)x[j], (float)y[j], acc);
    }
  } else {
    for (int k = lane; k < K; k += TL_WAVE) acc = fmaf((float)a[k], (float)w[k], acc);
  }
  return wave_sum(acc);
}

__device__ __forceinline__ int expert_of(const int32_t* tokens, const int32_t* table, int t, int j, int top, int vocab,
                                         int experts) {
  int tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  int e = table[(int64_t)tok * top + j];
  return e < 0 ? 0 : (e >= experts ? experts - 1 : e);
}

// out[t * top + j, n] = sum_k a[t, k] * w[e(t, j)][n, k]
template <typename T>
__global__ __launch_bounds__(kThreads) void table_moe_up_kernel(const T* __restrict__ a, int64_t a_stride,
                                                                const T* __restrict__ w,
                                                                const int32_t* __restrict__ tokens,
                                                                const int32_t* __restrict__ table, T* __restrict__ out,
                                                                int top, int experts, int vocab, int N, int K) {
  const int row = blockIdx.x, t = row / top, j = row - t * top;
  const int wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
  const int e = expert_of(tokens, table, t, j, top, vocab, experts);
  const T* arow = a + (int64_t)t * a_stride;
  const T* we = w + (int64_t)e * N * K;
  const int n0 = blockIdx.y * kCols + wave * (kCols / kWaves);
  for (int n = n0; n < min(N, n0 + kCols / kWaves); ++n) {
    const float v = dot_lanes(arow, we + (int64_t)n * K, K, lane);
    if (lane == 0) out[(int64_t)row * N + n] = from_f32<T>(v);
  }
}

// out[t, c] = base[t, c] * base_scale[t] + coef * sum_j sum_k z[t * top + j, k] * w[e(t, j)][c, k]
// (base and base_scale optional; the experts of a token are added in the table's order)
template <typename T>
__global__ __launch_bounds__(kThreads) void table_moe_down_kernel(const T* __restrict__ z, const T* __restrict__ w,
                                                                  const int32_t* __restrict__ tokens,
                                                                  const int32_t* __restrict__ table,
                                                                  const float* __restrict__ base,
                                                                  const float* __restrict__ base_scale,
                                                                  float* __restrict__ out, int top, int experts,
                                                                  int vocab, int N, int K, float coef) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
  const int n0 = blockIdx.y * kCols + wave * (kCols / kWaves);
  const float bsc = base_scale ? base_scale[t] : 1.f;
  for (int n = n0; n < min(N, n0 + kCols / kWaves); ++n) {
    float acc = 0.f;
    for (int j = 0; j < top; ++j) {
      const int e = expert_of(tokens, table, t, j, top, vocab, experts);
      acc += dot_lanes(z + ((int64_t)t * top + j) * K, w + ((int64_t)e * N + n) * K, K, lane);
    }
    if (lane == 0) {
      const float b = base ? base[(int64_t)t * N + n] * bsc : 0.f;
      out[(int64_t)t * N + n] = fmaf(coef, acc, b);
    }
  }
}

// out[t] = sigmoid(a[t, :] . w): one wave a row.
template <typename T>
__global__ __launch_bounds__(TL_WAVE) void row_dot_sigmoid_kernel(const T* __restrict__ a, int64_t a_stride,
                                                                  const T* __restrict__ w, float* __restrict__ out,
                                                                  int K) {
  const float v = dot_lanes(a + (int64_t)blockIdx.x * a_stride, w, K, threadIdx.x);
  if (threadIdx.x == 0) out[blockIdx.x] = 1.f / (1.f + expf(-v));
}

}  // namespace

extern "C" {

// a: [n_tokens, K] (row stride a_stride); w: [experts, N, K]; table: int32 [vocab, top]; out: [n_tokens * top, N].
int tl_table_moe_up(const void* a, int64_t a_stride, const void* w, const int32_t* tokens, const int32_t* table, void* out,
                    int n_tokens, int top, int experts, int vocab, int N, int K, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (top <= 0 || experts <= 0 || vocab <= 0 || N <= 0 || K <= 0 || a_stride < K || !a || !w || !tokens || !table || !out ||
      (int64_t)n_tokens * top > 0x7fffffff || (N + kCols - 1) / kCols > 65535)
    return TL_ERR_ARG;
  dim3 g(n_tokens * top, (N + kCols - 1) / kCols), b(kThreads);
  if (dtype == 0)
    hipLaunchKernelGGL(table_moe_up_kernel<float>, g, b, 0, stream, (const float*)a, a_stride, (const float*)w, tokens,
                       table, (float*)out, top, experts, vocab, N, K);
  else if (dtype == 1)
    hipLaunchKernelGGL(table_moe_up_kernel<bf16_t>, g, b, 0, stream, (const bf16_t*)a, a_stride, (const bf16_t*)w, tokens,
                       table, (bf16_t*)out, top, experts, vocab, N, K);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

// z: [n_tokens * top, K]; w: [experts, N, K]; base: float32 [n_tokens, N] or null; base_scale: float32 [n_tokens] or
// null; out: float32 [n_tokens, N] (may be base).
int tl_table_moe_down(const void* z, const void* w, const int32_t* tokens, const int32_t* table, const float* base,
                      const float* base_scale, float* out, int n_tokens, int top, int experts, int vocab, int N, int K,
                      float coef, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (top <= 0 || experts <= 0 || vocab <= 0 || N <= 0 || K <= 0 || !z || !w || !tokens || !table || !out ||
      (N + kCols - 1) / kCols > 65535)
    return TL_ERR_ARG;
  dim3 g(n_tokens, (N + kCols - 1) / kCols), b(kThreads);
  if (dtype == 0)
    hipLaunchKernelGGL(table_moe_down_kernel<float>, g, b, 0, stream, (const float*)z, (const float*)w, tokens, table,
                       base, base_scale, out, top, experts, vocab, N, K, coef);
  else if (dtype == 1)
    hipLaunchKernelGGL(table_moe_down_kernel<bf16_t>, g, b, 0, stream, (const bf16_t*)z, (const bf16_t*)w, tokens, table,
                       base, base_scale, out, top, experts, vocab, N, K, coef);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

int tl_row_dot_sigmoid(const void* a, int64_t a_stride, const void* w, float* out, int n_rows, int K, int dtype,
                       hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (K <= 0 || a_stride < K || !a || !w || !out) return TL_ERR_ARG;
  dim3 g(n_rows), b(TL_WAVE);
  if (dtype == 0)
    hipLaunchKernelGGL(row_dot_sigmoid_kernel<float>, g, b, 0, stream, (const float*)a, a_stride, (const float*)w, out, K);
  else if (dtype == 1)
    hipLaunchKernelGGL(row_dot_sigmoid_kernel<bf16_t>, g, b, 0, stream, (const bf16_t*)a, a_stride, (const bf16_t*)w, out,
                       K);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

}  // extern "C"
