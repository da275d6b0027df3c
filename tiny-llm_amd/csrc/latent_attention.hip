// Attention over a cache of latent vectors: per token the cache holds one normed latent c
// [kv_rank] and one rotated key part kr [rot] that all heads share.  A head's unrotated key is
// W_uk c and its value W_uv c; neither is ever formed.  With q' = W_uk^T q_unrotated the score is
// (q' . c + q_rot . kr) * scale, and the head's output is W_uv (sum_j p_j c_j): the kernel works on
// [q' | q_rot] against [c | kr] and returns sum_j p_j c_j; the two small products per head run
// outside.  Scores, softmax and the weighted sum are float32 whatever the cache's element type.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / TL_WAVE;
constexpr int kMaxRank = 512;                 // latent size the attention kernel takes
constexpr int kRPL = kMaxRank / TL_WAVE;      // latent dims per lane
constexpr int kMaxQ = 1024;                   // kv_rank + rot

// One workgroup per token.  Row t of `d` holds the down projections side by side:
// [q latent (q_rank) at q_off | kv latent (kv_rank) then the shared key part (rot) at kv_off].
// cq[t] = w_q * rms_unit(q latent); if the layer keeps a cache of its own (kv_rank > 0):
// latent[slot] = w_kv * rms_unit(kv latent), rope[slot] = the key part rotated by the angle
// table's row positions[t] (its first `rdims` dims, pair i with i + rdims/2).  A negative slot stores nothing.
template <typename T>
__global__ void latent_prepare_kernel(const T* __restrict__ d, int64_t d_stride, int q_off, int q_rank, int kv_off,
                                      int kv_rank, int rot, int rdims, const float* __restrict__ w_q,
                                      const float* __restrict__ w_kv, float eps, const int32_t* __restrict__ positions,
                                      const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                      const int32_t* __restrict__ slot_mapping, T* __restrict__ cq,
                                      T* __restrict__ latent, T* __restrict__ rope) {
  __shared__ float red[kWaves];
  const int t = blockIdx.x;
  const T* row = d + (int64_t)t * d_stride;
  float ss = 0.f;
  for (int j = threadIdx.x; j < q_rank; j += kThreads) {
    const float v = to_f32(row[q_off + j]);
    ss += v * v;
  }
  ss = block_sum<kWaves>(ss, red);
  float r = 1.f / sqrtf(ss / (float)q_rank + eps);
  for (int j = threadIdx.x; j < q_rank; j += kThreads)
    cq[(int64_t)t * q_rank + j] = from_f32<T>(to_f32(row[q_off + j]) * r * w_q[j]);
  if (kv_rank <= 0) return;
  const int slot = slot_mapping[t];
  ss = 0.f;
  for (int j = threadIdx.x; j < kv_rank; j += kThreads) {
    const float v = to_f32(row[kv_off + j]);
    ss += v * v;
  }
  ss = block_sum<kWaves>(ss, red);
  if (slot < 0) return;
  r = 1.f / sqrtf(ss / (float)kv_rank + eps);
  for (int j = threadIdx.x; j < kv_rank; j += kThreads)
    latent[(int64_t)slot * kv_rank + j] = from_f32<T>(to_f32(row[kv_off + j]) * r * w_kv[j]);
  const int half = rdims / 2;
  const int pos = positions[t];
  for (int i = threadIdx.x; i < half; i += kThreads) {
    const float c = cos_t[(int64_t)pos * half + i], s = sin_t[(int64_t)pos * half + i];
    const float u = to_f32(row[kv_off + kv_rank + i]), v = to_f32(row[kv_off + kv_rank + half + i]);
    rope[(int64_t)slot * rot + i] = from_f32<T>(u * c - v * s);
    rope[(int64_t)slot * rot + half + i] = from_f32<T>(v * c + u * s);
  }
  for (int i = rdims + threadIdx.x; i < rot; i += kThreads)       // dims beyond the rotated ones pass unchanged
    rope[(int64_t)slot * rot + i] = row[kv_off + kv_rank + i];
}

// out[t, h, out_off + i] (float32) = the `rot` dims at in_off of head h of row t, the first `rdims`
// of them rotated by the angle table's row positions[t] (pair i with i + rdims/2).
template <typename T>
__global__ void rotate_into_kernel(const T* __restrict__ q, int64_t q_stride, int head_width, int in_off, int rot,
                                   int rdims, int heads, const int32_t* __restrict__ positions, const float* __restrict__ cos_t,
                                   const float* __restrict__ sin_t, float* __restrict__ out, int out_width,
                                   int out_off) {
  const int t = blockIdx.x;
  const int half = rdims / 2, rest = rot - rdims, per_head = half + rest;
  const int pos = positions[t];
  for (int e = threadIdx.x; e < heads * per_head; e += kThreads) {
    const int h = e / per_head, i = e - h * per_head;
    const T* src = q + (int64_t)t * q_stride + (int64_t)h * head_width + in_off;
    float* dst = out + ((int64_t)t * heads + h) * out_width + out_off;
    if (i >= half) {
      dst[rdims + i - half] = to_f32(src[rdims + i - half]);
      continue;
    }
    const float c = cos_t[(int64_t)pos * half + i], s = sin_t[(int64_t)pos * half + i];
    const float u = to_f32(src[i]), v = to_f32(src[half + i]);
    dst[i] = u * c - v * s;
    dst[half + i] = v * c + u * s;
  }
}

// One wave64 per (token, head).  Lanes split the keys of a 64-key tile for the scores and the
// latent's dims for the weighted sum.  The result is multiplied by sigmoid(gate[t, h]) (optional).
template <typename T>
__global__ __launch_bounds__(TL_WAVE) void latent_attention_kernel(
    const float* __restrict__ qa, const T* __restrict__ latent, const T* __restrict__ rope,
    const int32_t* __restrict__ block_tables, int max_blocks, const int32_t* __restrict__ req_of_token,
    const int32_t* __restrict__ positions, const T* __restrict__ gate, int64_t gate_stride, T* __restrict__ out,
    int heads, int kv_rank, int rot, int block_size, float scale) {
  __shared__ float qs[kMaxQ];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int r = req_of_token[t];
  const int kv_end = positions[t] + 1;
  const int32_t* bt = block_tables + (int64_t)r * max_blocks;
  const int width = kv_rank + rot;
  const float* qrow = qa + ((int64_t)t * heads + h) * width;
  for (int dd = lane; dd < width; dd += TL_WAVE) qs[dd] = qrow[dd];
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float o[kRPL];
#pragma unroll
  for (int i = 0; i < kRPL; ++i) o[i] = 0.f;

  for (int base = 0; base < kv_end; base += TL_WAVE) {
    const int j = base + lane;
    const bool valid = j < kv_end;
    float s = -INFINITY;
    int slot = 0;
    if (valid) {
      slot = bt[j / block_size] * block_size + (j % block_size);
      const T* cp = latent + (int64_t)slot * kv_rank;
      const T* kp = rope + (int64_t)slot * rot;
      float dot = 0.f;
      for (int dd = 0; dd < kv_rank; ++dd) dot = fmaf(qs[dd], to_f32(cp[dd]), dot);
      for (int dd = 0; dd < rot; ++dd) dot = fmaf(qs[kv_rank + dd], to_f32(kp[dd]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));      // lane 0 of every tile is valid: m_new is finite
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);
    l = l * alpha + wave_sum(p);
#pragma unroll
    for (int i = 0; i < kRPL; ++i) o[i] *= alpha;
    const int n_keys = min(TL_WAVE, kv_end - base);
    for (int jj = 0; jj < n_keys; ++jj) {
      const float pj = __shfl(p, jj, TL_WAVE);
      const T* cp = latent + (int64_t)__shfl(slot, jj, TL_WAVE) * kv_rank;
#pragma unroll
      for (int i = 0; i < kRPL; ++i) {
        const int dd = lane + i * TL_WAVE;
        if (dd < kv_rank) o[i] = fmaf(pj, to_f32(cp[dd]), o[i]);
      }
    }
    m = m_new;
  }
  float f = 1.f / l;
  if (gate) f /= 1.f + expf(-to_f32(gate[(int64_t)t * gate_stride + h]));
  T* orow = out + ((int64_t)t * heads + h) * kv_rank;
#pragma unroll
  for (int i = 0; i < kRPL; ++i) {
    const int dd = lane + i * TL_WAVE;
    if (dd < kv_rank) orow[dd] = from_f32<T>(o[i] * f);
  }
}

// Small products per head for steps of few rows: out[t, h, n] = sum_k w[h, k, n] * in[t, h, k].
// The weights lie [heads, inner, cols], so that the threads of a workgroup (one per output column)
// read them in whole lines; a workgroup takes up to kRows rows at a time, whose inputs it keeps in LDS.
constexpr int kRows = 8;
constexpr int kMaxInner = 1024;
template <typename TI, typename TW, typename TO>
__global__ __launch_bounds__(kThreads) void head_products_kernel(const TI* __restrict__ in, int64_t in_stride,
                                                                 int in_head_width, const TW* __restrict__ w,
                                                                 TO* __restrict__ out, int64_t out_stride,
                                                                 int out_head_width, int n_rows, int inner, int cols) {
  __shared__ float xs[kRows][kMaxInner];
  const int h = blockIdx.x, n = blockIdx.y * kThreads + threadIdx.x;
  const int t0 = blockIdx.z * kRows, rows = min(kRows, n_rows - t0);
  for (int e = threadIdx.x; e < rows * inner; e += kThreads) {
    const int r = e / inner, k = e - r * inner;
    xs[r][k] = to_f32(in[(int64_t)(t0 + r) * in_stride + (int64_t)h * in_head_width + k]);
  }
  __syncthreads();
  if (n >= cols) return;
  float acc[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) acc[r] = 0.f;
  const TW* wp = w + (int64_t)h * inner * cols + n;
  for (int k = 0; k < inner; ++k) {
    const float wv = to_f32(wp[(int64_t)k * cols]);
#pragma unroll
    for (int r = 0; r < kRows; ++r) acc[r] = fmaf(wv, xs[r][k], acc[r]);      // rows beyond `rows` hold stale LDS: never stored
  }
#pragma unroll
  for (int r = 0; r < kRows; ++r)
    if (r < rows) out[(int64_t)(t0 + r) * out_stride + (int64_t)h * out_head_width + n] = from_f32<TO>(acc[r]);
}

}  // namespace

#define TL_DISPATCH_T(dtype, ...)                 \
  if ((dtype) == 0) { using T = float; __VA_ARGS__ } \
  else if ((dtype) == 1) { using T = bf16_t; __VA_ARGS__ } \
  else return TL_ERR_ARG;

extern "C" {

// kv_rank == 0: a layer that keeps no cache of its own (it only needs its query latent).
int tl_latent_prepare(const void* d, int64_t d_stride, int q_off, int q_rank, int kv_off, int kv_rank, int rot,
                      int rdims, const float* w_q, const float* w_kv, float eps, const int32_t* positions, const float* cos_t,
                      const float* sin_t, const int32_t* slot_mapping, void* cq, void* latent, void* rope,
                      int n_tokens, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (q_rank <= 0 || kv_rank < 0 || rot < 0 || rdims < 0 || rdims % 2 || rdims > rot) return TL_ERR_ARG;
  if (kv_rank > 0 && (!slot_mapping || !latent || (rot > 0 && !rope) || (rdims > 0 && (!cos_t || !sin_t || !positions))))
    return TL_ERR_ARG;
  TL_DISPATCH_T(dtype, hipLaunchKernelGGL(latent_prepare_kernel<T>, dim3(n_tokens), dim3(kThreads), 0, stream,
                                          (const T*)d, d_stride, q_off, q_rank, kv_off, kv_rank, rot, rdims, w_q, w_kv, eps,
                                          positions, cos_t, sin_t, slot_mapping, (T*)cq, (T*)latent, (T*)rope);)
  return tl_launch_status();
}

int tl_rotate_into(const void* q, int64_t q_stride, int head_width, int in_off, int rot, int rdims, int heads,
                   const int32_t* positions, const float* cos_t, const float* sin_t, float* out, int out_width,
                   int out_off, int n_tokens, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || rot == 0) return TL_OK;
  if (rot < 0 || rdims < 0 || rdims % 2 || rdims > rot || heads <= 0 || in_off + rot > head_width ||
      out_off + rot > out_width)
    return TL_ERR_ARG;
  TL_DISPATCH_T(dtype, hipLaunchKernelGGL(rotate_into_kernel<T>, dim3(n_tokens), dim3(kThreads), 0, stream,
                                          (const T*)q, q_stride, head_width, in_off, rot, rdims, heads, positions, cos_t,
                                          sin_t, out, out_width, out_off);)
  return tl_launch_status();
}

int tl_latent_attention(const float* qa, const void* latent, const void* rope, const int32_t* block_tables,
                        int max_blocks, const int32_t* req_of_token, const int32_t* positions, const void* gate,
                        int64_t gate_stride, void* out, int n_tokens, int heads, int kv_rank, int rot,
                        int block_size, float scale, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (heads <= 0 || heads > 65535 || kv_rank <= 0 || kv_rank > kMaxRank || rot < 0 || kv_rank + rot > kMaxQ ||
      block_size <= 0 || max_blocks <= 0)
    return TL_ERR_ARG;
  dim3 g(n_tokens, heads), b(TL_WAVE);
  TL_DISPATCH_T(dtype, hipLaunchKernelGGL(latent_attention_kernel<T>, g, b, 0, stream, qa, (const T*)latent,
                                          (const T*)rope, block_tables, max_blocks, req_of_token, positions,
                                          (const T*)gate, gate_stride, (T*)out, heads, kv_rank, rot, block_size,
                                          scale);)
  return tl_launch_status();
}

// in / out: rows with a stride, head h at column h * head_width.  w [heads, inner, cols] of in's type;
// out float32 (out_dtype 0) or of in's type.
int tl_head_products(const void* in, int64_t in_stride, int in_head_width, const void* w, void* out,
                     int64_t out_stride, int out_head_width, int n_rows, int heads, int inner, int cols, int dtype,
                     int out_dtype, hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (heads <= 0 || inner <= 0 || inner > kMaxInner || cols <= 0 || inner > in_head_width || cols > out_head_width ||
      (n_rows + kRows - 1) / kRows > 65535 || (cols + kThreads - 1) / kThreads > 65535)
    return TL_ERR_ARG;
  dim3 g(heads, (cols + kThreads - 1) / kThreads, (n_rows + kRows - 1) / kRows), b(kThreads);
#define TL_HP(TI, TO)                                                                                              \
  hipLaunchKernelGGL((head_products_kernel<TI, TI, TO>), g, b, 0, stream, (const TI*)in, in_stride, in_head_width, \
                     (const TI*)w, (TO*)out, out_stride, out_head_width, n_rows, inner, cols)
  if (dtype == 0 && out_dtype == 0) TL_HP(float, float);
  else if (dtype == 1 && out_dtype == 0) TL_HP(bf16_t, float);
  else if (dtype == 1 && out_dtype == 1) TL_HP(bf16_t, bf16_t);
  else return TL_ERR_ARG;
#undef TL_HP
  return tl_launch_status();
}

}  // extern "C"
