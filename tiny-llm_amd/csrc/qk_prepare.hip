// Between the query/key product and the attention kernel, for attention whose queries and keys carry a
// bias, are rotated on part of their dims and then scaled to unit root mean square, and whose values
// may be the keys themselves as projected; and behind the attention kernel, a sigmoid gate per head.
//
// Everything here is float32 arithmetic on the float32 result of the product; what leaves is rounded
// once to the engine's element type (queries, cached keys and values).
#include "common.h"

namespace {

// One wave per (token, head); heads 0 .. nq - 1 are queries, nq .. nq + nkv - 1 keys.
//   a = p[t, head, :] + bias[head, :]
//   keys with values_are_keys: v_cache[slot] = a           (before rotation and norm)
//   values otherwise (v_off >= 0): v_cache[slot] = p[t, v_off + kv head, :]
//   a <- rotate(a) on the first `rot` dims, pair i = (2i, 2i + 1) or (i, i + rot / 2), angle table row of the position
//   a <- a / sqrt(mean(a^2) + eps)   if unit_norm
//   queries -> q_out[t, head, :], keys -> k_cache[slot]    (a negative slot stores nothing)
template <typename T>
__global__ __launch_bounds__(TL_WAVE) void qk_prepare_kernel(
    const float* __restrict__ p, int64_t p_stride, const float* __restrict__ bias, const int32_t* __restrict__ positions,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, const int32_t* __restrict__ slot_mapping,
    T* __restrict__ q_out, int64_t q_stride, T* __restrict__ k_cache, T* __restrict__ v_cache, int nq, int nkv, int hd,
    int rot, int interleaved, int unit_norm, float eps, int values_are_keys, int v_off, int block_size) {
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const bool is_key = head >= nq;
  const int slot = slot_mapping ? slot_mapping[t] : -1;
  if (is_key && slot < 0) return;
  const float* src = p + (int64_t)t * p_stride + (int64_t)head * hd;
  const float* bs = bias ? bias + (int64_t)head * hd : nullptr;
  const int half = rot / 2, pairs = hd / 2;       // hd is even
  const int pos = positions[t];
  const float* cs = cos_t ? cos_t + (int64_t)pos * half : nullptr;
  const float* sn = sin_t ? sin_t + (int64_t)pos * half : nullptr;
  int64_t cache_row = 0;
  if (is_key) cache_row = (((int64_t)(slot / block_size) * nkv + (head - nq)) * block_size + slot % block_size) * hd;
  constexpr int kPairs = 2;                        // head sizes up to 256: at most 128 pairs, two a lane
  float ra[kPairs], rb[kPairs];
  int ia[kPairs], ib[kPairs];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kPairs; ++i) {
    const int j = lane + i * TL_WAVE;
    ra[i] = rb[i] = 0.f;
    ia[i] = ib[i] = 0;
    if (j < pairs) {
      if (j < half) {
        ia[i] = interleaved ? 2 * j : j;
        ib[i] = interleaved ? 2 * j + 1 : j + half;
      } else {
        ia[i] = rot + 2 * (j - half);
        ib[i] = ia[i] + 1;
      }
      float a = src[ia[i]], b = src[ib[i]];
      if (bs) {
        a += bs[ia[i]];
        b += bs[ib[i]];
      }
      if (is_key && values_are_keys) {
        v_cache[cache_row + ia[i]] = from_f32<T>(a);
        v_cache[cache_row + ib[i]] = from_f32<T>(b);
      }
      if (j < half) {
        const float c = cs[j], s = sn[j];
        ra[i] = c * a - s * b;
        rb[i] = s * a + c * b;
      } else {
        ra[i] = a;
        rb[i] = b;
      }
      ss += ra[i] * ra[i] + rb[i] * rb[i];
    }
  }
  float r = 1.f;
  if (unit_norm) r = 1.f / sqrtf(wave_sum(ss) / (float)hd + eps);
  T* dst = is_key ? k_cache + cache_row : q_out + (int64_t)t * q_stride + (int64_t)head * hd;
#pragma unroll
  for (int i = 0; i < kPairs; ++i) {
    const int j = lane + i * TL_WAVE;
    if (j < pairs) {
      dst[ia[i]] = from_f32<T>(ra[i] * r);
      dst[ib[i]] = from_f32<T>(rb[i] * r);
    }
  }
  if (is_key && !values_are_keys && v_off >= 0) {
    const float* vs = p + (int64_t)t * p_stride + v_off + (int64_t)(head - nq) * hd;
    for (int d = lane; d < hd; d += TL_WAVE) v_cache[cache_row + d] = from_f32<T>(vs[d]);
  }
}

// z[t, h, :] = a[t, h, :] * sigmoid(g[t, h]) * scale; one thread an element.
template <typename T>
__global__ void head_gate_kernel(const T* __restrict__ a, int64_t a_stride, const float* __restrict__ g, int64_t g_stride,
                                 T* __restrict__ z, int64_t z_stride, int64_t total, int heads, int hd, float scale) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int width = heads * hd;
  const int64_t t = i / width;
  const int c = (int)(i - t * width);
  const float gate = 1.f / (1.f + expf(-g[t * g_stride + c / hd]));
  z[t * z_stride + c] = from_f32<T>(to_f32(a[t * a_stride + c]) * gate * scale);
}

}  // namespace

extern "C" {

// p: float32 [n_tokens, >= (nq + nkv) * hd] (row stride p_stride): query heads, then key heads; with
// values_are_keys == 0 and v_off >= 0 the value heads start at column v_off.  bias: [(nq + nkv) * hd] or null.
// cos_t / sin_t: [positions, rot / 2] (null when rot == 0).  Caches: [blocks, nkv, block_size, hd].
int tl_qk_prepare(const float* p, int64_t p_stride, const float* bias, const int32_t* positions, const float* cos_t,
                  const float* sin_t, const int32_t* slot_mapping, void* q_out, int64_t q_stride, void* k_cache,
                  void* v_cache, int n_tokens, int nq, int nkv, int hd, int rot, int interleaved, int unit_norm, float eps,
                  int values_are_keys, int v_off, int block_size, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (nq <= 0 || nkv < 0 || nq + nkv > 65535 || hd <= 0 || hd > 256 || (hd & 1) || rot < 0 || rot > hd || (rot & 1) ||
      block_size <= 0 || !p || !positions || !q_out)
    return TL_ERR_ARG;
  if (rot > 0 && (!cos_t || !sin_t)) return TL_ERR_ARG;
  if (slot_mapping && (!k_cache || !v_cache)) return TL_ERR_ARG;
  if (interleaved != 0 && interleaved != 1) return TL_ERR_ARG;
  dim3 g(n_tokens, nq + nkv), b(TL_WAVE);
  if (dtype == 0)
    hipLaunchKernelGGL(qk_prepare_kernel<float>, g, b, 0, stream, p, p_stride, bias, positions, cos_t, sin_t, slot_mapping,
                       (float*)q_out, q_stride, (float*)k_cache, (float*)v_cache, nq, nkv, hd, rot, interleaved, unit_norm,
                       eps, values_are_keys, v_off, block_size);
  else if (dtype == 1)
    hipLaunchKernelGGL(qk_prepare_kernel<bf16_t>, g, b, 0, stream, p, p_stride, bias, positions, cos_t, sin_t,
                       slot_mapping, (bf16_t*)q_out, q_stride, (bf16_t*)k_cache, (bf16_t*)v_cache, nq, nkv, hd, rot,
                       interleaved, unit_norm, eps, values_are_keys, v_off, block_size);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

// a, z: [n_tokens, heads * hd] of the engine's type (z may be a); g: float32, one number per token and head.
int tl_head_gate(const void* a, int64_t a_stride, const float* g, int64_t g_stride, void* z, int64_t z_stride,
                 int n_tokens, int heads, int hd, float scale, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (heads <= 0 || hd <= 0 || !a || !g || !z) return TL_ERR_ARG;
  const int64_t total = (int64_t)n_tokens * heads * hd;
  dim3 grid((unsigned)ceil_div64(total, 256)), b(256);
  if (dtype == 0)
    hipLaunchKernelGGL(head_gate_kernel<float>, grid, b, 0, stream, (const float*)a, a_stride, g, g_stride, (float*)z,
                       z_stride, total, heads, hd, scale);
  else if (dtype == 1)
    hipLaunchKernelGGL(head_gate_kernel<bf16_t>, grid, b, 0, stream, (const bf16_t*)a, a_stride, g, g_stride,
                       (bf16_t*)z, z_stride, total, heads, hd, scale);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

}  // extern "C"
