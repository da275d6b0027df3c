// Time mixing with a decaying matrix state per head (a linear recurrence whose decay is a vector per
// token, one factor per head and key channel, and whose current token gets a bonus):
//     o_t = (S + diag(u) k_t v_t^T)^T r_t,      S <- diag(w_t) S + k_t v_t^T,      w_t = exp(-exp(x_t + w0))
// and the token shift in front of its projections: each projection reads h_t + (h_(t-1) - h_t) * mu.
//
// Per request the state row holds S of every head and the last token's h, all float32.  Everything
// that enters the recurrence is float32 in both precisions (r, k, v and x are products' float32 results).
#include "common.h"

namespace {

constexpr int kThreads = 256;

// out[m, t, c] = h[t, c] + (prev - h[t, c]) * mu[m, c]; prev is h[t - 1, c], or for the first token a request
// brings in this step what the state row keeps at prev_off (zero for a request's very first token).
template <typename T>
__global__ __launch_bounds__(kThreads) void shift_mix_kernel(const T* __restrict__ h, int64_t h_stride,
                                                             const float* __restrict__ state, int64_t state_stride,
                                                             int64_t prev_off, const int32_t* __restrict__ req_of_token,
                                                             const int32_t* __restrict__ cu,
                                                             const int32_t* __restrict__ slots,
                                                             const float* __restrict__ mu, T* __restrict__ out,
                                                             int64_t plane, int n_mix, int width, int save_single) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * kThreads + threadIdx.x;
  if (c >= width) return;
  const int r = req_of_token[t];
  const float cur = to_f32(h[(int64_t)t * h_stride + c]);
  float prev;
  if (t == cu[r]) {
    float* saved = const_cast<float*>(state) + (int64_t)slots[r] * state_stride + prev_off + c;
    prev = *saved;
    // a request's only token of the step is also its last: this thread has read what the state kept and leaves
    // the token's h in its place (steps of single tokens then need no kernel of their own for that)
    if (save_single && cu[r + 1] == t + 1) *saved = cur;
  } else {
    prev = to_f32(h[(int64_t)(t - 1) * h_stride + c]);
  }
  const float d = prev - cur;
  for (int m = 0; m < n_mix; ++m)
    out[(int64_t)m * plane + (int64_t)t * width + c] = from_f32<T>(fmaf(d, mu[(int64_t)m * width + c], cur));
}

// The last token a request brings becomes the state's saved h.  A request without tokens keeps its state.
template <typename T>
__global__ __launch_bounds__(kThreads) void shift_save_kernel(const T* __restrict__ h, int64_t h_stride,
                                                              float* __restrict__ state, int64_t state_stride,
                                                              int64_t prev_off, const int32_t* __restrict__ cu,
                                                              const int32_t* __restrict__ slots, int width) {
  const int r = blockIdx.x;
  const int c = blockIdx.y * kThreads + threadIdx.x;
  const int t0 = cu[r], t1 = cu[r + 1];
  if (c >= width || t1 <= t0) return;
  state[(int64_t)slots[r] * state_stride + prev_off + c] = to_f32(h[(int64_t)(t1 - 1) * h_stride + c]);
}

// The recurrence.  A workgroup owns EC value columns of one (request, head) and walks the request's
// tokens of this step in order.  The key channels are cut into P slices of 4 (P a power of two, 4 P >= dim);
// thread (e, p) keeps S[4 p .. 4 p + 3, e] in registers, and the P lanes of a column are neighbours, so the sum
// over the channels ends with log2 P lane exchanges (moves inside a row of 16 lanes, then lane swaps).  The
// order of additions is the same whatever the step holds.  Per token a thread's chain is one multiply-add a
// state element; a head's columns are shared out over V / EC workgroups, so that one long prompt still fills
// many compute units.  r, k and the decays of 16 tokens at a time are staged in LDS, the next 16 requested
// before these are worked on.  In memory S lies as [head][s][e][p] (s the index within a slice): a wave's
// accesses to the state are contiguous.
constexpr int kSlice = 4;
constexpr int kChunk = 16;

template <int P>
__device__ __forceinline__ float sum_over_slices(float v) {
  if constexpr (P >= 2) v += dpp_f32<TL_DPP_XOR1>(v);
  if constexpr (P >= 4) v += dpp_f32<TL_DPP_XOR2>(v);
  if constexpr (P >= 8) v += dpp_f32<TL_DPP_HALF_MIRROR>(v);      // the quads of a half row hold one value each by now
  if constexpr (P >= 16) v += dpp_f32<TL_DPP_MIRROR>(v);
  if constexpr (P >= 32) {
    float a, b;
    pair16(v, a, b);
    v = a + b;
  }
  if constexpr (P >= 64) {
    float a, b;
    pair32(v, a, b);
    v = a + b;
  }
  return v;
}

template <int P>
__global__ __launch_bounds__(kThreads) void time_mix_recurrence_kernel(
    const float* __restrict__ x, int64_t x_stride, int r_off, int k_off, int v_off, int w_off,
    const float* __restrict__ w0, const float* __restrict__ u, float* __restrict__ state, int64_t state_stride,
    const int32_t* __restrict__ cu, const int32_t* __restrict__ slots, float* __restrict__ o, int heads, int dim, int vdim) {
  constexpr int EC = kThreads / P, Dp = kSlice * P;
  constexpr int NST = (kChunk * Dp + kThreads - 1) / kThreads, NV = (kChunk * EC + kThreads - 1) / kThreads;
  __shared__ __align__(16) float r_s[kChunk * Dp];
  __shared__ __align__(16) float k_s[kChunk * Dp];
  __shared__ __align__(16) float w_s[kChunk * Dp];
  __shared__ float v_s[kChunk * EC];
  const int req = blockIdx.z, head = blockIdx.y;
  const int t0 = cu[req], n = cu[req + 1] - t0;
  if (n <= 0) return;                     // a request without tokens touches no state
  const int tid = threadIdx.x, p = tid % P, el = tid / P;
  const int e = blockIdx.x * EC + el;
  const bool col = e < vdim;
  float* Sg = state + (int64_t)slots[req] * state_stride + (((int64_t)head * kSlice) * vdim + (col ? e : 0)) * P + p;
  const int64_t s_step = (int64_t)vdim * P;
  float S[kSlice], uu[kSlice];
#pragma unroll
  for (int s = 0; s < kSlice; ++s) {
    S[s] = col ? Sg[s * s_step] : 0.f;
    const int d = p * kSlice + s;
    uu[s] = d < dim ? u[head * dim + d] : 0.f;
  }
  // what this thread stages of a chunk: element i = tid + j * kThreads of [token][channel], token i / Dp
  float pr[NST], pk[NST], pw[NST], pv[NV];
  auto fetch = [&](int c0) {
    const int m = min(kChunk, n - c0);
#pragma unroll
    for (int j = 0; j < NST; ++j) {
      const int i = tid + j * kThreads, tt = i / Dp, d = i % Dp;
      pr[j] = pk[j] = 0.f;
      pw[j] = -INFINITY;                   // a channel beyond the head's: decay exp(-exp(-inf)) = 1, nothing added
      if (i < kChunk * Dp && tt < m && d < dim) {
        const float* row = x + (int64_t)(t0 + c0 + tt) * x_stride + head * dim + d;
        pr[j] = row[r_off];
        pk[j] = row[k_off];
        pw[j] = row[w_off] + w0[head * dim + d];
      }
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = tid + j * kThreads, tt = i / EC, ee = blockIdx.x * EC + i % EC;
      pv[j] = (i < kChunk * EC && tt < m && ee < vdim) ? x[(int64_t)(t0 + c0 + tt) * x_stride + v_off + head * vdim + ee] : 0.f;
    }
  };
  fetch(0);
  for (int c0 = 0; c0 < n; c0 += kChunk) {
    const int m = min(kChunk, n - c0);
    __syncthreads();                       // the chunk before is done with
#pragma unroll
    for (int j = 0; j < NST; ++j) {
      const int i = tid + j * kThreads;
      if (i < kChunk * Dp) {
        r_s[i] = pr[j];
        k_s[i] = pk[j];
        w_s[i] = expf(-expf(pw[j]));
      }
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = tid + j * kThreads;
      if (i < kChunk * EC) v_s[i] = pv[j];
    }
    __syncthreads();
    if (c0 + kChunk < n) fetch(c0 + kChunk);      // on its way while this chunk is worked on
    float* orow = o + (int64_t)(t0 + c0) * ((int64_t)heads * vdim) + head * vdim + e;
    auto token = [&](int tt) {
      const float vv = v_s[tt * EC + el];
      const f32x4 r4 = *(const f32x4*)(r_s + tt * Dp + p * kSlice), k4 = *(const f32x4*)(k_s + tt * Dp + p * kSlice),
                  w4 = *(const f32x4*)(w_s + tt * Dp + p * kSlice);
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < kSlice; ++j) {
        const float kv = k4[j] * vv;
        acc = fmaf(r4[j], fmaf(uu[j], kv, S[j]), acc);
        S[j] = fmaf(w4[j], S[j], kv);
      }
      acc = sum_over_slices<P>(acc);
      if (p == 0 && col) orow[(int64_t)tt * heads * vdim] = acc;
    };
    if (m == kChunk) {
#pragma unroll
      for (int tt = 0; tt < kChunk; ++tt) token(tt);
    } else {
      for (int tt = 0; tt < m; ++tt) token(tt);
    }
  }
  if (col) {
#pragma unroll
    for (int s = 0; s < kSlice; ++s) Sg[s * s_step] = S[s];
  }
}

// out[i] = tanh(in[i]) rounded to T (the middle of a low-rank projection).
template <typename T>
__global__ void tanh_kernel(const float* __restrict__ in, int64_t in_stride, T* __restrict__ out, int64_t total, int n) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / n;
  out[i] = from_f32<T>(tanhf(in[t * in_stride + (i - t * n)]));
}

}  // namespace

extern "C" {

int tl_time_mix_slices(int dim) {
  int P = 1;
  while (P * kSlice < dim) P *= 2;
  return P;
}

// h: [n_tokens, width] of the engine's type; mu: float32 [n_mix, width]; out: [n_mix, n_tokens, width].
// save_single: a request that brings exactly one token also gets that token's h saved in its state row (requests
// with more tokens need tl_shift_save behind this kernel).
int tl_shift_mix(const void* h, int64_t h_stride, float* state, int64_t state_stride, int64_t prev_off,
                 const int32_t* req_of_token, const int32_t* cu, const int32_t* slots, const float* mu, void* out,
                 int n_tokens, int n_mix, int width, int save_single, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (width <= 0 || n_mix <= 0 || !h || !state || !req_of_token || !cu || !slots || !mu || !out) return TL_ERR_ARG;
  dim3 g(n_tokens, (width + kThreads - 1) / kThreads), b(kThreads);
  const int64_t plane = (int64_t)n_tokens * width;
  if (dtype == 0)
    hipLaunchKernelGGL(shift_mix_kernel<float>, g, b, 0, stream, (const float*)h, h_stride, state, state_stride, prev_off,
                       req_of_token, cu, slots, mu, (float*)out, plane, n_mix, width, save_single);
  else if (dtype == 1)
    hipLaunchKernelGGL(shift_mix_kernel<bf16_t>, g, b, 0, stream, (const bf16_t*)h, h_stride, state, state_stride,
                       prev_off, req_of_token, cu, slots, mu, (bf16_t*)out, plane, n_mix, width, save_single);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

int tl_shift_save(const void* h, int64_t h_stride, float* state, int64_t state_stride, int64_t prev_off,
                  const int32_t* cu, const int32_t* slots, int n_requests, int width, int dtype, hipStream_t stream) {
  if (n_requests <= 0) return TL_OK;
  if (width <= 0 || !h || !state || !cu || !slots) return TL_ERR_ARG;
  dim3 g(n_requests, (width + kThreads - 1) / kThreads), b(kThreads);
  if (dtype == 0)
    hipLaunchKernelGGL(shift_save_kernel<float>, g, b, 0, stream, (const float*)h, h_stride, state, state_stride, prev_off,
                       cu, slots, width);
  else if (dtype == 1)
    hipLaunchKernelGGL(shift_save_kernel<bf16_t>, g, b, 0, stream, (const bf16_t*)h, h_stride, state, state_stride,
                       prev_off, cu, slots, width);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

// x: float32 rows that hold r, k, the decay's pre-activation (heads * dim columns each, from r_off, k_off, w_off)
// and v (heads * vdim columns from v_off).  state rows: S as [heads][4][vdim][P] floats from column 0, P =
// tl_time_mix_slices(dim).  o: float32 [n_tokens, heads * vdim].
int tl_time_mix_recurrence(const float* x, int64_t x_stride, int r_off, int k_off, int v_off, int w_off, const float* w0,
                           const float* u, float* state, int64_t state_stride, const int32_t* cu, const int32_t* slots,
                           float* o, int n_requests, int heads, int dim, int vdim, hipStream_t stream) {
  if (n_requests <= 0) return TL_OK;
  if (heads <= 0 || heads > 65535 || n_requests > 65535 || dim <= 0 || dim > 256 || vdim <= 0 || !x || !w0 || !u ||
      !state || !cu || !slots || !o)
    return TL_ERR_ARG;
  const int P = tl_time_mix_slices(dim);
  if (state_stride < (int64_t)heads * kSlice * vdim * P) return TL_ERR_ARG;
  const int EC = kThreads / P;
  if ((vdim + EC - 1) / EC > 65535) return TL_ERR_ARG;
  dim3 g((vdim + EC - 1) / EC, heads, n_requests), b(kThreads);
#define TL_TIME_MIX(PP)                                                                                               \
  case PP:                                                                                                            \
    hipLaunchKernelGGL(time_mix_recurrence_kernel<PP>, g, b, 0, stream, x, x_stride, r_off, k_off, v_off, w_off, w0, u, \
                       state, state_stride, cu, slots, o, heads, dim, vdim);                                          \
    break;
  switch (P) {
    TL_TIME_MIX(1) TL_TIME_MIX(2) TL_TIME_MIX(4) TL_TIME_MIX(8) TL_TIME_MIX(16) TL_TIME_MIX(32) TL_TIME_MIX(64)
    default: return TL_ERR_ARG;
  }
#undef TL_TIME_MIX
  return tl_launch_status();
}

// out[t, j] = tanh(in[t, j]) for j < n; in float32 with row stride in_stride, out [n_rows, n] of the engine's type.
int tl_tanh_rows(const float* in, int64_t in_stride, void* out, int n_rows, int n, int dtype, hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (n <= 0 || in_stride < n || !in || !out) return TL_ERR_ARG;
  const int64_t total = (int64_t)n_rows * n;
  dim3 g((unsigned)ceil_div64(total, kThreads)), b(kThreads);
  if (dtype == 0)
    hipLaunchKernelGGL(tanh_kernel<float>, g, b, 0, stream, in, in_stride, (float*)out, total, n);
  else if (dtype == 1)
    hipLaunchKernelGGL(tanh_kernel<bf16_t>, g, b, 0, stream, in, in_stride, (bf16_t*)out, total, n);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

}  // extern "C"
