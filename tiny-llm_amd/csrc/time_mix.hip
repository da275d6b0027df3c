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
                                                             int64_t plane, int n_mix, int width) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * kThreads + threadIdx.x;
  if (c >= width) return;
  const int r = req_of_token[t];
  const float cur = to_f32(h[(int64_t)t * h_stride + c]);
  float prev;
  if (t == cu[r]) prev = state[(int64_t)slots[r] * state_stride + prev_off + c];
  else prev = to_f32(h[(int64_t)(t - 1) * h_stride + c]);
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
// tokens of this step in order.  The key channels are cut into P slices of 16 (P a power of two, 16 P >= dim);
// thread (e, p) keeps S[16 p .. 16 p + 15, e] in registers, and the P lanes of a column are neighbours, so the sum
// over the channels ends with log2 P lane exchanges.  The order of additions is the same whatever the step holds.
// r, k and the decays of 16 tokens at a time are staged in LDS.  In memory S lies as [head][s][e][p]
// (s the index within a slice): a wave's accesses to the state are contiguous.
constexpr int kSlice = 16;
constexpr int kChunk = 16;

__global__ __launch_bounds__(kThreads) void time_mix_recurrence_kernel(
    const float* __restrict__ x, int64_t x_stride, int r_off, int k_off, int v_off, int w_off,
    const float* __restrict__ w0, const float* __restrict__ u, float* __restrict__ state, int64_t state_stride,
    const int32_t* __restrict__ cu, const int32_t* __restrict__ slots, float* __restrict__ o, int heads, int dim, int vdim,
    int P) {
  extern __shared__ __align__(16) float lds[];
  const int EC = kThreads / P, Dp = kSlice * P;
  float* r_s = lds;                       // [kChunk][Dp]
  float* k_s = r_s + kChunk * Dp;
  float* w_s = k_s + kChunk * Dp;
  float* v_s = w_s + kChunk * Dp;         // [kChunk][EC]
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
  for (int c0 = 0; c0 < n; c0 += kChunk) {
    const int m = min(kChunk, n - c0);
    __syncthreads();
    for (int i = tid; i < m * Dp; i += kThreads) {
      const int tt = i / Dp, d = i - tt * Dp;
      float rr = 0.f, kk = 0.f, ww = 1.f;
      if (d < dim) {
        const float* row = x + (int64_t)(t0 + c0 + tt) * x_stride + head * dim + d;
        rr = row[r_off];
        kk = row[k_off];
        ww = expf(-expf(row[w_off] + w0[head * dim + d]));
      }
      r_s[i] = rr;
      k_s[i] = kk;
      w_s[i] = ww;
    }
    for (int i = tid; i < m * EC; i += kThreads) {
      const int tt = i / EC, ee = blockIdx.x * EC + (i - tt * EC);
      v_s[i] = ee < vdim ? x[(int64_t)(t0 + c0 + tt) * x_stride + v_off + head * vdim + ee] : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < m; ++tt) {
      const float vv = v_s[tt * EC + el];
      const float* rp = r_s + tt * Dp + p * kSlice;
      const float* kp = k_s + tt * Dp + p * kSlice;
      const float* wp = w_s + tt * Dp + p * kSlice;
      float acc = 0.f;
#pragma unroll
      for (int s4 = 0; s4 < kSlice; s4 += 4) {
        const f32x4 r4 = *(const f32x4*)(rp + s4), k4 = *(const f32x4*)(kp + s4), w4 = *(const f32x4*)(wp + s4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float kv = k4[j] * vv;
          acc = fmaf(r4[j], fmaf(uu[s4 + j], kv, S[s4 + j]), acc);
          S[s4 + j] = fmaf(w4[j], S[s4 + j], kv);
        }
      }
      for (int sh = P >> 1; sh >= 1; sh >>= 1) acc += __shfl_xor(acc, sh, TL_WAVE);
      if (p == 0 && col) o[(int64_t)(t0 + c0 + tt) * ((int64_t)heads * vdim) + head * vdim + e] = acc;
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
int tl_shift_mix(const void* h, int64_t h_stride, const float* state, int64_t state_stride, int64_t prev_off,
                 const int32_t* req_of_token, const int32_t* cu, const int32_t* slots, const float* mu, void* out,
                 int n_tokens, int n_mix, int width, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (width <= 0 || n_mix <= 0 || !h || !state || !req_of_token || !cu || !slots || !mu || !out) return TL_ERR_ARG;
  dim3 g(n_tokens, (width + kThreads - 1) / kThreads), b(kThreads);
  const int64_t plane = (int64_t)n_tokens * width;
  if (dtype == 0)
    hipLaunchKernelGGL(shift_mix_kernel<float>, g, b, 0, stream, (const float*)h, h_stride, state, state_stride, prev_off,
                       req_of_token, cu, slots, mu, (float*)out, plane, n_mix, width);
  else if (dtype == 1)
    hipLaunchKernelGGL(shift_mix_kernel<bf16_t>, g, b, 0, stream, (const bf16_t*)h, h_stride, state, state_stride,
                       prev_off, req_of_token, cu, slots, mu, (bf16_t*)out, plane, n_mix, width);
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
// and v (heads * vdim columns from v_off).  state rows: S as [heads][16][vdim][P] floats from column 0, P =
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
  const size_t smem = (size_t)kChunk * (3 * kSlice * P + EC) * sizeof(float);
  dim3 g((vdim + EC - 1) / EC, heads, n_requests), b(kThreads);
  hipLaunchKernelGGL(time_mix_recurrence_kernel, g, b, smem, stream, x, x_stride, r_off, k_off, v_off, w_off, w0, u, state,
                     state_stride, cu, slots, o, heads, dim, vdim, P);
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
