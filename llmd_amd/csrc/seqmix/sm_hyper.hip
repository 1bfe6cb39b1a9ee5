// Hyper-connected residual streams and the gated activation.
//
// The residual of a stack is S fp32 streams X [S, T, d]. One workgroup owns one token row of
// all streams, so a sublayer's whole bookkeeping is one pass:
//   hyper_embed       : X[s, t] = table[ids[t]] for every s.
//   hyper_norm        : layer norm (weight, no bias) of u = sum_s in[s] X[s, t].
//   hyper_update_norm : X[j, t] <- sum_s mix[s, j] X[s, t] + out[j] y[t] for all j from the old
//                       values (each column is read for all streams, then written), and from the same
//                       registers u' = sum_j in'[j] X[j, t] with its layer norm - the next sublayer's
//                       input, or the model's final norm over the plain sum.
// The layer norm is two-pass in fp32 (mean, then the mean of squared deviations) over u kept in
// LDS; all sums have a fixed order, so a row's result does not depend on the rest of the step.
//   gated_act         : act(g) * u over the two halves of a fused [gate | up] projection.
#include "seqmix_common.h"

using namespace sm;

namespace {

constexpr int NT = 256;
constexpr int MAXS = 16;  // streams

template <typename T>
__global__ __launch_bounds__(NT) void hyper_embed_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table,
                                                         int64_t rows, float* __restrict__ X, int S, int Tn, int d) {
  const int64_t t = blockIdx.x;
  const int64_t id = ids[t];
  const bool ok = id >= 0 && id < rows;
  for (int c = threadIdx.x; c < d; c += NT) {
    const float v = ok ? ld(table + id * d + c) : 0.f;
    for (int s = 0; s < S; ++s) X[((int64_t)s * Tn + t) * d + c] = v;
  }
}

// Layer norm of the row u[0..d) held in LDS; writes out[t].
template <typename T>
__device__ __forceinline__ void ln_row(const float* u, int d, const T* __restrict__ w, float eps, T* __restrict__ o,
                                       float* red) {
  float s = 0.f;
  for (int c = threadIdx.x; c < d; c += NT) s += u[c];
  const float mean = block_sum<NT>(s, red) / (float)d;
  float q = 0.f;
  for (int c = threadIdx.x; c < d; c += NT) {
    const float dv = u[c] - mean;
    q += dv * dv;
  }
  const float var = block_sum<NT>(q, red) / (float)d;
  const float inv = 1.f / sqrtf(var + eps);
  for (int c = threadIdx.x; c < d; c += NT) st(o + c, (u[c] - mean) * inv * ld(w + c));
}

template <typename T>
__global__ __launch_bounds__(NT) void hyper_norm_kernel(const float* __restrict__ X, const float* __restrict__ w_in,
                                                        const T* __restrict__ norm_w, float eps, T* __restrict__ out,
                                                        int S, int Tn, int d) {
  extern __shared__ float u[];
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x; c < d; c += NT) {
    float a = 0.f;
    for (int s = 0; s < S; ++s) a += w_in[s] * X[((int64_t)s * Tn + t) * d + c];
    u[c] = a;
  }
  __syncthreads();
  ln_row<T>(u, d, norm_w, eps, out + t * d, red);
}

template <typename T>
__global__ __launch_bounds__(NT) void hyper_update_norm_kernel(float* __restrict__ X, const T* __restrict__ y,
                                                               int64_t y_stride, const float* __restrict__ mix,
                                                               const float* __restrict__ w_out,
                                                               const float* __restrict__ next_in,
                                                               const T* __restrict__ next_w, float eps,
                                                               T* __restrict__ out, int S, int Tn, int d) {
  extern __shared__ float u[];
  __shared__ float red[NT / 64];
  __shared__ float sm_mix[MAXS * MAXS], sm_out[MAXS], sm_in[MAXS];
  if (threadIdx.x < S * S) sm_mix[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    sm_out[threadIdx.x] = w_out[threadIdx.x];
    sm_in[threadIdx.x] = next_in ? next_in[threadIdx.x] : 0.f;
  }
  __syncthreads();
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x; c < d; c += NT) {
    float x[MAXS];
#pragma unroll
    for (int s = 0; s < MAXS; ++s) x[s] = s < S ? X[((int64_t)s * Tn + t) * d + c] : 0.f;
    const float yv = ld(y + t * y_stride + c);
    float a = 0.f;
#pragma unroll
    for (int j = 0; j < MAXS; ++j) {
      if (j >= S) break;
      float n = 0.f;
#pragma unroll
      for (int s = 0; s < MAXS; ++s)
        if (s < S) n += sm_mix[s * S + j] * x[s];
      n += sm_out[j] * yv;
      X[((int64_t)j * Tn + t) * d + c] = n;
      a += sm_in[j] * n;
    }
    u[c] = a;
  }
  if (next_w == nullptr) return;
  __syncthreads();
  ln_row<T>(u, d, next_w, eps, out + t * d, red);
}

template <typename T, int KIND>
__global__ __launch_bounds__(NT) void gated_act_kernel(const T* __restrict__ gu, int64_t stride, int F,
                                                       T* __restrict__ out, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x;
  if (i >= n) return;
  const int64_t t = i / F;
  const int j = (int)(i - t * F);
  const float g = ld(gu + t * stride + j), v = ld(gu + t * stride + F + j);
  float a;
  if (KIND == 0) a = 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
  else a = g / (1.f + expf(-g));
  st(out + i, a * v);
}

}  // namespace

extern "C" {

void sm_hyper_embed(const int64_t* ids, const void* table, int64_t rows, float* X, int S, int T, int d, int f32,
                    hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    hipLaunchKernelGGL((hyper_embed_kernel<float>), dim3(T), dim3(NT), 0, stream, ids, (const float*)table, rows, X, S,
                       T, d);
  else
    hipLaunchKernelGGL((hyper_embed_kernel<bf16_t>), dim3(T), dim3(NT), 0, stream, ids, (const bf16_t*)table, rows, X,
                       S, T, d);
}

void sm_hyper_norm(const float* X, const float* w_in, const void* norm_w, float eps, void* out, int S, int T, int d,
                   int f32, hipStream_t stream) {
  if (T == 0) return;
  const size_t lds = (size_t)d * sizeof(float);
  if (f32)
    hipLaunchKernelGGL((hyper_norm_kernel<float>), dim3(T), dim3(NT), lds, stream, X, w_in, (const float*)norm_w, eps,
                       (float*)out, S, T, d);
  else
    hipLaunchKernelGGL((hyper_norm_kernel<bf16_t>), dim3(T), dim3(NT), lds, stream, X, w_in, (const bf16_t*)norm_w,
                       eps, (bf16_t*)out, S, T, d);
}

void sm_hyper_update_norm(float* X, const void* y, int64_t y_stride, const float* mix, const float* w_out,
                          const float* next_in, const void* next_w, float eps, void* out, int S, int T, int d, int f32,
                          hipStream_t stream) {
  if (T == 0) return;
  const size_t lds = (size_t)d * sizeof(float);
  if (f32)
    hipLaunchKernelGGL((hyper_update_norm_kernel<float>), dim3(T), dim3(NT), lds, stream, X, (const float*)y, y_stride,
                       mix, w_out, next_in, (const float*)next_w, eps, (float*)out, S, T, d);
  else
    hipLaunchKernelGGL((hyper_update_norm_kernel<bf16_t>), dim3(T), dim3(NT), lds, stream, X, (const bf16_t*)y,
                       y_stride, mix, w_out, next_in, (const bf16_t*)next_w, eps, (bf16_t*)out, S, T, d);
}

void sm_gated_act(const void* gu, int64_t stride, int F, int kind, void* out, int T, int f32, hipStream_t stream) {
  const int64_t n = (int64_t)T * F;
  if (n == 0) return;
  const dim3 grid((unsigned)((n + NT - 1) / NT));
#define SM_GO(TYPE, K) \
  hipLaunchKernelGGL((gated_act_kernel<TYPE, K>), grid, dim3(NT), 0, stream, (const TYPE*)gu, stride, F, (TYPE*)out, n)
  if (f32) {
    if (kind == 0) SM_GO(float, 0);
    else SM_GO(float, 1);
  } else {
    if (kind == 0) SM_GO(bf16_t, 0);
    else SM_GO(bf16_t, 1);
  }
#undef SM_GO
}

}  // extern "C"
