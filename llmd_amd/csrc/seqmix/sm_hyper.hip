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

// Four columns per thread and step (d % 4 == 0, 16-byte aligned rows): the streams move as float4.
__device__ __forceinline__ void ld4(const float* p, float (&v)[4]) {
  const float4 t = *reinterpret_cast<const float4*>(p);
  v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void ld4(const bf16_t* p, float (&v)[4]) {
  const uint2 t = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
  v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}
__device__ __forceinline__ void st4(float* p, const float (&v)[4]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void st4(bf16_t* p, const float (&v)[4]) {
  uint32_t w[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const __bf16 a = (__bf16)v[2 * i], b = (__bf16)v[2 * i + 1];  // round to nearest even
    w[i] = (uint32_t)__builtin_bit_cast(uint16_t, a) | ((uint32_t)__builtin_bit_cast(uint16_t, b) << 16);
  }
  *reinterpret_cast<uint2*>(p) = make_uint2(w[0], w[1]);
}

constexpr int VMAXS = 4;  // streams of the float4 form

template <typename T>
__global__ __launch_bounds__(NT) void hyper_update_norm_vec_kernel(float* __restrict__ X, const T* __restrict__ y,
                                                                   int64_t y_stride, const float* __restrict__ mix,
                                                                   const float* __restrict__ w_out,
                                                                   const float* __restrict__ next_in,
                                                                   const T* __restrict__ next_w, float eps,
                                                                   T* __restrict__ out, int S, int Tn, int d) {
  extern __shared__ __attribute__((aligned(16))) float u[];
  __shared__ float red[NT / 64];
  __shared__ float sm_mix[VMAXS * VMAXS], sm_out[VMAXS], sm_in[VMAXS];
  if (threadIdx.x < S * S) sm_mix[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    sm_out[threadIdx.x] = w_out[threadIdx.x];
    sm_in[threadIdx.x] = next_in ? next_in[threadIdx.x] : 0.f;
  }
  __syncthreads();
  const int64_t t = blockIdx.x;
  float psum = 0.f;
  for (int c = threadIdx.x * 4; c < d; c += NT * 4) {
    float x[VMAXS][4], yv[4], a[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < VMAXS; ++s)
      if (s < S) ld4(X + ((int64_t)s * Tn + t) * d + c, x[s]);
    ld4(y + t * y_stride + c, yv);
#pragma unroll
    for (int j = 0; j < VMAXS; ++j) {
      if (j >= S) break;
      float n[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = 0.f;
#pragma unroll
        for (int s = 0; s < VMAXS; ++s)
          if (s < S) v += sm_mix[s * S + j] * x[s][i];   // the order of the scalar kernel
        v += sm_out[j] * yv[i];
        n[i] = v;
        a[i] += sm_in[j] * v;
      }
      st4(X + ((int64_t)j * Tn + t) * d + c, n);
    }
    st4(u + c, a);
    psum += (a[0] + a[1]) + (a[2] + a[3]);
  }
  if (next_w == nullptr) return;
  // two-pass layer norm; a thread re-reads only the columns it wrote itself
  const float mean = block_sum<NT>(psum, red) / (float)d;
  float q = 0.f;
  for (int c = threadIdx.x * 4; c < d; c += NT * 4) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float dv = u[c + i] - mean;
      q += dv * dv;
    }
  }
  const float var = block_sum<NT>(q, red) / (float)d;
  const float inv = 1.f / sqrtf(var + eps);
  for (int c = threadIdx.x * 4; c < d; c += NT * 4) {
    float w[4], o[4];
    ld4(next_w + c, w);
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (u[c + i] - mean) * inv * w[i];
    st4(out + t * d + c, o);
  }
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

// bf16, F % 8 == 0, 16-byte aligned rows: eight columns per thread from 16-byte loads.
template <int KIND>
__global__ __launch_bounds__(NT) void gated_act_vec_kernel(const bf16_t* __restrict__ gu, int64_t stride, int F,
                                                           bf16_t* __restrict__ out, int64_t n8) {
  const int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x;
  if (i >= n8) return;
  const int f8 = F / 8;
  const int64_t t = i / f8;
  const int j = (int)(i - t * f8) * 8;
  float g[8], v[8], o[8];
  ld4(gu + t * stride + j, *reinterpret_cast<float(*)[4]>(&g[0]));
  ld4(gu + t * stride + j + 4, *reinterpret_cast<float(*)[4]>(&g[4]));
  ld4(gu + t * stride + F + j, *reinterpret_cast<float(*)[4]>(&v[0]));
  ld4(gu + t * stride + F + j + 4, *reinterpret_cast<float(*)[4]>(&v[4]));
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    float a;
    if (KIND == 0) a = 0.5f * g[q] * (1.f + tanhf(0.7978845608028654f * (g[q] + 0.044715f * g[q] * g[q] * g[q])));
    else a = g[q] / (1.f + expf(-g[q]));
    o[q] = a * v[q];
  }
  st4(out + t * F + j, *reinterpret_cast<float(*)[4]>(&o[0]));
  st4(out + t * F + j + 4, *reinterpret_cast<float(*)[4]>(&o[4]));
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
  const size_t es = f32 ? 4 : 2;
  if (S <= VMAXS && d % 4 == 0 && y_stride % 4 == 0 && ((uintptr_t)X & 15) == 0 && ((uintptr_t)y & (4 * es - 1)) == 0 &&
      ((uintptr_t)next_w & (4 * es - 1)) == 0 && ((uintptr_t)out & (4 * es - 1)) == 0) {
    if (f32)
      hipLaunchKernelGGL((hyper_update_norm_vec_kernel<float>), dim3(T), dim3(NT), lds, stream, X, (const float*)y,
                         y_stride, mix, w_out, next_in, (const float*)next_w, eps, (float*)out, S, T, d);
    else
      hipLaunchKernelGGL((hyper_update_norm_vec_kernel<bf16_t>), dim3(T), dim3(NT), lds, stream, X, (const bf16_t*)y,
                         y_stride, mix, w_out, next_in, (const bf16_t*)next_w, eps, (bf16_t*)out, S, T, d);
    return;
  }
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
  if (!f32 && F % 8 == 0 && stride % 8 == 0 && (((uintptr_t)gu | (uintptr_t)out) & 15) == 0) {
    const int64_t n8 = n / 8;
    const dim3 g8((unsigned)((n8 + NT - 1) / NT));
    if (kind == 0)
      hipLaunchKernelGGL((gated_act_vec_kernel<0>), g8, dim3(NT), 0, stream, (const bf16_t*)gu, stride, F, (bf16_t*)out, n8);
    else
      hipLaunchKernelGGL((gated_act_vec_kernel<1>), g8, dim3(NT), 0, stream, (const bf16_t*)gu, stride, F, (bf16_t*)out, n8);
    return;
  }
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
