// Row kernels of per-layer stacks: embedding with scale, zero-centred RMS norms on the fp32
// residual, post-norm + layer scale + residual add (+ the next pre-norm in the same pass),
// the depth average (+ the norm that follows it), xIELU and the logit soft cap.
// One workgroup of 256 threads per token row; the fp32 residual is read and written once.
#include "seqmix_common.h"

using namespace sm;

namespace {

constexpr int NT = 256;

template <typename T>
__global__ __launch_bounds__(NT) void embed_scale_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table,
                                                        float scale, float* __restrict__ o0, float* __restrict__ o1,
                                                        int d, int64_t V) {
  const int64_t row = blockIdx.x;
  const int64_t id = min(max(ids[row], (int64_t)0), V - 1);  // a bad id must not read outside the table
  const T* src = table + id * (int64_t)d;
  for (int c = threadIdx.x; c < d; c += NT) {
    const float v = ld(src + c) * scale;
    o0[row * d + c] = v;
    o1[row * d + c] = v;
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void zc_norm_kernel(const float* __restrict__ x, const T* __restrict__ w, float eps,
                                                    T* __restrict__ out, int d) {
  __shared__ float red[NT / 64];
  const int64_t row = blockIdx.x;
  const float* xr = x + row * d;
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += NT) ss += xr[c] * xr[c];
  ss = block_sum<NT>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += NT) st(out + row * d + c, xr[c] * inv * (1.f + ld(w + c)));
}

// x += ls * (y / rms(y) * (1 + wp));  optionally out = x / rms(x) * (1 + wn)
template <typename T>
__global__ __launch_bounds__(NT) void add_post_norm_kernel(const T* __restrict__ y, int64_t y_stride,
                                                          const T* __restrict__ wp, const T* __restrict__ ls,
                                                          float* __restrict__ x, float eps, const T* __restrict__ wn,
                                                          T* __restrict__ out, int d) {
  __shared__ float red[NT / 64];
  const int64_t row = blockIdx.x;
  const T* yr = y + row * y_stride;
  float* xr = x + row * d;
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += NT) {
    const float v = ld(yr + c);
    ss += v * v;
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)d + eps);
  float s2 = 0.f;
  for (int c = threadIdx.x; c < d; c += NT) {
    const float v = xr[c] + ld(ls + c) * (ld(yr + c) * inv * (1.f + ld(wp + c)));
    xr[c] = v;
    s2 += v * v;
  }
  if (wn == nullptr) return;
  s2 = block_sum<NT>(s2, red);
  const float inv2 = 1.f / sqrtf(s2 / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += NT) st(out + row * d + c, xr[c] * inv2 * (1.f + ld(wn + c)));
}

// hist[dst] = sum_{j<n} coef[j] hist[j];  out = zero-centred norm of it
template <typename T>
__global__ __launch_bounds__(NT) void depth_avg_norm_kernel(float* __restrict__ hist, int64_t plane, int n,
                                                           const float* __restrict__ coef, int dst,
                                                           const T* __restrict__ w, float eps, T* __restrict__ out,
                                                           int d) {
  __shared__ float red[NT / 64];
  const int64_t row = blockIdx.x;
  float* dr = hist + dst * plane + row * d;
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += NT) {
    float s = 0.f;
    for (int j = 0; j < n; ++j) s += coef[j] * hist[j * plane + row * d + c];
    dr[c] = s;
    ss += s * s;
  }
  ss = block_sum<NT>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += NT) st(out + row * d + c, dr[c] * inv * (1.f + ld(w + c)));
}

template <typename T>
__global__ __launch_bounds__(NT) void xielu_kernel(const T* __restrict__ z, float ap, float aq, T* __restrict__ out,
                                                  int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x;
  if (i >= n) return;
  const float v = ld(z + i);
  st(out + i, v > 0.f ? ap * v * v + 0.5f * v : aq * (expm1f(v) - v) + 0.5f * v);
}

__global__ __launch_bounds__(NT) void softcap_kernel(float* __restrict__ x, float cap, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

}  // namespace

extern "C" {

void sm_embed_scale(const int64_t* ids, const void* table, float scale, float* o0, float* o1, int T, int d,
                    int64_t V, int f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32) hipLaunchKernelGGL((embed_scale_kernel<float>), dim3(T), dim3(NT), 0, stream, ids, (const float*)table, scale, o0, o1, d, V);
  else hipLaunchKernelGGL((embed_scale_kernel<bf16_t>), dim3(T), dim3(NT), 0, stream, ids, (const bf16_t*)table, scale, o0, o1, d, V);
}

void sm_zc_norm(const float* x, const void* w, float eps, void* out, int T, int d, int f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32) hipLaunchKernelGGL((zc_norm_kernel<float>), dim3(T), dim3(NT), 0, stream, x, (const float*)w, eps, (float*)out, d);
  else hipLaunchKernelGGL((zc_norm_kernel<bf16_t>), dim3(T), dim3(NT), 0, stream, x, (const bf16_t*)w, eps, (bf16_t*)out, d);
}

void sm_add_post_norm(const void* y, int64_t y_stride, const void* wp, const void* ls, float* x, float eps,
                      const void* wn, void* out, int T, int d, int f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    hipLaunchKernelGGL((add_post_norm_kernel<float>), dim3(T), dim3(NT), 0, stream, (const float*)y, y_stride,
                       (const float*)wp, (const float*)ls, x, eps, (const float*)wn, (float*)out, d);
  else
    hipLaunchKernelGGL((add_post_norm_kernel<bf16_t>), dim3(T), dim3(NT), 0, stream, (const bf16_t*)y, y_stride,
                       (const bf16_t*)wp, (const bf16_t*)ls, x, eps, (const bf16_t*)wn, (bf16_t*)out, d);
}

void sm_depth_avg_norm(float* hist, int64_t plane, int n, const float* coef, int dst, const void* w, float eps,
                       void* out, int T, int d, int f32, hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    hipLaunchKernelGGL((depth_avg_norm_kernel<float>), dim3(T), dim3(NT), 0, stream, hist, plane, n, coef, dst,
                       (const float*)w, eps, (float*)out, d);
  else
    hipLaunchKernelGGL((depth_avg_norm_kernel<bf16_t>), dim3(T), dim3(NT), 0, stream, hist, plane, n, coef, dst,
                       (const bf16_t*)w, eps, (bf16_t*)out, d);
}

void sm_xielu(const void* z, float ap, float aq, void* out, int64_t n, int f32, hipStream_t stream) {
  if (n == 0) return;
  const dim3 grid((unsigned)((n + NT - 1) / NT));
  if (f32) hipLaunchKernelGGL((xielu_kernel<float>), grid, dim3(NT), 0, stream, (const float*)z, ap, aq, (float*)out, n);
  else hipLaunchKernelGGL((xielu_kernel<bf16_t>), grid, dim3(NT), 0, stream, (const bf16_t*)z, ap, aq, (bf16_t*)out, n);
}

void sm_softcap(float* x, float cap, int64_t n, hipStream_t stream) {
  if (n == 0) return;
  hipLaunchKernelGGL(softcap_kernel, dim3((unsigned)((n + NT - 1) / NT)), dim3(NT), 0, stream, x, cap, n);
}

}  // extern "C"
