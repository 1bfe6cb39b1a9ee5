// Shared helpers of the sequence-mixer op library (gfx950 / CDNA4, wave 64).
// Kernels are templated on the activation storage type: float, or bf16 as raw 16-bit words.
// All arithmetic is fp32.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sm {

typedef uint16_t bf16_t;

__device__ __forceinline__ float ld(const float* p) { return *p; }
__device__ __forceinline__ float ld(const bf16_t* p) { return __uint_as_float(((uint32_t)*p) << 16); }
__device__ __forceinline__ void st(float* p, float v) { *p = v; }
__device__ __forceinline__ void st(bf16_t* p, float v) {
  __bf16 h = (__bf16)v;  // round to nearest even
  *p = __builtin_bit_cast(uint16_t, h);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
// Sum over a workgroup of NT threads (NT a multiple of 64); every thread gets the result.
// The order of the additions is fixed, so a row's result does not depend on the launch.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NT / 64; ++i) s += red[i];
  __syncthreads();
  return s;
}

// fp32 transcendentals for the sequential scans. float32 storage: the precise library functions.
// bfloat16 storage: the hardware exp2 / log2 / reciprocal forms (about 1 ulp of fp32, far below the
// rounding of the values they are applied to); on a single wave per SIMD the precise forms are most
// of a token's latency.
template <typename T> struct Fn {
  static __device__ __forceinline__ float exp(float x) { return expf(x); }
  static __device__ __forceinline__ float sigmoid(float x) { return 1.f / (1.f + expf(-x)); }
  static __device__ __forceinline__ float silu(float x) { return x / (1.f + expf(-x)); }
  static __device__ __forceinline__ float softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }
  static __device__ __forceinline__ float rsqrt(float x) { return 1.f / sqrtf(x); }
};
template <> struct Fn<uint16_t> {
  static __device__ __forceinline__ float exp(float x) { return __expf(x); }
  static __device__ __forceinline__ float sigmoid(float x) { return __frcp_rn(1.f + __expf(-x)); }
  static __device__ __forceinline__ float silu(float x) { return x * __frcp_rn(1.f + __expf(-x)); }
  static __device__ __forceinline__ float softplus(float x) { return x > 20.f ? x : __logf(1.f + __expf(x)); }
  static __device__ __forceinline__ float rsqrt(float x) { return __frsqrt_rn(x); }
};

__device__ __forceinline__ float siluf_(float x) { return x / (1.f + expf(-x)); }

}  // namespace sm
