// Recurrent mixers over a step's per-sequence token runs (seq_start [n+1]), each continuing the
// state in its slot (seq_slot) or starting from zero (seq_init == 0). States are fp32.
//
// causal_conv_silu : per-channel short convolution + SiLU; the last taps-1 inputs of a sequence
//                    are its convolution state (a second small kernel rolls it forward).
// selective_scan   : S[c,n] <- exp(dt_c A[c,n]) S[c,n] + dt_c x_c B_n; y_c = sum_n S[c,n] C_n + D_c x_c;
//                    y * silu(z). A channel's states sit in neighbouring lanes (groups of NL), the
//                    sum over n is a shuffle reduction; softplus, exp and the state are fp32.
// gdelta_scan      : S <- diag(w) S - (a u)(u^T S) + k v^T, o = S^T r per head; one workgroup per
//                    (head, sequence), a thread owns one value column of S in registers, the token's
//                    key-side vectors are broadcast from LDS; then the head's RMS norm, weight and gate.
#include "seqmix_common.h"

using namespace sm;

namespace {

constexpr int NT = 256;

template <typename T>
__global__ __launch_bounds__(NT) void conv_silu_kernel(const T* __restrict__ xz, int64_t xz_stride, int C,
                                                      const T* __restrict__ w, const T* __restrict__ b, int taps,
                                                      const T* __restrict__ state, const int* __restrict__ seq_start,
                                                      const int* __restrict__ seq_slot,
                                                      const int* __restrict__ seq_init, T* __restrict__ out, int seg) {
  const int c = blockIdx.x * NT + threadIdx.x;
  const int s = blockIdx.y;
  const int lo = seq_start[s], hi = seq_start[s + 1];
  const int p0 = blockIdx.z * seg;
  if (c >= C || lo + p0 >= hi) return;
  const int p1 = min(hi - lo, p0 + seg);
  const bool init = seq_init[s] != 0;
  const T* st_ = state + (int64_t)seq_slot[s] * (taps - 1) * C;
  const float bias = ld(b + c);
  for (int p = p0; p < p1; ++p) {
    float a = bias;
    for (int j = 0; j < taps; ++j) {
      const int pp = p - (taps - 1 - j);  // the last tap is the current token's
      float v = 0.f;
      if (pp >= 0) v = ld(xz + (int64_t)(lo + pp) * xz_stride + c);
      else if (init) v = ld(st_ + (int64_t)(taps - 1 + pp) * C + c);
      a += ld(w + (int64_t)c * taps + j) * v;
    }
    st(out + (int64_t)(lo + p) * C + c, siluf_(a));
  }
}

// state[j] <- input at run position len - (taps-1) + j (from the run, or from the old state)
template <typename T>
__global__ __launch_bounds__(NT) void conv_state_kernel(const T* __restrict__ xz, int64_t xz_stride, int C, int taps,
                                                       T* __restrict__ state, const int* __restrict__ seq_start,
                                                       const int* __restrict__ seq_slot,
                                                       const int* __restrict__ seq_init) {
  const int c = blockIdx.x * NT + threadIdx.x;
  const int s = blockIdx.y;
  if (c >= C) return;
  const int lo = seq_start[s], len = seq_start[s + 1] - lo;
  const bool init = seq_init[s] != 0;
  T* st_ = state + (int64_t)seq_slot[s] * (taps - 1) * C;
  for (int j = 0; j < taps - 1; ++j) {  // ascending j reads old entries j + len > j not yet rewritten
    const int pp = len - (taps - 1) + j;
    float v = 0.f;
    if (pp >= 0) v = ld(xz + (int64_t)(lo + pp) * xz_stride + c);
    else if (init) v = ld(st_ + (int64_t)(taps - 1 + pp) * C + c);
    st(st_ + (int64_t)j * C + c, v);
  }
}

// NL lanes per channel (power of two <= 64), SPL states per lane.
template <typename T, int SPL>
__global__ __launch_bounds__(NT) void selective_scan_kernel(
    const T* __restrict__ xc, const T* __restrict__ dt_raw, const T* __restrict__ dt_bias,
    const float* __restrict__ A, const T* __restrict__ bc, int64_t bc_stride, int R, int N, const T* __restrict__ D,
    const T* __restrict__ xz, int64_t xz_stride, int C, float* __restrict__ state, const int* __restrict__ seq_start,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_init, T* __restrict__ out, int NL) {
  const int cpb = NT / NL;
  const int c = blockIdx.x * cpb + threadIdx.x / NL;
  const int nl = threadIdx.x % NL;
  const int s = blockIdx.y;
  const int lo = seq_start[s], hi = seq_start[s + 1];
  const bool ok = c < C;
  const int cc = ok ? c : C - 1;  // idle lanes follow the last channel and store nothing
  float* sp = state + ((int64_t)seq_slot[s] * C + cc) * N;
  float S[SPL], Ac[SPL];
#pragma unroll
  for (int i = 0; i < SPL; ++i) {
    const int n = nl + i * NL;
    Ac[i] = n < N ? A[(int64_t)cc * N + n] : 0.f;
    S[i] = (n < N && seq_init[s]) ? sp[n] : 0.f;
  }
  const float bias = ld(dt_bias + cc), Dc = ld(D + cc);
  // inputs are fetched one token ahead of the recurrence
  float ndt = 0.f, nx = 0.f, nz = 0.f, nB[SPL], nC[SPL];
  auto fetch = [&](int t) {
    if (t >= hi) return;
    ndt = ld(dt_raw + (int64_t)t * C + cc);
    nx = ld(xc + (int64_t)t * C + cc);
    nz = ld(xz + (int64_t)t * xz_stride + C + cc);
    const T* bt = bc + (int64_t)t * bc_stride + R;
#pragma unroll
    for (int i = 0; i < SPL; ++i) {
      const int n = nl + i * NL;
      nB[i] = n < N ? ld(bt + n) : 0.f;
      nC[i] = n < N ? ld(bt + N + n) : 0.f;
    }
  };
  fetch(lo);
  for (int t = lo; t < hi; ++t) {
    const float dt = softplusf_(ndt + bias), x = nx, z = nz;
    float Bv[SPL], Cv[SPL];
#pragma unroll
    for (int i = 0; i < SPL; ++i) {
      Bv[i] = nB[i];
      Cv[i] = nC[i];
    }
    fetch(t + 1);
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < SPL; ++i) {
      const int n = nl + i * NL;
      if (n < N) {
        S[i] = expf(dt * Ac[i]) * S[i] + dt * x * Bv[i];
        part += S[i] * Cv[i];
      }
    }
    for (int o = NL >> 1; o > 0; o >>= 1) part += __shfl_xor(part, o, 64);
    if (ok && nl == 0) st(out + (int64_t)t * C + c, (part + Dc * x) * siluf_(z));
  }
  if (ok) {
#pragma unroll
    for (int i = 0; i < SPL; ++i) {
      const int n = nl + i * NL;
      if (n < N) sp[n] = S[i];
    }
  }
}

constexpr float DECAY_K = 0.6065306597126334f;  // exp(-1/2)

// KD >= d key channels per thread column; blockDim = BT (a multiple of 64 >= d).
template <typename T, int KD, int BT>
__global__ __launch_bounds__(BT) void gdelta_scan_kernel(
    const T* __restrict__ proj, int64_t p_stride, const T* __restrict__ wl, const T* __restrict__ w0,
    const T* __restrict__ a_b, const T* __restrict__ norm_w, float eps, int H, int d, float* __restrict__ state,
    const int* __restrict__ seq_start, const int* __restrict__ seq_slot, const int* __restrict__ seq_init,
    T* __restrict__ out) {
  __shared__ __attribute__((aligned(16))) float sw[KD], sau[KD], su[KD], sk[KD], sr[KD];
  __shared__ float red[BT / 64];
  const int h = blockIdx.x, s = blockIdx.y;
  const int j = threadIdx.x;
  const bool col = j < d;
  const int HD = H * d;
  const int lo = seq_start[s], hi = seq_start[s + 1];
  float* sp = state + ((int64_t)seq_slot[s] * H + h) * d * d;
  float S[KD];
  const bool init = seq_init[s] != 0;
#pragma unroll
  for (int i = 0; i < KD; ++i) S[i] = (col && i < d && init) ? sp[(int64_t)i * d + j] : 0.f;
  for (int i = d + j; i < KD; i += BT) sw[i] = sau[i] = su[i] = sk[i] = sr[i] = 0.f;
  const int e = h * d + (col ? j : 0);
  const float w0e = ld(w0 + e), abe = ld(a_b + e), nwe = ld(norm_w + e);
  // the token's seven inputs of this column are fetched one token ahead, so their latency
  // overlaps the previous token's arithmetic and barriers
  float nk = 0.f, na = 0.f, nwl = 0.f, nr = 0.f, nv = 0.f, ng = 0.f;
  auto fetch = [&](int t) {
    if (!col || t >= hi) return;
    const T* pr = proj + (int64_t)t * p_stride;
    nr = ld(pr + e);
    nk = ld(pr + HD + e);
    nv = ld(pr + 2 * HD + e);
    ng = ld(pr + 3 * HD + e);
    na = ld(pr + 4 * HD + e);
    nwl = ld(wl + (int64_t)t * HD + e);
  };
  fetch(lo);
  for (int t = lo; t < hi; ++t) {
    const float kj = nk, aj = na, wlj = nwl, rj = nr, v = nv, gj = ng;
    fetch(t + 1);
    const float ksum = block_sum<BT>(kj * kj, red);  // also fences the previous token's LDS reads
    if (col) {
      const float u = kj / sqrtf(ksum + 1e-6f);
      const float a = sigmoidf_(aj + abe);
      sw[j] = expf(-DECAY_K * sigmoidf_(wlj + w0e));
      sau[j] = a * u;
      su[j] = u;
      sk[j] = kj;
      sr[j] = rj;
    }
    __syncthreads();
    float o = 0.f;
    if (col) {
      // the key-side vectors come as 16-byte LDS broadcasts; entries beyond d are zero
      // (written below), so whole groups of four need no bound
      float sa = 0.f;
#pragma unroll
      for (int i = 0; i < KD; i += 4) {
        if (i < d) {
          const float4 u4 = *reinterpret_cast<const float4*>(&su[i]);
          sa += u4.x * S[i] + u4.y * S[i + 1] + u4.z * S[i + 2] + u4.w * S[i + 3];
        }
      }
#pragma unroll
      for (int i = 0; i < KD; i += 4) {
        if (i < d) {
          const float4 w4 = *reinterpret_cast<const float4*>(&sw[i]);
          const float4 a4 = *reinterpret_cast<const float4*>(&sau[i]);
          const float4 k4 = *reinterpret_cast<const float4*>(&sk[i]);
          const float4 r4 = *reinterpret_cast<const float4*>(&sr[i]);
          S[i] = w4.x * S[i] - a4.x * sa + k4.x * v;
          S[i + 1] = w4.y * S[i + 1] - a4.y * sa + k4.y * v;
          S[i + 2] = w4.z * S[i + 2] - a4.z * sa + k4.z * v;
          S[i + 3] = w4.w * S[i + 3] - a4.w * sa + k4.w * v;
          o += S[i] * r4.x + S[i + 1] * r4.y + S[i + 2] * r4.z + S[i + 3] * r4.w;
        }
      }
    }
    const float ss = block_sum<BT>(o * o, red);
    if (col) st(out + (int64_t)t * HD + e, o / sqrtf(ss / (float)d + eps) * nwe * sigmoidf_(gj));
  }
  if (col) {
#pragma unroll
    for (int i = 0; i < KD; ++i)
      if (i < d) sp[(int64_t)i * d + j] = S[i];
  }
}

}  // namespace

extern "C" {

void sm_causal_conv_silu(const void* xz, int64_t xz_stride, int C, const void* w, const void* b, int taps, void* state,
                         const int* seq_start, const int* seq_slot, const int* seq_init, void* out, int nseq,
                         int max_q, int f32, hipStream_t stream) {
  if (nseq == 0 || max_q == 0) return;
  const int seg = 64;
  const dim3 g1((C + NT - 1) / NT, nseq, (max_q + seg - 1) / seg), g2((C + NT - 1) / NT, nseq);
  if (f32) {
    hipLaunchKernelGGL((conv_silu_kernel<float>), g1, dim3(NT), 0, stream, (const float*)xz, xz_stride, C,
                       (const float*)w, (const float*)b, taps, (const float*)state, seq_start, seq_slot, seq_init,
                       (float*)out, seg);
    if (taps > 1)
      hipLaunchKernelGGL((conv_state_kernel<float>), g2, dim3(NT), 0, stream, (const float*)xz, xz_stride, C, taps,
                         (float*)state, seq_start, seq_slot, seq_init);
  } else {
    hipLaunchKernelGGL((conv_silu_kernel<bf16_t>), g1, dim3(NT), 0, stream, (const bf16_t*)xz, xz_stride, C,
                       (const bf16_t*)w, (const bf16_t*)b, taps, (const bf16_t*)state, seq_start, seq_slot, seq_init,
                       (bf16_t*)out, seg);
    if (taps > 1)
      hipLaunchKernelGGL((conv_state_kernel<bf16_t>), g2, dim3(NT), 0, stream, (const bf16_t*)xz, xz_stride, C, taps,
                         (bf16_t*)state, seq_start, seq_slot, seq_init);
  }
}

// Returns 0, or 1 when the state size does not fit (N > 256).
int sm_selective_scan(const void* xc, const void* dt_raw, const void* dt_bias, const float* A, const void* bc,
                      int64_t bc_stride, int R, int N, const void* D, const void* xz, int64_t xz_stride, int C,
                      float* state, const int* seq_start, const int* seq_slot, const int* seq_init, void* out,
                      int nseq, int f32, hipStream_t stream) {
  if (nseq == 0) return 0;
  int NL = 1;
  while (NL < N && NL < 64) NL <<= 1;
  const int spl = (N + NL - 1) / NL;
  if (spl > 4) return 1;
  const dim3 grid((C + NT / NL - 1) / (NT / NL), nseq);
#define SM_GO(TYPE, SPL)                                                                                              \
  hipLaunchKernelGGL((selective_scan_kernel<TYPE, SPL>), grid, dim3(NT), 0, stream, (const TYPE*)xc,                  \
                     (const TYPE*)dt_raw, (const TYPE*)dt_bias, A, (const TYPE*)bc, bc_stride, R, N, (const TYPE*)D,  \
                     (const TYPE*)xz, xz_stride, C, state, seq_start, seq_slot, seq_init, (TYPE*)out, NL)
  if (f32) {
    if (spl == 1) SM_GO(float, 1);
    else if (spl == 2) SM_GO(float, 2);
    else SM_GO(float, 4);
  } else {
    if (spl == 1) SM_GO(bf16_t, 1);
    else if (spl == 2) SM_GO(bf16_t, 2);
    else SM_GO(bf16_t, 4);
  }
#undef SM_GO
  return 0;
}

// Returns 0, or 1 when the head size does not fit (d > 256).
int sm_gdelta_scan(const void* proj, int64_t p_stride, const void* wl, const void* w0, const void* a_b,
                   const void* norm_w, float eps, int H, int d, float* state, const int* seq_start,
                   const int* seq_slot, const int* seq_init, void* out, int nseq, int f32, hipStream_t stream) {
  if (nseq == 0) return 0;
  const dim3 grid(H, nseq);
#define SM_GO(TYPE, KD, BT)                                                                                       \
  hipLaunchKernelGGL((gdelta_scan_kernel<TYPE, KD, BT>), grid, dim3(BT), 0, stream, (const TYPE*)proj, p_stride,  \
                     (const TYPE*)wl, (const TYPE*)w0, (const TYPE*)a_b, (const TYPE*)norm_w, eps, H, d, state,   \
                     seq_start, seq_slot, seq_init, (TYPE*)out)
  if (f32) {
    if (d <= 32) SM_GO(float, 32, 64);
    else if (d <= 64) SM_GO(float, 64, 64);
    else if (d <= 128) SM_GO(float, 128, 128);
    else if (d <= 256) SM_GO(float, 256, 256);
    else return 1;
  } else {
    if (d <= 32) SM_GO(bf16_t, 32, 64);
    else if (d <= 64) SM_GO(bf16_t, 64, 64);
    else if (d <= 128) SM_GO(bf16_t, 128, 128);
    else if (d <= 256) SM_GO(bf16_t, 256, 256);
    else return 1;
  }
#undef SM_GO
  return 0;
}

}  // extern "C"
