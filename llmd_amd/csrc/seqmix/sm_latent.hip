// Latent attention of any size over a paged latent cache (one row [latent R | rotated key dr]
// per token, shared by all heads).
//
// latent_rope_cache: rotate the query's rotary part (rotate-half pairs over the first
//   rot_dims dimensions, angles from an fp32 cos/sin table) into the absorbed query, RMS-norm the
//   latent with its plain weight, rotate the shared key part and write the cache row.
// latent_attention: one workgroup = QT consecutive token rows x 4 heads (one wave per head).
//   Keys stream through LDS in tiles of KT rows (fp32) shared by all 4 x QT (row, head) pairs;
//   a lane scores one key (dot over R + dr from LDS), the wave keeps an online softmax per pair,
//   and the lanes then own output columns for the P x latent product. Scores, softmax and the
//   accumulators are fp32. A row's result depends only on its own keys and the fixed tile
//   size, never on what else is in the step.
#include "seqmix_common.h"

using namespace sm;

namespace {

constexpr int NT = 256;

template <typename T>
__global__ __launch_bounds__(NT) void latent_rope_cache_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ kv, int64_t kv_stride,
    const T* __restrict__ norm_w, float eps, const int64_t* __restrict__ positions,
    const float* __restrict__ cos_sin, int H, int dn, int dr, int rot_dims, int R,
    const int64_t* __restrict__ slots, T* __restrict__ cache, T* __restrict__ q_abs) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const int half = rot_dims >> 1;
  const float* cs = cos_sin + positions[t] * rot_dims;  // [cos(half) | sin(half)]
  const int Dk = R + dr;
  // query: rotary part of every head -> q_abs[t, h, R + i]
  for (int e = threadIdx.x; e < H * dr; e += NT) {
    const int h = e / dr, i = e - h * dr;
    const T* src = q + t * q_stride + (int64_t)h * (dn + dr) + dn;
    float v;
    if (i < half) v = ld(src + i) * cs[i] - ld(src + i + half) * cs[half + i];
    else if (i < rot_dims) v = ld(src + i) * cs[i - half] + ld(src + i - half) * cs[i];
    else v = ld(src + i);
    st(q_abs + (t * H + h) * Dk + R + i, v);
  }
  // latent: RMS norm with a plain weight
  const T* kr = kv + t * kv_stride;
  float ss = 0.f;
  for (int c = threadIdx.x; c < R; c += NT) {
    const float v = ld(kr + c);
    ss += v * v;
  }
  ss = block_sum<NT>(ss, red);
  const int64_t slot = slots[t];
  if (slot < 0) return;
  const float inv = 1.f / sqrtf(ss / (float)R + eps);
  T* row = cache + slot * Dk;
  for (int c = threadIdx.x; c < R; c += NT) st(row + c, ld(kr + c) * inv * ld(norm_w + c));
  const T* src = kr + R;
  for (int i = threadIdx.x; i < dr; i += NT) {
    float v;
    if (i < half) v = ld(src + i) * cs[i] - ld(src + i + half) * cs[half + i];
    else if (i < rot_dims) v = ld(src + i) * cs[i - half] + ld(src + i - half) * cs[i];
    else v = ld(src + i);
    st(row + R + i, v);
  }
}

// RC = ceil(R / 64) output columns per lane; QT token rows per workgroup.
template <typename T, int RC, int QT>
__global__ __launch_bounds__(NT) void latent_attention_kernel(
    const T* __restrict__ q_abs, const T* __restrict__ cache, const int* __restrict__ tables, int W, int bs,
    const int* __restrict__ row_seq, const int* __restrict__ row_len, float scale, int H, int R, int Dk, int KT,
    int T_rows, T* __restrict__ out) {
  extern __shared__ float lds[];
  const int KS = Dk + 1;                 // key row stride in LDS (odd: lanes hit distinct banks)
  float* sK = lds;                       // [KT][KS]
  float* sQ = lds + KT * KS;             // [QT][4][Dk], pre-scaled
  const int t0 = blockIdx.x * QT;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h = blockIdx.y * 4 + wave;
  const bool head_ok = h < H;

  for (int e = threadIdx.x; e < QT * 4 * Dk; e += NT) {
    const int r = e / (4 * Dk), rem = e - r * 4 * Dk;
    const int w = rem / Dk, d = rem - w * Dk;
    const int t = t0 + r, hh = blockIdx.y * 4 + w;
    sQ[e] = (t < T_rows && hh < H) ? ld(q_abs + ((int64_t)t * H + hh) * Dk + d) * scale : 0.f;
  }

  int seq_r[QT], len_r[QT];
  bool done[QT];
#pragma unroll
  for (int r = 0; r < QT; ++r) {
    const int t = t0 + r;
    done[r] = t >= T_rows;
    seq_r[r] = done[r] ? -1 : row_seq[t];
    len_r[r] = done[r] ? 0 : row_len[t];
  }

  for (int pass = 0; pass < QT; ++pass) {
    // rows of this pass: those of the first unfinished row's sequence
    int seq = -1;
#pragma unroll
    for (int r = 0; r < QT; ++r)
      if (seq < 0 && !done[r]) seq = seq_r[r];
    if (seq < 0) break;
    bool act[QT];
    int maxlen = 0;
#pragma unroll
    for (int r = 0; r < QT; ++r) {
      act[r] = !done[r] && seq_r[r] == seq;
      if (act[r]) maxlen = max(maxlen, len_r[r]);
    }
    float m[QT], l[QT], acc[QT][RC];
#pragma unroll
    for (int r = 0; r < QT; ++r) {
      m[r] = -INFINITY;
      l[r] = 0.f;
#pragma unroll
      for (int c = 0; c < RC; ++c) acc[r][c] = 0.f;
    }
    const int* bt = tables + (int64_t)seq * W;
    for (int k0 = 0; k0 < maxlen; k0 += KT) {
      __syncthreads();  // previous tile fully used (and sQ written, first time)
      for (int e = threadIdx.x; e < KT * Dk; e += NT) {
        const int j = e / Dk, d = e - j * Dk;
        const int key = k0 + j;
        float v = 0.f;
        if (key < maxlen) {
          const int64_t rowi = (int64_t)bt[key / bs] * bs + (key % bs);
          v = ld(cache + rowi * Dk + d);
        }
        sK[j * KS + d] = v;
      }
      __syncthreads();
      if (!head_ok) continue;
#pragma unroll
      for (int r = 0; r < QT; ++r) {
        if (!act[r] || k0 >= len_r[r]) continue;
        const bool valid = lane < KT && k0 + lane < len_r[r];
        float s = -INFINITY;
        if (valid) {
          const float* qv = sQ + (r * 4 + wave) * Dk;
          const float* kr = sK + lane * KS;
          float a = 0.f;
          for (int d = 0; d < Dk; ++d) a += qv[d] * kr[d];
          s = a;
        }
        const float mn = fmaxf(m[r], wave_max(s));
        const float corr = expf(m[r] - mn);  // exp(-inf) = 0 on the first tile
        const float p = valid ? expf(s - mn) : 0.f;
        l[r] = l[r] * corr + wave_sum(p);
        m[r] = mn;
#pragma unroll
        for (int c = 0; c < RC; ++c) acc[r][c] *= corr;
        const int nk = min(KT, len_r[r] - k0);
        for (int j = 0; j < nk; ++j) {
          const float pj = __shfl(p, j, 64);
          const float* kr = sK + j * KS;
#pragma unroll
          for (int c = 0; c < RC; ++c) {
            const int col = lane + 64 * c;
            if (col < R) acc[r][c] += pj * kr[col];
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < QT; ++r) {
      if (!act[r]) continue;
      done[r] = true;
      if (!head_ok) continue;
      const float inv = 1.f / l[r];
#pragma unroll
      for (int c = 0; c < RC; ++c) {
        const int col = lane + 64 * c;
        if (col < R) st(out + ((int64_t)(t0 + r) * H + h) * R + col, acc[r][c] * inv);
      }
    }
  }
}

template <typename T, int RC>
int launch_attn(const void* q_abs, const void* cache, const int* tables, int W, int bs, const int* row_seq,
                const int* row_len, float scale, int H, int R, int Dk, int T_rows, int QT, void* out,
                hipStream_t stream) {
  // key tile: as many of 64 / 32 / 16 rows as fit beside the queries in 128 KB of LDS
  int KT = 64;
  while (KT > 16 && ((size_t)KT * (Dk + 1) + (size_t)QT * 4 * Dk) * 4 > 128 * 1024) KT >>= 1;
  const size_t lds = ((size_t)KT * (Dk + 1) + (size_t)QT * 4 * Dk) * 4;
  if (lds > 160 * 1024) return 1;
  const dim3 grid((T_rows + QT - 1) / QT, (H + 3) / 4);
  auto go = [&](auto kern) {
    if (lds > 64 * 1024) (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(kern, grid, dim3(NT), lds, stream, (const T*)q_abs, (const T*)cache, tables, W, bs, row_seq,
                       row_len, scale, H, R, Dk, KT, T_rows, (T*)out);
  };
  if (QT == 4) go(latent_attention_kernel<T, RC, 4>);
  else go(latent_attention_kernel<T, RC, 1>);
  return 0;
}

}  // namespace

extern "C" {

void sm_latent_rope_cache(const void* q, int64_t q_stride, const void* kv, int64_t kv_stride, const void* norm_w,
                          float eps, const int64_t* positions, const float* cos_sin, int H, int dn, int dr,
                          int rot_dims, int R, const int64_t* slots, void* cache, void* q_abs, int T, int f32,
                          hipStream_t stream) {
  if (T == 0) return;
  if (f32)
    hipLaunchKernelGGL((latent_rope_cache_kernel<float>), dim3(T), dim3(NT), 0, stream, (const float*)q, q_stride,
                       (const float*)kv, kv_stride, (const float*)norm_w, eps, positions, cos_sin, H, dn, dr,
                       rot_dims, R, slots, (float*)cache, (float*)q_abs);
  else
    hipLaunchKernelGGL((latent_rope_cache_kernel<bf16_t>), dim3(T), dim3(NT), 0, stream, (const bf16_t*)q, q_stride,
                       (const bf16_t*)kv, kv_stride, (const bf16_t*)norm_w, eps, positions, cos_sin, H, dn, dr,
                       rot_dims, R, slots, (bf16_t*)cache, (bf16_t*)q_abs);
}

// Returns 0, or 1 when the sizes do not fit the kernel (R > 1024 or rows too wide for LDS).
int sm_latent_attention(const void* q_abs, const void* cache, const int* tables, int W, int bs, const int* row_seq,
                        const int* row_len, float scale, int H, int R, int Dk, int T, int QT, void* out, int f32,
                        hipStream_t stream) {
  if (T == 0) return 0;
  const int rc = (R + 63) / 64;
#define SM_GO(TYPE, RC) return launch_attn<TYPE, RC>(q_abs, cache, tables, W, bs, row_seq, row_len, scale, H, R, Dk, T, QT, out, stream)
  if (f32) {
    if (rc <= 1) SM_GO(float, 1);
    if (rc <= 2) SM_GO(float, 2);
    if (rc <= 4) SM_GO(float, 4);
    if (rc <= 8) SM_GO(float, 8);
    if (rc <= 16) SM_GO(float, 16);
  } else {
    if (rc <= 1) SM_GO(bf16_t, 1);
    if (rc <= 2) SM_GO(bf16_t, 2);
    if (rc <= 4) SM_GO(bf16_t, 4);
    if (rc <= 8) SM_GO(bf16_t, 8);
    if (rc <= 16) SM_GO(bf16_t, 16);
  }
#undef SM_GO
  return 1;
}

}  // extern "C"
