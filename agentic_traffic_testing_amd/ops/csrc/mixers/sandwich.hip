// Sandwich-norm layer boundary, the inverse RMS of whole q / k projections, and scaled,
// soft-capped logits.
//
// * norm_add_norm: one workgroup per row of the fp32 residual x [T, W]:
//     x += norm(y) * w_post          (skipped when y is nullptr)
//     h  = norm(x) * w_next          (skipped when h is nullptr)
//   norm = layer norm without bias, (v - mean) / sqrt(var + eps) with var the mean squared
//   deviation (two passes over registers: the mean first, then the deviations), or RMS norm,
//   v / sqrt(mean(v^2) + eps).  The vector form (W % 8 == 0, W <= 32 * blockDim) keeps the row of
//   y and of x in registers between the passes and issues every load before the first store.
// * proj_inv_rms: one wave per (row, projection): out[t, p] = 1 / sqrt(mean(row^2) + eps) over
//   ALL channels of the q (p = 0) or k (p = 1) projection of row t - the norm that
//   qk_norm_rope_cache then applies per head with weights indexed by the projection's channel.
// * scale_softcap: out = cap * tanh(x * scale / cap) in fp32 (cap 0: x * scale).
#include "mix_common.h"
#include "mixers.h"

namespace mixk {

constexpr int kSwGroups = 4;

// mean (LAYER) and inverse deviation of the values v[g][e] of this block's row; elements at or
// beyond W are not counted (their registers are never read).
template <bool LAYER>
__device__ __forceinline__ void row_stats(float (&v)[kSwGroups][8], int W, float eps,
                                          float* scratch, float& mean, float& inv) {
  mean = 0.f;
  if (LAYER) {
    float s = 0.f;
#pragma unroll
    for (int g = 0; g < kSwGroups; ++g)
      if ((g * blockDim.x + threadIdx.x) * 8 < W)
#pragma unroll
        for (int e = 0; e < 8; ++e) s += v[g][e];
    mean = block_sum(s, scratch) / static_cast<float>(W);
  }
  float ss = 0.f;
#pragma unroll
  for (int g = 0; g < kSwGroups; ++g)
    if ((g * blockDim.x + threadIdx.x) * 8 < W)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = v[g][e] - mean;
        ss += d * d;
      }
  inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(W) + eps);
}

template <typename T, bool LAYER>
__global__ void norm_add_norm_vec_kernel(T* __restrict__ h, float* __restrict__ x,
                                         const T* __restrict__ y, const T* __restrict__ w_post,
                                         const T* __restrict__ w_next, int W, float eps) {
  __shared__ float scratch[16];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * W;
  float xv[kSwGroups][8], yv[kSwGroups][8];
#pragma unroll
  for (int g = 0; g < kSwGroups; ++g) {
    const int i = (g * blockDim.x + threadIdx.x) * 8;
    if (i < W) {
      ld8(x + base + i, xv[g]);
      if (y != nullptr) ld8(y + base + i, yv[g]);
    }
  }
  float mean, inv;
  if (y != nullptr) {
    row_stats<LAYER>(yv, W, eps, scratch, mean, inv);
#pragma unroll
    for (int g = 0; g < kSwGroups; ++g) {
      const int i = (g * blockDim.x + threadIdx.x) * 8;
      if (i < W) {
        float wv[8];
        ld8(w_post + i, wv);
#pragma unroll
        for (int e = 0; e < 8; ++e) xv[g][e] += (yv[g][e] - mean) * inv * wv[e];
        st8(x + base + i, xv[g]);
      }
    }
  }
  if (h == nullptr) return;
  row_stats<LAYER>(xv, W, eps, scratch, mean, inv);
#pragma unroll
  for (int g = 0; g < kSwGroups; ++g) {
    const int i = (g * blockDim.x + threadIdx.x) * 8;
    if (i < W) {
      float wv[8];
      ld8(w_next + i, wv);
#pragma unroll
      for (int e = 0; e < 8; ++e) wv[e] = (xv[g][e] - mean) * inv * wv[e];
      st8(h + base + i, wv);
    }
  }
}

// Any width: the row is re-read from memory in every pass (a thread re-reads only elements it
// wrote itself).
template <typename T, bool LAYER>
__global__ void norm_add_norm_kernel(T* __restrict__ h, float* __restrict__ x,
                                     const T* __restrict__ y, const T* __restrict__ w_post,
                                     const T* __restrict__ w_next, int W, float eps) {
  __shared__ float scratch[16];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * W;
  float* xr = x + base;
  if (y != nullptr) {
    const T* yr = y + base;
    float mean = 0.f;
    if (LAYER) {
      float s = 0.f;
      for (int i = threadIdx.x; i < W; i += blockDim.x) s += ldf(yr + i);
      mean = block_sum(s, scratch) / static_cast<float>(W);
    }
    float ss = 0.f;
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      const float d = ldf(yr + i) - mean;
      ss += d * d;
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(W) + eps);
    for (int i = threadIdx.x; i < W; i += blockDim.x)
      xr[i] += (ldf(yr + i) - mean) * inv * ldf(w_post + i);
  }
  if (h == nullptr) return;
  float mean = 0.f;
  if (LAYER) {
    float s = 0.f;
    for (int i = threadIdx.x; i < W; i += blockDim.x) s += xr[i];
    mean = block_sum(s, scratch) / static_cast<float>(W);
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float d = xr[i] - mean;
    ss += d * d;
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(W) + eps);
  T* hr = h + base;
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    stf(hr + i, (xr[i] - mean) * inv * ldf(w_next + i));
}

template <typename T>
__global__ void proj_inv_rms_kernel(float* __restrict__ out, const T* __restrict__ qx,
                                    int64_t q_stride, int nq, const T* __restrict__ kx,
                                    int64_t k_stride, int nk, int T_, float eps, int vec) {
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (item >= 2 * T_) return;
  const int t = item >> 1, p = item & 1;
  const T* row = p ? kx + t * k_stride : qx + t * q_stride;
  const int n = p ? nk : nq;
  float ss = 0.f;
  if (vec) {
    for (int i = lane * 8; i < n; i += kWave * 8) {
      float v[8];
      ld8(row + i, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += v[e] * v[e];
    }
  } else {
    for (int i = lane; i < n; i += kWave) {
      const float v = ldf(row + i);
      ss += v * v;
    }
  }
  ss = wave_sum(ss);
  if (lane == 0) out[item] = 1.0f / sqrtf(ss / static_cast<float>(n) + eps);
}

template <typename T>
__global__ void scale_softcap_kernel(float* __restrict__ out, const T* __restrict__ x, int64_t n,
                                     float scale, float cap) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float z = ldf(x + i) * scale;
  out[i] = cap > 0.f ? cap * tanhf(z / cap) : z;
}

static int sandwich_threads(int W) {
  if (W % 8 != 0 || W > 8 * kSwGroups * 1024) return 0;
  int t = 64;
  while (t < 1024 && t * 8 * kSwGroups < W) t <<= 1;
  if (W >= 2048 && t < 256) t = 256;
  return t;
}

static bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
static bool al32(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 31) == 0; }

}  // namespace mixk

using namespace mixk;

extern "C" int mixk_norm_add_norm(void* h, float* x, const void* y, const void* w_post,
                                  const void* w_next, int T_, int W, float eps, int layer,
                                  int dtype, hipStream_t st) {
  if (T_ <= 0 || W <= 0) return 0;
  if ((y != nullptr && w_post == nullptr) || (h != nullptr && w_next == nullptr)) return -1;
  int threads = sandwich_threads(W);
  // 16-byte loads of the activation rows, 32-byte pairs of the fp32 residual
  if (!(al32(x) && (h == nullptr || al16(h)) && (y == nullptr || al16(y)) &&
        (w_post == nullptr || al16(w_post)) && (w_next == nullptr || al16(w_next))) ||
      (dtype == 2 && !((h == nullptr || al32(h)) && (y == nullptr || al32(y)) &&
                       (w_post == nullptr || al32(w_post)) && (w_next == nullptr || al32(w_next)))))
    threads = 0;
#define MIXK_SANDWICH(KERNEL, LAYER, THREADS)                                                    \
  hipLaunchKernelGGL((KERNEL<T, LAYER>), dim3(T_), dim3(THREADS), 0, st, static_cast<T*>(h), x,  \
                     static_cast<const T*>(y), static_cast<const T*>(w_post),                    \
                     static_cast<const T*>(w_next), W, eps)
  MIXK_DISPATCH(dtype, {
    if (threads && layer)
      MIXK_SANDWICH(norm_add_norm_vec_kernel, true, threads);
    else if (threads)
      MIXK_SANDWICH(norm_add_norm_vec_kernel, false, threads);
    else if (layer)
      MIXK_SANDWICH(norm_add_norm_kernel, true, 256);
    else
      MIXK_SANDWICH(norm_add_norm_kernel, false, 256);
  });
#undef MIXK_SANDWICH
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_proj_inv_rms(float* out, const void* qx, int64_t q_stride, int nq,
                                 const void* kx, int64_t k_stride, int nk, int T_, float eps,
                                 int dtype, hipStream_t st) {
  if (T_ <= 0) return 0;
  if (nq <= 0 || nk <= 0) return -1;
  const bool wide = dtype == 2;
  const int vec = nq % 8 == 0 && nk % 8 == 0 && q_stride % 8 == 0 && k_stride % 8 == 0 &&
                  (wide ? al32(qx) && al32(kx) : al16(qx) && al16(kx));
  MIXK_DISPATCH(dtype,
                hipLaunchKernelGGL(proj_inv_rms_kernel<T>, dim3((2 * T_ + 3) / 4), dim3(256), 0, st,
                                   out, static_cast<const T*>(qx), q_stride, nq,
                                   static_cast<const T*>(kx), k_stride, nk, T_, eps, vec));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_scale_softcap(float* out, const void* x, int64_t n, float scale, float cap,
                                  int dtype, hipStream_t st) {
  if (n <= 0) return 0;
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(scale_softcap_kernel<T>,
                                          dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256),
                                          0, st, out, static_cast<const T*>(x), n, scale, cap));
  return static_cast<int>(hipGetLastError());
}
