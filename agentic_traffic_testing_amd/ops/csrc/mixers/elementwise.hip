// Embeddings (token + hashed token-pair rows; token rows times a constant), fp32-residual RMS
// norm, RMS norm of activation rows, squared ReLU and xIELU (with bias), the residual sum of a
// layer's branches, the gated per-head output norm of the delta rule, the gate-then-norm of
// grouped fp32 rows, and the per-head sigmoid output gate of latent attention.
#include "mix_common.h"
#include "mixers.h"

namespace mixk {

// One block per row.  The token before a portion's first row is the sequence's state
// (prev_token[slot]); the block of that first row reads it and then replaces it with the
// portion's last token, so no other block touches the slot's entry in this launch.
template <typename T>
__global__ void embed_pair_kernel(float* __restrict__ out, const T* __restrict__ table,
                                  const T* __restrict__ pair, const int* __restrict__ ids,
                                  const int* __restrict__ positions,
                                  const int* __restrict__ seq_qstart,
                                  const int* __restrict__ seq_slot, int* __restrict__ prev_token,
                                  int S, int W, int64_t mul_prev, int64_t mul_cur,
                                  int64_t buckets) {
  __shared__ int64_t sh_row;
  __shared__ int sh_ok;
  const int r = blockIdx.x;
  if (threadIdx.x == 0) {
    const int s = seq_of_row(seq_qstart, S, r);
    const int slot = s < 0 ? -1 : seq_slot[s];
    sh_ok = slot >= 0;
    if (slot >= 0) {
      const int first = seq_qstart[s];
      const int64_t id = ids[r];
      int64_t row = buckets;
      if (positions[r] != 0) {
        const int64_t prev = r == first ? prev_token[slot] : ids[r - 1];
        row = (prev * mul_prev + id * mul_cur) % buckets;
      }
      sh_row = row;
      if (r == first) prev_token[slot] = ids[seq_qstart[s + 1] - 1];
    }
  }
  __syncthreads();
  float* o = out + static_cast<int64_t>(r) * W;
  if (!sh_ok) {
    for (int i = threadIdx.x; i < W; i += blockDim.x) o[i] = 0.f;
    return;
  }
  const T* e = table + static_cast<int64_t>(ids[r]) * W;
  const T* p = pair + sh_row * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) o[i] = ldf(e + i) + ldf(p + i);
}

template <typename T>
__global__ void rms_norm_f32_kernel(T* __restrict__ out, const float* __restrict__ x,
                                    const T* __restrict__ w, int W, float eps, float plus) {
  __shared__ float scratch[16];
  const float* xr = x + static_cast<int64_t>(blockIdx.x) * W;
  T* o = out + static_cast<int64_t>(blockIdx.x) * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) ss += xr[i] * xr[i];
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(W) + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) stf(o + i, xr[i] * inv * (ldf(w + i) + plus));
}

// Vector forms for W % 8 == 0, W <= 8 * 4 * blockDim: every thread keeps its (up to 4) groups of
// 8 elements in registers between the sum and the scaling pass, all loads issued up front.
constexpr int kNormGroups = 4;

template <typename T, bool ADD>
__global__ void norm_vec_kernel(T* __restrict__ h, float* __restrict__ x, const T* __restrict__ a,
                                float sa, const T* __restrict__ b, float sb,
                                const T* __restrict__ c, const T* __restrict__ w, int W, float eps,
                                float plus) {
  __shared__ float scratch[16];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * W;
  float xv[kNormGroups][8];
  float ss = 0.f;
#pragma unroll
  for (int g = 0; g < kNormGroups; ++g) {
    const int i = (g * blockDim.x + threadIdx.x) * 8;
    if (i < W) {
      ld8(x + base + i, xv[g]);
      if (ADD) {
        float t[8];
        ld8(a + base + i, t);
#pragma unroll
        for (int e = 0; e < 8; ++e) t[e] *= sa;
        if (b != nullptr) {
          float u[8];
          ld8(b + base + i, u);
#pragma unroll
          for (int e = 0; e < 8; ++e) t[e] += u[e] * sb;
        }
        if (c != nullptr) {
          float u[8];
          ld8(c + base + i, u);
#pragma unroll
          for (int e = 0; e < 8; ++e) t[e] += u[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) xv[g][e] += t[e];
        st8(x + base + i, xv[g]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += xv[g][e] * xv[g][e];
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(W) + eps);
#pragma unroll
  for (int g = 0; g < kNormGroups; ++g) {
    const int i = (g * blockDim.x + threadIdx.x) * 8;
    if (i < W) {
      float wv[8];
      ld8(w + i, wv);
#pragma unroll
      for (int e = 0; e < 8; ++e) wv[e] = xv[g][e] * inv * (wv[e] + plus);
      st8(h + base + i, wv);
    }
  }
}

// block size of the vector norm kernels for width W (0: use the scalar kernel)
static int norm_vec_threads(int W) {
  if (W % 8 != 0 || W > 8 * kNormGroups * 1024) return 0;
  int t = 64;
  while (t < 1024 && t * 8 * kNormGroups < W) t <<= 1;
  if (W >= 2048 && t < 256) t = 256;
  return t;
}

template <typename T>
__global__ void relu_sq_vec_kernel(T* __restrict__ out, const T* __restrict__ x, int N,
                                   int64_t x_stride) {
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (i >= N) return;
  float v[8];
  ld8(x + blockIdx.x * x_stride + i, v);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float r = fmaxf(v[e], 0.f);
    v[e] = r * r;
  }
  st8(out + static_cast<int64_t>(blockIdx.x) * N + i, v);
}

template <typename T>
__global__ void relu_sq_kernel(T* __restrict__ out, const T* __restrict__ x, int N,
                               int64_t x_stride) {
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= N) return;
  const float v = fmaxf(ldf(x + blockIdx.x * x_stride + i), 0.f);
  stf(out + static_cast<int64_t>(blockIdx.x) * N + i, v * v);
}

template <typename T>
__global__ void residual_add_kernel(float* __restrict__ x, const T* __restrict__ a, float sa,
                                    const T* __restrict__ b, float sb, const T* __restrict__ c,
                                    int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float y = ldf(a + i) * sa;
  if (b != nullptr) y += ldf(b + i) * sb;
  if (c != nullptr) y += ldf(c + i);
  x[i] += y;
}

// Layer boundary in one pass over the row: x += sa a [+ sb b] [+ c] (fp32, in place), then the
// next layer's norm of the new x: h = x / sqrt(mean(x^2) + eps) * (w + plus).
template <typename T>
__global__ void add_norm_kernel(T* __restrict__ h, float* __restrict__ x, const T* __restrict__ a,
                                float sa, const T* __restrict__ b, float sb,
                                const T* __restrict__ c, const T* __restrict__ w, int W, float eps,
                                float plus) {
  __shared__ float scratch[16];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float y = ldf(a + base + i) * sa;
    if (b != nullptr) y += ldf(b + base + i) * sb;
    if (c != nullptr) y += ldf(c + base + i);
    const float v = x[base + i] + y;
    x[base + i] = v;
    ss += v * v;
  }
  ss = block_sum(ss, scratch);   // also orders this thread's writes of x before its re-reads
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(W) + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    stf(h + base + i, x[base + i] * inv * (ldf(w + i) + plus));
}

// One wave per (row, head): o / sqrt(mean(o^2) + eps) * w * act(gate).
template <typename T>
__global__ void gated_rms_norm_kernel(T* __restrict__ out, const float* __restrict__ o,
                                      const T* __restrict__ gate, int64_t gate_stride,
                                      const T* __restrict__ w, int H, int dv, float eps, int act) {
  const int t = blockIdx.x / H, h = blockIdx.x % H;
  const float* orow = o + (static_cast<int64_t>(t) * H + h) * dv;
  const T* g = gate + t * gate_stride + h * dv;
  T* y = out + (static_cast<int64_t>(t) * H + h) * dv;
  float ss = 0.f;
  for (int i = threadIdx.x; i < dv; i += kWave) ss += orow[i] * orow[i];
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(dv) + eps);
  for (int i = threadIdx.x; i < dv; i += kWave) {
    const float gv = ldf(g + i);
    const float ga = act == 1 ? sigmoidf_(gv) : siluf_(gv);
    stf(y + i, orow[i] * inv * ldf(w + i) * ga);
  }
}


// Token embedding times a constant into the fp32 residual stream, `copies` times per row (the
// streams of a multi-stream residual all start as the embedding); one block per row.
template <typename T>
__global__ void embed_scale_kernel(float* __restrict__ out, const T* __restrict__ table,
                                   const int* __restrict__ ids, int W, int vocab, float scale,
                                   int copies) {
  const int id = ids[blockIdx.x];
  float* o = out + static_cast<int64_t>(blockIdx.x) * copies * W;
  const bool ok = id >= 0 && id < vocab;
  const T* e = table + static_cast<int64_t>(ok ? id : 0) * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float v = ok ? ldf(e + i) * scale : 0.f;
    for (int c = 0; c < copies; ++c) o[c * W + i] = v;
  }
}

// RMS norm with a plain weight over rows of activations (row-strided input): one wave per row.
template <typename T>
__global__ void rms_norm_rows_kernel(T* __restrict__ out, const T* __restrict__ x,
                                     int64_t x_stride, const T* __restrict__ w, int T_, int N,
                                     float eps) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= T_) return;
  const T* xr = x + t * x_stride;
  float ss = 0.f;
  for (int i = lane; i < N; i += kWave) {
    const float v = ldf(xr + i);
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(N) + eps);
  T* o = out + static_cast<int64_t>(t) * N;
  for (int i = lane; i < N; i += kWave) stf(o + i, ldf(xr + i) * inv * ldf(w + i));
}

// xIELU on z = x + bias: z > 0: ap z^2 + z / 2;  z <= 0: (1/2 + aq) (exp(z) - 1 - z) + z / 2,
// with ap, aq the (positive) softplus of the layer's two learned numbers.
__device__ __forceinline__ float xielu_(float z, float ap, float aq) {
  return z > 0.f ? ap * z * z + 0.5f * z : (0.5f + aq) * (expm1f(z) - z) + 0.5f * z;
}

template <typename T>
__global__ void xielu_bias_kernel(T* __restrict__ out, const T* __restrict__ x, int64_t x_stride,
                                  const T* __restrict__ bias, int N, float ap, float aq) {
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= N) return;
  const float z = ldf(x + blockIdx.x * x_stride + i) + (bias != nullptr ? ldf(bias + i) : 0.f);
  stf(out + static_cast<int64_t>(blockIdx.x) * N + i, xielu_(z, ap, aq));
}

template <typename T>
__global__ void xielu_bias_vec_kernel(T* __restrict__ out, const T* __restrict__ x,
                                      int64_t x_stride, const T* __restrict__ bias, int N,
                                      float ap, float aq) {
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (i >= N) return;
  float v[8], b[8];
  ld8(x + blockIdx.x * x_stride + i, v);
  if (bias != nullptr) {
    ld8(bias + i, b);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] += b[e];
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = xielu_(v[e], ap, aq);
  st8(out + static_cast<int64_t>(blockIdx.x) * N + i, v);
}

// RMS norm of fp32 rows in equal groups, with an optional SiLU gate applied BEFORE the norm:
// u = y * silu(gate) (or y), out = u / sqrt(mean_group(u^2) + eps) * w.  One wave per
// (row, group); w has `gs` entries (shared by the groups) or n_groups * gs (w_full).
template <typename T>
__global__ void group_rms_norm_kernel(T* __restrict__ out, const float* __restrict__ y,
                                      const T* __restrict__ gate, int64_t gate_stride,
                                      const T* __restrict__ w, int T_, int n_groups, int gs,
                                      float eps, int w_full) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (idx >= static_cast<int64_t>(T_) * n_groups) return;
  const int t = static_cast<int>(idx / n_groups), g = static_cast<int>(idx % n_groups);
  const float* yr = y + (static_cast<int64_t>(t) * n_groups + g) * gs;
  const T* gr = gate != nullptr ? gate + t * gate_stride + static_cast<int64_t>(g) * gs : nullptr;
  float ss = 0.f;
  for (int i = lane; i < gs; i += kWave) {
    const float u = gr != nullptr ? yr[i] * siluf_(ldf(gr + i)) : yr[i];
    ss += u * u;
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(gs) + eps);
  T* o = out + (static_cast<int64_t>(t) * n_groups + g) * gs;
  const T* wr = w + (w_full ? static_cast<int64_t>(g) * gs : 0);
  for (int i = lane; i < gs; i += kWave) {
    const float u = gr != nullptr ? yr[i] * siluf_(ldf(gr + i)) : yr[i];
    stf(o + i, u * inv * ldf(wr + i));
  }
}

// The same for wide groups: one workgroup per (row, group), every thread keeps its (up to 4)
// chunks of 8 gated values in registers between the sum and the scaling pass.
template <typename T>
__global__ void group_rms_norm_vec_kernel(T* __restrict__ out, const float* __restrict__ y,
                                          const T* __restrict__ gate, int64_t gate_stride,
                                          const T* __restrict__ w, int n_groups, int gs, float eps,
                                          int w_full) {
  __shared__ float scratch[16];
  const int t = blockIdx.x / n_groups, g = blockIdx.x % n_groups;
  const int64_t base = (static_cast<int64_t>(t) * n_groups + g) * gs;
  const T* gr = gate != nullptr ? gate + t * gate_stride + static_cast<int64_t>(g) * gs : nullptr;
  float u[kNormGroups][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < kNormGroups; ++c) {
    const int i = (c * blockDim.x + threadIdx.x) * 8;
    if (i < gs) {
      ld8(y + base + i, u[c]);
      if (gr != nullptr) {
        float gv[8];
        ld8(gr + i, gv);
#pragma unroll
        for (int e = 0; e < 8; ++e) u[c][e] *= siluf_(gv[e]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += u[c][e] * u[c][e];
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(gs) + eps);
  const T* wr = w + (w_full ? static_cast<int64_t>(g) * gs : 0);
#pragma unroll
  for (int c = 0; c < kNormGroups; ++c) {
    const int i = (c * blockDim.x + threadIdx.x) * 8;
    if (i < gs) {
      float wv[8];
      ld8(wr + i, wv);
#pragma unroll
      for (int e = 0; e < 8; ++e) wv[e] *= u[c][e] * inv;
      st8(out + base + i, wv);
    }
  }
}

// Per-head sigmoid output gate with the head-major to row-major move:
// out[t, h, :] = o[h, t, :] * sigmoid(gate[t, h]).
template <typename T>
__global__ void head_gate_kernel(T* __restrict__ out, const T* __restrict__ o,
                                 const T* __restrict__ gate, int64_t gate_stride, int T_, int H,
                                 int dv) {
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < H * dv; i += blockDim.x) {
    const int h = i / dv, j = i - h * dv;
    const float gv = sigmoidf_(ldf(gate + t * gate_stride + h));
    stf(out + static_cast<int64_t>(t) * H * dv + i,
        ldf(o + (static_cast<int64_t>(h) * T_ + t) * dv + j) * gv);
  }
}

}  // namespace mixk

using namespace mixk;

extern "C" int mixk_embed_pair(float* out, const void* table, const void* pair_table,
                               const int* ids, const int* positions, const int* seq_qstart,
                               const int* seq_slot, int* prev_token, int T_, int S, int W,
                               int64_t mul_prev, int64_t mul_cur, int64_t buckets, int dtype,
                               hipStream_t st) {
  if (T_ <= 0) return 0;
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(embed_pair_kernel<T>, dim3(T_), dim3(256), 0, st, out,
                                          static_cast<const T*>(table),
                                          static_cast<const T*>(pair_table), ids, positions,
                                          seq_qstart, seq_slot, prev_token, S, W, mul_prev,
                                          mul_cur, buckets));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_rms_norm_f32(void* out, const float* x, const void* w, int T_, int W,
                                 float eps, int one_plus, int dtype, hipStream_t st) {
  if (T_ <= 0) return 0;
  if (const int nt = norm_vec_threads(W)) {
    MIXK_DISPATCH(dtype, hipLaunchKernelGGL((norm_vec_kernel<T, false>), dim3(T_), dim3(nt), 0, st,
                                            static_cast<T*>(out), const_cast<float*>(x),
                                            static_cast<const T*>(nullptr), 0.f,
                                            static_cast<const T*>(nullptr), 0.f,
                                            static_cast<const T*>(nullptr),
                                            static_cast<const T*>(w), W, eps,
                                            one_plus ? 1.0f : 0.0f));
    return static_cast<int>(hipGetLastError());
  }
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(rms_norm_f32_kernel<T>, dim3(T_), dim3(256), 0, st,
                                          static_cast<T*>(out), x, static_cast<const T*>(w), W,
                                          eps, one_plus ? 1.0f : 0.0f));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_relu_sq(void* out, const void* x, int T_, int N, int64_t x_stride, int dtype,
                            hipStream_t st) {
  if (T_ <= 0 || N <= 0) return 0;
  if (N % 8 == 0 && x_stride % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
    MIXK_DISPATCH(dtype, hipLaunchKernelGGL(relu_sq_vec_kernel<T>, dim3(T_, (N / 8 + 255) / 256),
                                            dim3(256), 0, st, static_cast<T*>(out),
                                            static_cast<const T*>(x), N, x_stride));
    return static_cast<int>(hipGetLastError());
  }
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(relu_sq_kernel<T>, dim3(T_, (N + 255) / 256), dim3(256),
                                          0, st, static_cast<T*>(out), static_cast<const T*>(x), N,
                                          x_stride));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_residual_add(float* x, const void* a, float sa, const void* b, float sb,
                                 const void* c, int64_t n, int dtype, hipStream_t st) {
  if (n <= 0) return 0;
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(residual_add_kernel<T>,
                                          dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256),
                                          0, st, x, static_cast<const T*>(a), sa,
                                          static_cast<const T*>(b), sb, static_cast<const T*>(c),
                                          n));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_add_norm(void* h, float* x, const void* a, float sa, const void* b, float sb,
                             const void* c, const void* w, int T_, int W, float eps, int one_plus,
                             int dtype, hipStream_t st) {
  if (T_ <= 0) return 0;
  if (const int nt = norm_vec_threads(W)) {
    MIXK_DISPATCH(dtype, hipLaunchKernelGGL((norm_vec_kernel<T, true>), dim3(T_), dim3(nt), 0, st,
                                            static_cast<T*>(h), x, static_cast<const T*>(a), sa,
                                            static_cast<const T*>(b), sb, static_cast<const T*>(c),
                                            static_cast<const T*>(w), W, eps,
                                            one_plus ? 1.0f : 0.0f));
    return static_cast<int>(hipGetLastError());
  }
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(add_norm_kernel<T>, dim3(T_), dim3(256), 0, st,
                                          static_cast<T*>(h), x, static_cast<const T*>(a), sa,
                                          static_cast<const T*>(b), sb, static_cast<const T*>(c),
                                          static_cast<const T*>(w), W, eps,
                                          one_plus ? 1.0f : 0.0f));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_gated_rms_norm(void* out, const float* o, const void* gate,
                                   int64_t gate_stride, const void* w, int T_, int H, int dv,
                                   float eps, int act, int dtype, hipStream_t st) {
  if (T_ <= 0) return 0;
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(gated_rms_norm_kernel<T>, dim3(T_ * H), dim3(kWave), 0,
                                          st, static_cast<T*>(out), o,
                                          static_cast<const T*>(gate), gate_stride,
                                          static_cast<const T*>(w), H, dv, eps, act));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_embed_scale(float* out, const void* table, const int* ids, int T_, int W,
                                int vocab, float scale, int copies, int dtype, hipStream_t st) {
  if (T_ <= 0) return 0;
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(embed_scale_kernel<T>, dim3(T_), dim3(256), 0, st, out,
                                          static_cast<const T*>(table), ids, W, vocab, scale,
                                          copies));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_rms_norm_rows(void* out, const void* x, int64_t x_stride, const void* w,
                                  int T_, int N, float eps, int dtype, hipStream_t st) {
  if (T_ <= 0) return 0;
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(rms_norm_rows_kernel<T>, dim3((T_ + 3) / 4), dim3(256),
                                          0, st, static_cast<T*>(out), static_cast<const T*>(x),
                                          x_stride, static_cast<const T*>(w), T_, N, eps));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_xielu_bias(void* out, const void* x, int64_t x_stride, const void* bias,
                               int T_, int N, float ap, float aq, int dtype, hipStream_t st) {
  if (T_ <= 0 || N <= 0) return 0;
  const bool vec = N % 8 == 0 && x_stride % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(bias) % 16 == 0;
  MIXK_DISPATCH(dtype, {
    if (vec)
      hipLaunchKernelGGL(xielu_bias_vec_kernel<T>, dim3(T_, (N / 8 + 255) / 256), dim3(256), 0, st,
                         static_cast<T*>(out), static_cast<const T*>(x), x_stride,
                         static_cast<const T*>(bias), N, ap, aq);
    else
      hipLaunchKernelGGL(xielu_bias_kernel<T>, dim3(T_, (N + 255) / 256), dim3(256), 0, st,
                         static_cast<T*>(out), static_cast<const T*>(x), x_stride,
                         static_cast<const T*>(bias), N, ap, aq);
  });
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_group_rms_norm(void* out, const float* y, const void* gate,
                                   int64_t gate_stride, const void* w, int T_, int n_groups,
                                   int gs, float eps, int w_full, int dtype, hipStream_t st) {
  if (T_ <= 0) return 0;
  const int64_t waves = static_cast<int64_t>(T_) * n_groups;
  const bool aligned = gs % 8 == 0 && gate_stride % 8 == 0 &&
                       reinterpret_cast<uintptr_t>(gate) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(w) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(out) % 16 == 0;
  if (aligned && gs >= 512 && gs <= 8 * kNormGroups * 1024 && waves < (1ll << 31)) {
    int nt = 64;
    while (nt < 1024 && nt * 8 * kNormGroups < gs) nt <<= 1;
    if (gs >= 2048 && nt < 256) nt = 256;
    MIXK_DISPATCH(dtype, hipLaunchKernelGGL(group_rms_norm_vec_kernel<T>,
                                            dim3(static_cast<unsigned>(waves)), dim3(nt), 0, st,
                                            static_cast<T*>(out), y, static_cast<const T*>(gate),
                                            gate_stride, static_cast<const T*>(w), n_groups, gs,
                                            eps, w_full));
    return static_cast<int>(hipGetLastError());
  }
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(group_rms_norm_kernel<T>,
                                          dim3(static_cast<unsigned>((waves + 3) / 4)), dim3(256),
                                          0, st, static_cast<T*>(out), y,
                                          static_cast<const T*>(gate), gate_stride,
                                          static_cast<const T*>(w), T_, n_groups, gs, eps,
                                          w_full));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_head_gate(void* out, const void* o, const void* gate, int64_t gate_stride,
                              int T_, int H, int dv, int dtype, hipStream_t st) {
  if (T_ <= 0) return 0;
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(head_gate_kernel<T>, dim3(T_), dim3(256), 0, st,
                                          static_cast<T*>(out), static_cast<const T*>(o),
                                          static_cast<const T*>(gate), gate_stride, T_, H, dv));
  return static_cast<int>(hipGetLastError());
}
