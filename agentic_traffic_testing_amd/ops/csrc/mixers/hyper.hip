// Multi-stream residual (hyper-connections), token shift, the minGRU recurrence, element-wise
// gates and GELU.
//
// * hyper_update_norm: the residual is `ns` fp32 streams xs [T, ns, W].  One block per row does
//   the layer boundary in one pass: every stream at once from the old ones,
//   xs[t] = sum_s mix[s][t] xs[s] + w_out[t] y, then the next sub-layer's read
//   u = sum_t w_in[t] xs[t] and its RMS norm.  Either half can be left out (no y: norm only; no
//   norm weight: update only).  The row's u stays in registers between the sum of squares and the
//   scaling when W % 4 == 0 and W <= 16 * blockDim; wider or odd rows recompute it.
// * token_shift: h = n + (n_prev - n) * mu; the row before a portion is the sequence's state,
//   read and then replaced (with the portion's last row) by the block of the portion's first row
//   only, element by element in the same thread, so no other block touches it in this launch.
// * mingru_scan: S = S + sigmoid(z) (c - S), c = x + 1/2 (x >= 0) or sigmoid(x), out = S silu(g).
//   A workgroup owns 64 channels of one sequence's portion; its waves take consecutive time
//   segments.  Sweep 1 reduces every segment to the affine map S_out = A S_in + B, the maps are
//   composed through LDS into each segment's incoming state, sweep 2 reruns the segment from it
//   and writes the outputs.  Short portions use few waves (segments of at least 16 tokens); one
//   token is one wave and one sweep.
#include "mix_common.h"
#include "mixers.h"

namespace mixk {

typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4v;
__device__ __forceinline__ void ld4(const __bf16* p, float* o) {
  const bf16x4v v = *reinterpret_cast<const bf16x4v*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = static_cast<float>(v[i]);
}
__device__ __forceinline__ void ld4(const float* p, float* o) {
  const f32x4v v = *reinterpret_cast<const f32x4v*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = v[i];
}
__device__ __forceinline__ void st4(__bf16* p, const float* o) {
  bf16x4v v;
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = static_cast<__bf16>(o[i]);
  *reinterpret_cast<bf16x4v*>(p) = v;
}
__device__ __forceinline__ void st4(float* p, const float* o) {
  *reinterpret_cast<f32x4v*>(p) = f32x4v{o[0], o[1], o[2], o[3]};
}

constexpr int kMaxStreams = 8;
constexpr int kHyperGroups = 4;   // float4 groups per thread kept in registers

// Vector form, NS streams known at compile time, W % 4 == 0, W <= 16 * blockDim: every load of the
// row is issued before the first store (the streams are updated in place, so loads behind a store
// would wait for it), and u stays in registers between the sum of squares and the scaling.
template <typename TA, typename TO, int NS>
__global__ void hyper_update_norm_vec_kernel(TO* __restrict__ out, float* __restrict__ xs,
                                             const TA* __restrict__ y,
                                             const float* __restrict__ mix,
                                             const float* __restrict__ w_out,
                                             const float* __restrict__ w_in,
                                             const TA* __restrict__ w, int W, float eps) {
  __shared__ float scratch[16];
  float c_mix[NS][NS], c_out[NS], c_in[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    c_out[s] = y != nullptr ? w_out[s] : 0.f;
    c_in[s] = w != nullptr ? w_in[s] : 0.f;
#pragma unroll
    for (int t = 0; t < NS; ++t) c_mix[s][t] = y != nullptr ? mix[s * NS + t] : 0.f;
  }
  float* xr = xs + static_cast<int64_t>(blockIdx.x) * NS * W;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * W;
  float xv[kHyperGroups][NS][4], yv[kHyperGroups][4], wv[kHyperGroups][4];
#pragma unroll
  for (int g = 0; g < kHyperGroups; ++g) {
    const int i = (g * blockDim.x + threadIdx.x) * 4;
    if (i < W) {
#pragma unroll
      for (int s = 0; s < NS; ++s) ld4(xr + s * W + i, xv[g][s]);
      if (y != nullptr) ld4(y + row + i, yv[g]);
      if (w != nullptr) ld4(w + i, wv[g]);
    }
  }
  float ss = 0.f;
  float u[kHyperGroups][4];
#pragma unroll
  for (int g = 0; g < kHyperGroups; ++g) {
    const int i = (g * blockDim.x + threadIdx.x) * 4;
    if (i < W) {
      if (y != nullptr) {
        float nv[NS][4];
#pragma unroll
        for (int t = 0; t < NS; ++t)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float a = 0.f;
#pragma unroll
            for (int s = 0; s < NS; ++s) a += c_mix[s][t] * xv[g][s][e];
            nv[t][e] = a + c_out[t] * yv[g][e];
          }
#pragma unroll
        for (int t = 0; t < NS; ++t) {
          st4(xr + t * W + i, nv[t]);
#pragma unroll
          for (int e = 0; e < 4; ++e) xv[g][t][e] = nv[t][e];
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float a = 0.f;
#pragma unroll
        for (int s = 0; s < NS; ++s) a += c_in[s] * xv[g][s][e];
        u[g][e] = a;
        ss += a * a;
      }
    }
  }
  if (w == nullptr) return;
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(W) + eps);
#pragma unroll
  for (int g = 0; g < kHyperGroups; ++g) {
    const int i = (g * blockDim.x + threadIdx.x) * 4;
    if (i < W) {
#pragma unroll
      for (int e = 0; e < 4; ++e) wv[g][e] *= u[g][e] * inv;
      st4(out + row + i, wv[g]);
    }
  }
}

// Any number of streams up to kMaxStreams and any width: one element at a time, u recomputed.
template <typename TA, typename TO>
__global__ void hyper_update_norm_kernel(TO* __restrict__ out, float* __restrict__ xs,
                                         const TA* __restrict__ y, const float* __restrict__ mix,
                                         const float* __restrict__ w_out,
                                         const float* __restrict__ w_in, const TA* __restrict__ w,
                                         int ns, int W, float eps) {
  __shared__ float scratch[16];
  __shared__ float s_mix[kMaxStreams * kMaxStreams], s_out[kMaxStreams], s_in[kMaxStreams];
  if (threadIdx.x < ns * ns && y != nullptr) s_mix[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < ns) {
    s_out[threadIdx.x] = y != nullptr ? w_out[threadIdx.x] : 0.f;
    s_in[threadIdx.x] = w != nullptr ? w_in[threadIdx.x] : 0.f;
  }
  __syncthreads();
  float* xr = xs + static_cast<int64_t>(blockIdx.x) * ns * W;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float xv[kMaxStreams];
    for (int s = 0; s < ns; ++s) xv[s] = xr[s * W + i];
    if (y != nullptr) {
      const float yv = ldf(y + row + i);
      float nv[kMaxStreams];
      for (int t = 0; t < ns; ++t) {
        float a = 0.f;
        for (int s = 0; s < ns; ++s) a += s_mix[s * ns + t] * xv[s];
        nv[t] = a + s_out[t] * yv;
      }
      for (int t = 0; t < ns; ++t) {
        xr[t * W + i] = nv[t];
        xv[t] = nv[t];
      }
    }
    float a = 0.f;
    for (int s = 0; s < ns; ++s) a += s_in[s] * xv[s];
    ss += a * a;
  }
  if (w == nullptr) return;
  ss = block_sum(ss, scratch);   // also orders this thread's writes of xs before its re-reads
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(W) + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float a = 0.f;
    for (int s = 0; s < ns; ++s) a += s_in[s] * xr[s * W + i];
    stf(out + row + i, a * inv * ldf(w + i));
  }
}

// One block per row; the thread that reads an element of the slot's state is the one that
// replaces it, after all of its loads.
constexpr int kShiftGroups = 4;

template <typename T, bool VEC>
__global__ void token_shift_kernel(T* __restrict__ out, const float* __restrict__ n,
                                   const float* __restrict__ mu, float* __restrict__ state,
                                   const int* __restrict__ positions,
                                   const int* __restrict__ seq_qstart,
                                   const int* __restrict__ seq_slot, int S, int W) {
  const int r = blockIdx.x;
  const int s = seq_of_row(seq_qstart, S, r);
  const int slot = s < 0 ? -1 : seq_slot[s];
  T* o = out + static_cast<int64_t>(r) * W;
  if (slot < 0) {
    for (int i = threadIdx.x; i < W; i += blockDim.x) stf(o + i, 0.f);
    return;
  }
  const int first = seq_qstart[s], last = seq_qstart[s + 1] - 1;
  const float* cur = n + static_cast<int64_t>(r) * W;
  float* st = state + static_cast<int64_t>(slot) * W;
  const float* prev = r > first ? cur - W : (positions[r] == 0 ? nullptr : st);
  const float* tail = n + static_cast<int64_t>(last) * W;
  if (VEC) {
    float c[kShiftGroups][4], p[kShiftGroups][4], m[kShiftGroups][4], tl[kShiftGroups][4];
#pragma unroll
    for (int g = 0; g < kShiftGroups; ++g) {
      const int i = (g * blockDim.x + threadIdx.x) * 4;
      if (i < W) {
        ld4(cur + i, c[g]);
        ld4(mu + i, m[g]);
        if (prev != nullptr) {
          ld4(prev + i, p[g]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) p[g][e] = 0.f;
        }
        if (r == first) ld4(tail + i, tl[g]);
      }
    }
#pragma unroll
    for (int g = 0; g < kShiftGroups; ++g) {
      const int i = (g * blockDim.x + threadIdx.x) * 4;
      if (i < W) {
        if (r == first) st4(st + i, tl[g]);
#pragma unroll
        for (int e = 0; e < 4; ++e) c[g][e] += (p[g][e] - c[g][e]) * m[g][e];
        st4(o + i, c[g]);
      }
    }
    return;
  }
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float c = cur[i];
    const float p = prev != nullptr ? prev[i] : 0.f;
    if (r == first) st[i] = tail[i];
    stf(o + i, c + (p - c) * mu[i]);
  }
}

__device__ __forceinline__ float gelu_(float z, bool tanh_form) {
  if (tanh_form)
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  return 0.5f * z * (1.0f + erff(z * 0.7071067811865476f));
}

// act: 0 SiLU, 1 sigmoid, 2 tanh-form GELU
__device__ __forceinline__ float gate_act(float g, int act) {
  return act == 1 ? sigmoidf_(g) : act == 2 ? gelu_(g, true) : siluf_(g);
}

template <typename T>
__global__ void gate_mul_kernel(T* __restrict__ out, const T* __restrict__ a, int64_t a_stride,
                                const T* __restrict__ gate, int64_t gate_stride, int N, int act) {
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= N) return;
  const float g = ldf(gate + blockIdx.x * gate_stride + i);
  stf(out + static_cast<int64_t>(blockIdx.x) * N + i,
      ldf(a + blockIdx.x * a_stride + i) * gate_act(g, act));
}

template <typename T>
__global__ void gate_mul_vec_kernel(T* __restrict__ out, const T* __restrict__ a, int64_t a_stride,
                                    const T* __restrict__ gate, int64_t gate_stride, int N,
                                    int act) {
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (i >= N) return;
  float g[8], v[8];
  ld8(gate + blockIdx.x * gate_stride + i, g);
  ld8(a + blockIdx.x * a_stride + i, v);
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] *= gate_act(g[e], act);
  st8(out + static_cast<int64_t>(blockIdx.x) * N + i, v);
}

template <typename T>
__global__ void gelu_kernel(T* __restrict__ out, const T* __restrict__ x, int64_t x_stride, int N,
                            bool tanh_form) {
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= N) return;
  stf(out + static_cast<int64_t>(blockIdx.x) * N + i,
      gelu_(ldf(x + blockIdx.x * x_stride + i), tanh_form));
}

template <typename T>
__global__ void gelu_vec_kernel(T* __restrict__ out, const T* __restrict__ x, int64_t x_stride,
                                int N, bool tanh_form) {
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (i >= N) return;
  float v[8];
  ld8(x + blockIdx.x * x_stride + i, v);
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = gelu_(v[e], tanh_form);
  st8(out + static_cast<int64_t>(blockIdx.x) * N + i, v);
}

constexpr int kScanWaves = 16;
constexpr int kScanMinSeg = 16;
constexpr int kScanBatch = 16;  // tokens whose inputs are loaded before their recurrence steps run

__device__ __forceinline__ float mingru_candidate(float x) {
  return x >= 0.f ? x + 0.5f : sigmoidf_(x);
}

template <typename T>
__global__ void __launch_bounds__(64 * kScanWaves)
mingru_scan_kernel(T* __restrict__ out, float* __restrict__ state, const T* __restrict__ z,
                   int64_t z_stride, const T* __restrict__ x, int64_t x_stride,
                   const T* __restrict__ g, int64_t g_stride, const int* __restrict__ positions,
                   const int* __restrict__ seq_qstart, const int* __restrict__ seq_slot, int C) {
  __shared__ float sA[kScanWaves][64], sB[kScanWaves][64];
  const int s = blockIdx.y, slot = seq_slot[s];
  const int r0 = seq_qstart[s], n = seq_qstart[s + 1] - r0;
  if (slot < 0 || n <= 0) return;   // uniform over the workgroup
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  const bool ok = c < C;
  const int seg = max(kScanMinSeg, (n + nw - 1) / nw);
  const int t0 = min(n, wv * seg), t1 = min(n, t0 + seg);
  const int used = (n + seg - 1) / seg;   // waves with a non-empty segment
  const T* zp = z + c;
  const T* xp = x + c;
  const T* gp = g + c;
  if (used > 1) {
    float A = 1.f, B = 0.f;
    if (ok && wv < used - 1) {
      for (int tb = t0; tb < t1; tb += kScanBatch) {
        float zv[kScanBatch], xv[kScanBatch];
#pragma unroll
        for (int j = 0; j < kScanBatch; ++j) {
          const int64_t r = r0 + min(tb + j, t1 - 1);
          zv[j] = ldf(zp + r * z_stride);
          xv[j] = ldf(xp + r * x_stride);
        }
#pragma unroll
        for (int j = 0; j < kScanBatch; ++j) {
          if (tb + j < t1) {
            const float gate = sigmoidf_(zv[j]);
            A *= 1.0f - gate;
            B += gate * (mingru_candidate(xv[j]) - B);
          }
        }
      }
    }
    sA[wv][lane] = A;
    sB[wv][lane] = B;
    __syncthreads();
  }
  if (!ok || t0 >= t1) return;
  float S = positions[r0] == 0 ? 0.f : state[static_cast<int64_t>(slot) * C + c];
  for (int j = 0; j < wv; ++j) S = sA[j][lane] * S + sB[j][lane];
  for (int tb = t0; tb < t1; tb += kScanBatch) {
    float zv[kScanBatch], xv[kScanBatch], gv[kScanBatch];
#pragma unroll
    for (int j = 0; j < kScanBatch; ++j) {
      const int64_t r = r0 + min(tb + j, t1 - 1);
      zv[j] = ldf(zp + r * z_stride);
      xv[j] = ldf(xp + r * x_stride);
      gv[j] = ldf(gp + r * g_stride);
    }
#pragma unroll
    for (int j = 0; j < kScanBatch; ++j) {
      if (tb + j < t1) {
        S += sigmoidf_(zv[j]) * (mingru_candidate(xv[j]) - S);
        stf(out + static_cast<int64_t>(r0 + tb + j) * C + c, S * siluf_(gv[j]));
      }
    }
  }
  if (t1 == n) state[static_cast<int64_t>(slot) * C + c] = S;
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace mixk

using namespace mixk;

// out_f32: the norm's output is fp32 whatever the activation dtype.
extern "C" int mixk_hyper_update_norm(void* out, int out_f32, float* xs, const void* y,
                                      const float* mix, const float* w_out, const float* w_in,
                                      const void* w, int T_, int ns, int W, float eps, int dtype,
                                      hipStream_t st) {
  if (T_ <= 0) return 0;
  if (ns < 1 || ns > kMaxStreams) return -1;
  int threads = 64;
  while (threads < 1024 && threads * 4 * kHyperGroups < W) threads <<= 1;
  if (W >= 1024 && threads < 256) threads = 256;
  const bool vec = ns <= 4 && W % 4 == 0 && W <= 4 * kHyperGroups * threads;
#define MIXK_HYPER_VEC(TO, NS)                                                                  \
  hipLaunchKernelGGL((hyper_update_norm_vec_kernel<T, TO, NS>), dim3(T_), dim3(threads), 0, st, \
                     static_cast<TO*>(out), xs, static_cast<const T*>(y), mix, w_out, w_in,     \
                     static_cast<const T*>(w), W, eps)
#define MIXK_HYPER(TO)                                                                          \
  do {                                                                                          \
    if (vec && ns == 1) MIXK_HYPER_VEC(TO, 1);                                                  \
    else if (vec && ns == 2) MIXK_HYPER_VEC(TO, 2);                                             \
    else if (vec && ns == 3) MIXK_HYPER_VEC(TO, 3);                                             \
    else if (vec) MIXK_HYPER_VEC(TO, 4);                                                        \
    else                                                                                        \
      hipLaunchKernelGGL((hyper_update_norm_kernel<T, TO>), dim3(T_), dim3(threads), 0, st,     \
                         static_cast<TO*>(out), xs, static_cast<const T*>(y), mix, w_out, w_in, \
                         static_cast<const T*>(w), ns, W, eps);                                 \
  } while (0)
  MIXK_DISPATCH(dtype, {
    if (out_f32 || dtype == 2)
      MIXK_HYPER(float);
    else
      MIXK_HYPER(T);
  });
#undef MIXK_HYPER
#undef MIXK_HYPER_VEC
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_token_shift(void* out, const float* n, const float* mu, float* state,
                                const int* positions, const int* seq_qstart, const int* seq_slot,
                                int T_, int S, int W, int dtype, hipStream_t st) {
  if (T_ <= 0) return 0;
  int threads = 64;
  while (threads < 1024 && threads * 4 * kShiftGroups < W) threads <<= 1;
  const bool vec = W % 4 == 0 && W <= 4 * kShiftGroups * threads;
  MIXK_DISPATCH(dtype, {
    if (vec)
      hipLaunchKernelGGL((token_shift_kernel<T, true>), dim3(T_), dim3(threads), 0, st,
                         static_cast<T*>(out), n, mu, state, positions, seq_qstart, seq_slot, S, W);
    else
      hipLaunchKernelGGL((token_shift_kernel<T, false>), dim3(T_), dim3(threads), 0, st,
                         static_cast<T*>(out), n, mu, state, positions, seq_qstart, seq_slot, S, W);
  });
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_gate_mul(void* out, const void* a, int64_t a_stride, const void* gate,
                             int64_t gate_stride, int T_, int N, int act, int dtype,
                             hipStream_t st) {
  if (T_ <= 0 || N <= 0) return 0;
  if (act < 0 || act > 2) return -1;
  const bool vec = N % 8 == 0 && gate_stride % 8 == 0 && a_stride % 8 == 0 && aligned16(out) &&
                   aligned16(a) && aligned16(gate);
  MIXK_DISPATCH(dtype, {
    if (vec)
      hipLaunchKernelGGL(gate_mul_vec_kernel<T>, dim3(T_, (N / 8 + 255) / 256), dim3(256), 0, st,
                         static_cast<T*>(out), static_cast<const T*>(a), a_stride,
                         static_cast<const T*>(gate), gate_stride, N, act);
    else
      hipLaunchKernelGGL(gate_mul_kernel<T>, dim3(T_, (N + 255) / 256), dim3(256), 0, st,
                         static_cast<T*>(out), static_cast<const T*>(a), a_stride,
                         static_cast<const T*>(gate), gate_stride, N, act);
  });
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_gelu(void* out, const void* x, int64_t x_stride, int T_, int N, int tanh_form,
                         int dtype, hipStream_t st) {
  if (T_ <= 0 || N <= 0) return 0;
  const bool vec = N % 8 == 0 && x_stride % 8 == 0 && aligned16(out) && aligned16(x);
  MIXK_DISPATCH(dtype, {
    if (vec)
      hipLaunchKernelGGL(gelu_vec_kernel<T>, dim3(T_, (N / 8 + 255) / 256), dim3(256), 0, st,
                         static_cast<T*>(out), static_cast<const T*>(x), x_stride, N,
                         tanh_form != 0);
    else
      hipLaunchKernelGGL(gelu_kernel<T>, dim3(T_, (N + 255) / 256), dim3(256), 0, st,
                         static_cast<T*>(out), static_cast<const T*>(x), x_stride, N,
                         tanh_form != 0);
  });
  return static_cast<int>(hipGetLastError());
}

// few_rows: every portion is short (a decode step), one wave per workgroup is enough.
extern "C" int mixk_mingru_scan(void* out, float* state, const void* z, int64_t z_stride,
                                const void* x, int64_t x_stride, const void* g, int64_t g_stride,
                                const int* positions, const int* seq_qstart, const int* seq_slot,
                                int S, int C, int few_rows, int dtype, hipStream_t st) {
  if (S <= 0 || C <= 0) return 0;
  const int waves = few_rows ? 1 : kScanWaves;
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(mingru_scan_kernel<T>, dim3((C + 63) / 64, S),
                                          dim3(64 * waves), 0, st, static_cast<T*>(out), state,
                                          static_cast<const T*>(z), z_stride,
                                          static_cast<const T*>(x), x_stride,
                                          static_cast<const T*>(g), g_stride, positions,
                                          seq_qstart, seq_slot, C));
  return static_cast<int>(hipGetLastError());
}
