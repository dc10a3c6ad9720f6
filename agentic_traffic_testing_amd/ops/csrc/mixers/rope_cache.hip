// Per-head q / k RMS norm (plain weight or none; or a norm over the whole projection whose
// per-row inverse RMS is given), rotary positions on the first 2 * n_freq
// channels (pairs (2i, 2i + 1), or (i, i + n_freq) in the rotate-half layout; the norm before or
// after the rotation), and the paged K / V write of the softmax mixer; further down, the front
// end of latent attention (absorbed query assembly, rotate-half positions, latent K / V write).
//
// Grid (rows, (H + G) / 4), four waves per workgroup, one wave per (row, head): heads [0, H)
// are query heads (written to q_out [T, H, dim]), [H, H + G) key heads (normed, rotated,
// written to k_cache [nb, G, BS, dim] at the row's slot); the value heads go to the
// channel-major pages v_cache [nb, G, vdim, BS] in a kernel of their own (below).  cos / sin come from the step's fp32 table
// [rows, 2 n_freq] (rotary_table_kernel: cos | sin of position * inv_freq[i], computed once per
// step and shared by every layer with the same rotary parameters).
#include "mix_common.h"
#include "mixers.h"

namespace mixk {

__global__ void rotary_table_kernel(float* __restrict__ out, const int* __restrict__ positions,
                                    const float* __restrict__ inv_freq, int n_freq, int total) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int t = idx / n_freq, i = idx - t * n_freq;
  float sn, cs;
  sincosf(static_cast<float>(positions[t]) * inv_freq[i], &sn, &cs);
  out[static_cast<int64_t>(t) * 2 * n_freq + i] = cs;
  out[static_cast<int64_t>(t) * 2 * n_freq + n_freq + i] = sn;
}

constexpr int kMaxPairs = 4;  // pairs per lane: head width <= 2 * 64 * kMaxPairs = 512

template <typename T>
__global__ void qk_norm_rope_cache_kernel(T* __restrict__ q_out, const T* __restrict__ qx,
                                          int64_t q_stride, const T* __restrict__ kx,
                                          int64_t k_stride, const T* __restrict__ vx,
                                          int64_t v_stride, const T* __restrict__ q_norm,
                                          const T* __restrict__ k_norm, float eps,
                                          const int* __restrict__ positions,
                                          const int* __restrict__ slot_mapping,
                                          const float* __restrict__ cos_sin, int n_freq,
                                          T* __restrict__ k_cache, T* __restrict__ v_cache, int H,
                                          int G, int dim, int vdim, int block_size, int half,
                                          int norm_last, const float* __restrict__ row_inv) {
  const int t = blockIdx.x, head = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (head >= H + G) return;
  const int slot = slot_mapping[t];
  const bool is_q = head < H;
  if (!is_q && slot < 0) return;
  const T* src = is_q ? qx + t * q_stride + head * dim : kx + t * k_stride + (head - H) * dim;
  // row_inv [T, 2]: the norm runs over the whole q (k) projection - its inverse RMS was computed
  // per row beforehand and the weights are indexed by the projection's channel
  const T* w = is_q ? q_norm : k_norm;
  if (row_inv != nullptr && w != nullptr) w += (is_q ? head : head - H) * dim;
  T* dst = is_q ? q_out + (static_cast<int64_t>(t) * H + head) * dim
                : k_cache + ((static_cast<int64_t>(slot / block_size) * G + (head - H)) *
                                 block_size + slot % block_size) * dim;
  const int pairs = (dim + 1) >> 1;   // an odd width leaves the last pair half empty
  const float* tab = cos_sin + static_cast<int64_t>(t) * 2 * n_freq;   // [cos | sin] of row t
  float u[kMaxPairs], v[kMaxPairs];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < kMaxPairs; ++j) {
    const int i = lane + j * kWave;
    u[j] = v[j] = 0.f;
    if (i < pairs) {
      // pair i: channels (2i, 2i + 1), or (i, i + n_freq) for the rotated ones of the half layout
      const int ca = (half && i < n_freq) ? i : 2 * i, cb = (half && i < n_freq) ? i + n_freq : 2 * i + 1;
      u[j] = ldf(src + ca);
      v[j] = cb < dim ? ldf(src + cb) : 0.f;
      if (norm_last && i < n_freq) {
        const float cs = tab[i], sn = tab[n_freq + i];
        const float ra = u[j] * cs - v[j] * sn;
        v[j] = v[j] * cs + u[j] * sn;
        u[j] = ra;
      }
      ss += u[j] * u[j] + v[j] * v[j];
    }
  }
  float inv;
  if (row_inv != nullptr) {
    inv = row_inv[2 * static_cast<int64_t>(t) + (is_q ? 0 : 1)];
  } else {
    ss = wave_sum(ss);
    inv = 1.0f / sqrtf(ss / static_cast<float>(dim) + eps);
  }
#pragma unroll
  for (int j = 0; j < kMaxPairs; ++j) {
    const int i = lane + j * kWave;
    if (i >= pairs) continue;
    const int ca = (half && i < n_freq) ? i : 2 * i, cb = (half && i < n_freq) ? i + n_freq : 2 * i + 1;
    float a = u[j] * inv * (w != nullptr ? ldf(w + ca) : 1.0f);
    float b = v[j] * inv * (w != nullptr && cb < dim ? ldf(w + cb) : 1.0f);
    if (!norm_last && i < n_freq) {
      const float cs = tab[i], sn = tab[n_freq + i];
      const float ra = a * cs - b * sn;
      const float rb = b * cs + a * sn;
      a = ra;
      b = rb;
    }
    stf(dst + ca, a);
    if (cb < dim) stf(dst + cb, b);
  }
}

// V rows into the channel-major pages v_cache [nb, G, vdim, BS]: a workgroup takes 8 consecutive
// rows of one KV head.  When their slots are consecutive and start on a multiple of 8 (the usual
// case inside a portion; BS % 8 == 0 keeps them in one page) a thread gathers one channel of the
// 8 rows and writes it as one 16-byte (bf16) or two 16-byte (fp32) stores; otherwise it falls
// back to one element per store.
template <typename T>
__global__ void v_cache_write_kernel(const T* __restrict__ vx, int64_t v_stride,
                                     const int* __restrict__ slot_mapping,
                                     T* __restrict__ v_cache, int T_, int G, int vdim,
                                     int block_size) {
  const int r0 = blockIdx.x * 8, g = blockIdx.y;
  const int nrows = min(8, T_ - r0);
  const int s0 = slot_mapping[r0];
  bool run = nrows == 8 && s0 >= 0 && (s0 & 7) == 0 && (block_size & 7) == 0;
  if (run)
    for (int j = 1; j < 8; ++j) run = run && slot_mapping[r0 + j] == s0 + j;
  if (run) {
    T* page = v_cache + (static_cast<int64_t>(s0 / block_size) * G + g) * vdim * block_size +
              s0 % block_size;
    for (int ch = threadIdx.x; ch < vdim; ch += blockDim.x) {
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = ldf(vx + (r0 + j) * v_stride + g * vdim + ch);
      st8(page + static_cast<int64_t>(ch) * block_size, v);
    }
    return;
  }
  for (int j = 0; j < nrows; ++j) {
    const int slot = slot_mapping[r0 + j];
    if (slot < 0) continue;
    const T* src = vx + (r0 + j) * v_stride + g * vdim;
    T* dst = v_cache + (static_cast<int64_t>(slot / block_size) * G + g) * vdim * block_size +
             slot % block_size;
    for (int i = threadIdx.x; i < vdim; i += blockDim.x)
      dst[static_cast<int64_t>(i) * block_size] = src[i];
  }
}


// Latent attention front end (one shared key / value head of compressed rows): per row, one wave
// per query head assembles the absorbed query [q_lat | rotated q_rot] and one more wave norms
// the row's latent (RMS norm with a plain weight), rotates the shared key part and writes
// [latent | rotated key] to the K page; the normed latent also goes to `c_out` [T, rank], from
// where v_cache_write_kernel moves it to the channel-major V pages.  The rotation pairs channel
// i with i + n_freq ("rotate half") over the first 2 n_freq channels of the rotated part.
//   q_lat  [H, T, rank]       queries already multiplied by the key up-projection
//   qx     [T, H, qdim + rot] un-absorbed queries; only the last `rot` channels are read
//   kvx    [T, rank + rot]    row-strided down-projection (nullptr: the layer reads another
//                             layer's pages and writes none)
template <typename T>
__device__ __forceinline__ float rot_half(const T* x, int i, int n_freq, const float* tab) {
  if (i < n_freq) return ldf(x + i) * tab[i] - ldf(x + i + n_freq) * tab[n_freq + i];
  if (i < 2 * n_freq) {
    const int j = i - n_freq;
    return ldf(x + i) * tab[j] + ldf(x + j) * tab[n_freq + j];
  }
  return ldf(x + i);
}

template <typename T>
__global__ void latent_rope_cache_kernel(T* __restrict__ q_out, const T* __restrict__ q_lat,
                                         const T* __restrict__ qx, const T* __restrict__ kvx,
                                         int64_t kv_stride, const T* __restrict__ c_norm, float eps,
                                         const int* __restrict__ slot_mapping,
                                         const float* __restrict__ cos_sin, int n_freq,
                                         T* __restrict__ k_cache, T* __restrict__ c_out, int T_,
                                         int H, int qdim, int rank, int rot, int block_size) {
  const int t = blockIdx.x, head = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (head > H || (head == H && kvx == nullptr)) return;
  const float* tab = cos_sin + static_cast<int64_t>(t) * 2 * n_freq;
  const int kd = rank + rot;
  if (head < H) {
    T* dst = q_out + (static_cast<int64_t>(t) * H + head) * kd;
    const T* lat = q_lat + (static_cast<int64_t>(head) * T_ + t) * rank;
    for (int i = lane; i < rank; i += kWave) dst[i] = lat[i];
    const T* x = qx + (static_cast<int64_t>(t) * H + head) * (qdim + rot) + qdim;
    for (int i = lane; i < rot; i += kWave) stf(dst + rank + i, rot_half(x, i, n_freq, tab));
    return;
  }
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  const T* x = kvx + t * kv_stride;
  float ss = 0.f;
  for (int i = lane; i < rank; i += kWave) {
    const float v = ldf(x + i);
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(rank) + eps);
  T* dst = k_cache + (static_cast<int64_t>(slot / block_size) * block_size + slot % block_size) * kd;
  T* cd = c_out + static_cast<int64_t>(t) * rank;
  for (int i = lane; i < rank; i += kWave) {
    const float v = ldf(x + i) * inv * ldf(c_norm + i);
    stf(dst + i, v);
    stf(cd + i, v);
  }
  for (int i = lane; i < rot; i += kWave) stf(dst + rank + i, rot_half(x + rank, i, n_freq, tab));
}

}  // namespace mixk

using namespace mixk;

extern "C" int mixk_qk_norm_rope_cache(void* q_out, const void* qx, int64_t q_stride,
                                       const void* kx, int64_t k_stride, const void* vx,
                                       int64_t v_stride, const void* q_norm, const void* k_norm,
                                       float eps, const int* positions, const int* slot_mapping,
                                       const float* cos_sin, int n_freq, void* k_cache,
                                       void* v_cache, int T_, int H, int G, int dim, int vdim,
                                       int block_size, int half, int norm_last,
                                       const float* row_inv, int dtype, hipStream_t st) {
  if (T_ <= 0) return 0;
  if (dim > 2 * kWave * kMaxPairs || (row_inv != nullptr && norm_last)) return -1;
  MIXK_DISPATCH(dtype,
                hipLaunchKernelGGL(v_cache_write_kernel<T>, dim3((T_ + 7) / 8, G), dim3(128), 0,
                                   st, static_cast<const T*>(vx), v_stride, slot_mapping,
                                   static_cast<T*>(v_cache), T_, G, vdim, block_size));
  MIXK_DISPATCH(dtype,
                hipLaunchKernelGGL(qk_norm_rope_cache_kernel<T>, dim3(T_, (H + G + 3) / 4), dim3(256),
                                   0, st, static_cast<T*>(q_out), static_cast<const T*>(qx),
                                   q_stride, static_cast<const T*>(kx), k_stride,
                                   static_cast<const T*>(vx), v_stride,
                                   static_cast<const T*>(q_norm), static_cast<const T*>(k_norm),
                                   eps, positions, slot_mapping, cos_sin, n_freq,
                                   static_cast<T*>(k_cache), static_cast<T*>(v_cache), H, G, dim,
                                   vdim, block_size, half, norm_last, row_inv));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_rotary_table(float* out, const int* positions, const float* inv_freq, int T_,
                                 int n_freq, hipStream_t st) {
  const int total = T_ * n_freq;
  if (total <= 0) return 0;
  hipLaunchKernelGGL(rotary_table_kernel, dim3((total + 255) / 256), dim3(256), 0, st, out,
                     positions, inv_freq, n_freq, total);
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_latent_rope_cache(void* q_out, const void* q_lat, const void* qx,
                                      const void* kvx, int64_t kv_stride, const void* c_norm,
                                      float eps, const int* slot_mapping, const float* cos_sin,
                                      int n_freq, void* k_cache, void* v_cache, void* c_out,
                                      int T_, int H, int qdim, int rank, int rot, int block_size,
                                      int dtype, hipStream_t st) {
  if (T_ <= 0) return 0;
  if (2 * n_freq > rot || rank <= 0) return -1;
  MIXK_DISPATCH(dtype, {
    hipLaunchKernelGGL(latent_rope_cache_kernel<T>, dim3(T_, (H + 1 + 3) / 4), dim3(256), 0, st,
                       static_cast<T*>(q_out), static_cast<const T*>(q_lat),
                       static_cast<const T*>(qx), static_cast<const T*>(kvx), kv_stride,
                       static_cast<const T*>(c_norm), eps, slot_mapping, cos_sin, n_freq,
                       static_cast<T*>(k_cache), static_cast<T*>(c_out), T_, H, qdim, rank, rot,
                       block_size);
    if (kvx != nullptr)
      hipLaunchKernelGGL(v_cache_write_kernel<T>, dim3((T_ + 7) / 8, 1), dim3(128), 0, st,
                         static_cast<const T*>(c_out), static_cast<int64_t>(rank), slot_mapping,
                         static_cast<T*>(v_cache), T_, 1, rank, block_size);
  });
  return static_cast<int>(hipGetLastError());
}
