// Causal paged softmax attention for any head widths, with an optional sink (one extra key of
// score 0 and no value in every denominator).  K pages are [nb, G, BS, dim], V pages are
// channel-major [nb, G, vdim, BS].  Three kernels:
//
// * rows kernel (any dtype, any widths; fp32 scores, weights and accumulation): a workgroup of
//   256 threads serves 16 "rows" against a stream of key tiles staged in LDS as fp32; thread
//   (r, c) = (tid / 16, tid % 16) scores row r against keys c, c + 16, ... of the tile, the 16
//   threads of a row share max / sum by lane shuffles (online softmax) and the same thread
//   accumulates value channels c, c + 16, ....  Prefill mode: rows = 16 query tokens of one
//   head (a 64-token tile is four workgroups).  Decode mode: rows = the query heads of one KV
//   head for a sequence's single new token, over one 128-key partition of the context; the
//   partials (m, l, unnormalised sum) are merged by the combine kernel, so a long context
//   spreads over many workgroups and the result never depends on what else is in the batch.
// * matrix-core prefill kernel (bf16, dim % 16 == 0, vdim % 32 == 0): 4 waves x 32 columns, a
//   column = (query token, query head of the KV head's group), 32-key tiles:
//     S^T[32 keys x 32 cols] = K . Q^T   (mfma 32x32x16, A = K rows from LDS, B = Q in registers)
//     O^T[vdim x 32 cols]   += V^T . P^T (A = V^T rows from LDS, B = P^T from the S^T registers)
//   The S^T accumulator keeps one column per lane, so softmax statistics are lane-local plus
//   one exchange with lane ^ 32; P^T feeds the second product from registers with the key
//   order inside each 16-key step permuted the way the accumulator holds it (keys 4h..4h+3,
//   8+4h..8+4h+3 for lane half h), and the V^T operand reads follow the same order.
// * combine kernel for the decode partials.
//
// A sliding window (`window` > 0: the query at position i sees keys j with 0 <= i - j < window)
// moves the first key tile of a workgroup up to the window's start and masks the tiles that
// touch its edge; decode then runs only the partitions that overlap the window (partition
// indices are relative to the first of them, for the partition kernel and the combine alike).
//
// The sink enters as the initial state of the online softmax: running max = the sink's score,
// running sum 1, zero accumulator.  The sink's score is 0, or one learned number per query head
// (`sink_val`, unscaled).
#include "mix_common.h"
#include "mixers.h"

namespace mixk {

constexpr int kRows = 16;         // rows per workgroup of the rows kernel
constexpr int kMaxVPer = 32;      // value channels per thread: vdim <= 512
constexpr int kTileTokens = 64;   // query tokens per prefill tile (host tiling)
constexpr int kPartTokens = 128;  // keys per decode partition
constexpr float kNegBig = -1.0e30f;

struct AttnArgs {
  const int* block_tables;
  const int* seq_kvlen;
  const int* seq_qstart;
  const int* tile_seq;
  const int* tile_qoff;
  float* part;          // decode partials [S, H, max_parts, vdim + 2]
  const float* sink_val;  // [H] score of the sink per query head (nullptr: 0)
  int bt_width, H, G, dim, vdim, block_size, sink, KT, max_parts, bs_shift;
  float scale;
  int window;   // 0: every earlier key
};

// first key a query at position qpos sees
__device__ __forceinline__ int window_start(int qpos, int window) {
  return window > 0 ? max(0, qpos - window + 1) : 0;
}

template <typename T, bool DECODE>
__global__ void __launch_bounds__(256)
sink_attention_rows_kernel(T* __restrict__ out, const T* __restrict__ q,
                           const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                           AttnArgs a) {
  extern __shared__ float smem[];
  const int H = a.H, G = a.G, dim = a.dim, vdim = a.vdim, KT = a.KT, bs = a.block_size;
  const int rep = H / G;
  int s, g, nrows, kbeg, kend, kvlen, n, row0, qo = 0, h0;
  if (DECODE) {
    // blockIdx.y = (KV head, block of up to kRows query heads of its group)
    const int hb = (rep + kRows - 1) / kRows;
    s = blockIdx.x;
    g = blockIdx.y / hb;
    row0 = a.seq_qstart[s];
    n = 1;
    kvlen = a.seq_kvlen[s];
    h0 = g * rep + (blockIdx.y % hb) * kRows;
    nrows = min(kRows, (g + 1) * rep - h0);
    if (kvlen <= 0) return;
    const int wstart = window_start(kvlen - 1, a.window);
    kbeg = (wstart / kPartTokens + blockIdx.z) * kPartTokens;
    kend = min(kvlen, kbeg + kPartTokens);
    kbeg = max(kbeg, wstart);
    if (kbeg >= kend) return;
  } else {
    const int tile = blockIdx.x >> 2;
    s = a.tile_seq[tile];
    qo = a.tile_qoff[tile] + kRows * (blockIdx.x & 3);
    h0 = blockIdx.y;
    g = h0 / rep;
    row0 = a.seq_qstart[s];
    n = a.seq_qstart[s + 1] - row0;
    kvlen = a.seq_kvlen[s];
    if (n <= 0 || kvlen <= 0 || qo >= n) return;
    nrows = min(kRows, n - qo);
    kbeg = window_start(kvlen - n + qo, a.window);
    kend = min(kvlen, kvlen - n + qo + nrows);
  }
  const int tid = threadIdx.x, r = tid >> 4, c = tid & 15;
  const int kstride = dim + 1, vstride = vdim + 1;
  float* Qs = smem;                        // [kRows][dim]
  float* Ks = Qs + kRows * dim;            // [KT][dim + 1]
  float* Vs = Ks + KT * kstride;           // [KT][vdim + 1]
  float* Ps = Vs + KT * vstride;           // [kRows][KT]
  for (int i = tid; i < kRows * dim; i += 256) {
    const int rr = i / dim, d = i - rr * dim;
    float v = 0.f;
    if (rr < nrows) {
      const int64_t qrow = DECODE ? row0 : row0 + qo + rr;
      const int head = DECODE ? h0 + rr : h0;
      v = ldf(q + (qrow * H + head) * dim + d);
    }
    Qs[i] = v;
  }
  const bool row_ok = r < nrows;
  const int qpos = DECODE ? kvlen - 1 : kvlen - n + qo + r;
  const int qlow = window_start(qpos, a.window);
  const bool use_sink = a.sink && !DECODE;   // decode: the combine kernel adds the sink once
  float m = kNegBig, l = 0.f;
  if (use_sink) {
    m = a.sink_val != nullptr ? a.sink_val[min(h0 + (DECODE ? r : 0), H - 1)] : 0.f;
    l = 1.f;
  }
  float acc[kMaxVPer];
#pragma unroll
  for (int j = 0; j < kMaxVPer; ++j) acc[j] = 0.f;
  const int* bt = a.block_tables + static_cast<int64_t>(s) * a.bt_width;
  const int kper = KT >> 4;
  for (int k0 = kbeg; k0 < kend; k0 += KT) {
    __syncthreads();  // previous tile fully consumed (and Qs written, first time round)
    for (int i = tid; i < KT * dim; i += 256) {
      const int kk = i / dim, d = i - kk * dim;
      const int tok = k0 + kk;
      float val = 0.f;
      if (tok < kend) {
        const int64_t page = bt[tok / bs];
        val = ldf(k_cache + ((page * G + g) * bs + tok % bs) * dim + d);
      }
      Ks[kk * kstride + d] = val;
    }
    for (int i = tid; i < KT * vdim; i += 256) {
      const int d = i / KT, kk = i - d * KT;   // keys fastest: contiguous inside a page row
      const int tok = k0 + kk;
      float val = 0.f;
      if (tok < kend) {
        const int64_t page = bt[tok / bs];
        val = ldf(v_cache + ((page * G + g) * vdim + d) * bs + tok % bs);
      }
      Vs[kk * vstride + d] = val;
    }
    __syncthreads();
    float sc[4];
    float tmax = kNegBig;
    for (int j = 0; j < kper; ++j) {
      const int kk = c + 16 * j;
      const float* kr = Ks + kk * kstride;
      const float* qr = Qs + r * dim;
      float dot = 0.f;
      if (row_ok)
        for (int d = 0; d < dim; ++d) dot += qr[d] * kr[d];
      const int tok = k0 + kk;
      sc[j] = (row_ok && tok <= qpos && tok >= qlow && tok < kend) ? dot * a.scale : kNegBig;
      tmax = fmaxf(tmax, sc[j]);
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, o, kWave));
    const float m_new = fmaxf(m, tmax);
    const float alpha = expf(m - m_new);
    float psum = 0.f;
    for (int j = 0; j < kper; ++j) {
      const float p = sc[j] <= kNegBig ? 0.f : expf(sc[j] - m_new);
      Ps[r * KT + c + 16 * j] = p;
      psum += p;
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) psum += __shfl_xor(psum, o, kWave);
    l = l * alpha + psum;
    m = m_new;
    __syncthreads();
    const float* pr = Ps + r * KT;
#pragma unroll
    for (int j = 0; j < kMaxVPer; ++j) {
      const int d = c + 16 * j;
      if (d < vdim && row_ok) {
        float av = acc[j] * alpha;
        for (int kk = 0; kk < KT; ++kk) av += pr[kk] * Vs[kk * vstride + d];
        acc[j] = av;
      }
    }
  }
  if (!row_ok) return;
  if (DECODE) {
    float* po = a.part + ((static_cast<int64_t>(s) * H + h0 + r) * a.max_parts + blockIdx.z) *
                             (vdim + 2);
#pragma unroll
    for (int j = 0; j < kMaxVPer; ++j) {
      const int d = c + 16 * j;
      if (d < vdim) po[d] = acc[j];
    }
    if (c == 0) {
      po[vdim] = m;
      po[vdim + 1] = l;
    }
    return;
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  T* o = out + (static_cast<int64_t>(row0 + qo + r) * H + h0) * vdim;
#pragma unroll
  for (int j = 0; j < kMaxVPer; ++j) {
    const int d = c + 16 * j;
    if (d < vdim) stf(o + d, acc[j] * inv);
  }
}

// One wave per (decode sequence, head): merge the partitions' (m, l, sum) and the sink.  Lane p
// fetches partition p's (m, l) (all in flight at once), the wave reduces them, and the
// per-partition weights go through LDS for the channel loop.
constexpr int kMaxParts = 2048;
template <typename T>
__global__ void sink_attention_combine_kernel(T* __restrict__ out, AttnArgs a) {
  __shared__ float wts[kMaxParts];
  const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int kvlen = a.seq_kvlen[s];
  if (kvlen <= 0) return;
  const int np = min(kMaxParts, (kvlen + kPartTokens - 1) / kPartTokens -
                                    window_start(kvlen - 1, a.window) / kPartTokens);
  const int vdim = a.vdim, ps = vdim + 2;
  const float* base = a.part + (static_cast<int64_t>(s) * a.H + h) * a.max_parts * ps;
  const float sink_score = a.sink_val != nullptr ? a.sink_val[h] : 0.f;
  float M = a.sink ? sink_score : kNegBig;
  for (int p = lane; p < np; p += kWave) M = fmaxf(M, base[p * ps + vdim]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o, kWave));
  float L = 0.f;
  for (int p = lane; p < np; p += kWave) {
    const float wp = expf(base[p * ps + vdim] - M);
    wts[p] = wp;
    L += base[p * ps + vdim + 1] * wp;
  }
  L = wave_sum(L) + (a.sink ? expf(sink_score - M) : 0.f);
  __syncthreads();
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  T* o = out + (static_cast<int64_t>(a.seq_qstart[s]) * a.H + h) * vdim;
  for (int d = lane; d < vdim; d += kWave) {
    float v = 0.f;
#pragma unroll 8
    for (int p = 0; p < np; ++p) v += base[p * ps + d] * wts[p];
    stf(o + d, v * inv);
  }
}

// ---- matrix-core prefill (bf16) -----------------------------------------------------------
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

constexpr int kKeys = 32;          // keys per tile
constexpr int kBtLds = 1024;       // block-table entries of the sequence kept in LDS
constexpr int kVStride = kKeys + 8;

// DECODE: one workgroup per (decode sequence, KV head, 128-key partition); the columns are the
// query heads of the group for the sequence's single new token, the output is the partition's
// partial (unnormalised sum, m, l) for the combine kernel.  Waves without a valid column only
// help to stage the tiles.
template <int ND, int NV, bool DECODE>  // dim <= 16 ND, vdim <= 32 NV
__global__ void __launch_bounds__(256, 2)
sink_attention_mfma_kernel(__bf16* __restrict__ out, const __bf16* __restrict__ q,
                           const __bf16* __restrict__ k_cache, const __bf16* __restrict__ v_cache,
                           AttnArgs a) {
  constexpr int KS = ND * 16 + 8;
  __shared__ __attribute__((aligned(16))) __bf16 lds_k[kKeys * KS];
  __shared__ __attribute__((aligned(16))) __bf16 lds_v[NV * 32 * kVStride];
  __shared__ int lds_bt[kBtLds];
  const int H = a.H, G = a.G, dim = a.dim, vdim = a.vdim, bs = a.block_size;
  const int rep = H / G, nd = dim >> 4, nv = vdim >> 5;
  const int g = blockIdx.y;
  // tiles are listed in sequence order, so the ones with the most keys come last: start those
  // first (the tail of the launch is then made of short tiles)
  const int tile = DECODE ? 0 : static_cast<int>(gridDim.x - 1 - blockIdx.x);
  const int s = DECODE ? blockIdx.x : a.tile_seq[tile];
  const int qo = DECODE ? 0 : a.tile_qoff[tile];
  const int row0 = a.seq_qstart[s];
  const int n = DECODE ? 1 : a.seq_qstart[s + 1] - row0;
  const int kvlen = a.seq_kvlen[s];
  if (n <= 0 || kvlen <= 0 || qo >= n) return;
  const int ntok = min(kTileTokens, n - qo);
  const int cols_total = ntok * rep;
  const int col0 = DECODE ? 0 : blockIdx.z * 128;
  if (col0 >= cols_total) return;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int col = col0 + w * 32 + r;
  const bool valid = col < cols_total;
  const int tok = valid ? col / rep : 0;
  const int head = g * rep + (valid ? col % rep : 0);
  const int64_t qrow = row0 + qo + tok;
  const int qpos = kvlen - n + qo + tok;
  const int last_tok = (min(cols_total, col0 + 128) - 1) / rep;
  // first key tile: the window's start of the workgroup's earliest column, on a tile boundary
  // (the V^T staging reads 8 keys at a time from 8-aligned slots)
  const int wstart = window_start(kvlen - n + qo + col0 / rep, a.window);
  const int part0 = DECODE ? (wstart / kPartTokens + blockIdx.z) * kPartTokens : 0;
  const int kbeg = max(part0, wstart & ~(kKeys - 1));
  const int kend = DECODE ? min(kvlen, part0 + kPartTokens)
                          : min(kvlen, kvlen - n + qo + last_tok + 1);
  if (kbeg >= kend) return;
  const bool wave_on = col0 + w * 32 < cols_total;   // wave-uniform
  const int qpos_first = kvlen - n + qo + (col0 + w * 32) / rep;   // the wave's earliest column
  // the wave's latest column: keys at or below its window start are outside somebody's window
  const int qpos_lastw = kvlen - n + qo + (min(cols_total, col0 + w * 32 + 32) - 1) / rep;
  const int edge_lo = a.window > 0 ? qpos_lastw - a.window : -1;
  const int qlow = window_start(qpos, a.window);
  const float scale2 = a.scale * 1.44269504088896341f;
  const bool use_sink = a.sink && !DECODE;           // decode: the combine kernel adds it once
  bf16x8 qf[ND];
#pragma unroll
  for (int st = 0; st < ND; ++st) {
    u32x4 z = {0u, 0u, 0u, 0u};
    if (valid && st < nd)
      z = *reinterpret_cast<const u32x4*>(q + (qrow * H + head) * dim + st * 16 + 8 * h);
    qf[st] = __builtin_bit_cast(bf16x8, z);
  }
  float m = kNegBig, l = 0.f;
  if (use_sink) {   // log2 units, like the scores
    m = a.sink_val != nullptr ? a.sink_val[head] * 1.44269504088896341f : 0.f;
    l = 1.f;
  }
  f32x16 O[NV];
#pragma unroll
  for (int vt = 0; vt < NV; ++vt)
#pragma unroll
    for (int i = 0; i < 16; ++i) O[vt][i] = 0.f;
  // the pages this workgroup walks, copied to LDS once: a key's page is then an LDS read and a
  // tile costs one global round trip, not two dependent ones
  const int* btg = a.block_tables + static_cast<int64_t>(s) * a.bt_width;
  const int page0 = kbeg >> a.bs_shift;
  const int npages = ((kend + bs - 1) >> a.bs_shift) - page0;
  const bool bt_lds = npages <= kBtLds;
  if (bt_lds)
    for (int i = tid; i < npages; i += 256) lds_bt[i] = btg[page0 + i];
  auto page_of = [&](int idx) -> int64_t { return bt_lds ? lds_bt[idx - page0] : btg[idx]; };
  // Staging plan of this thread, fixed for the whole loop: which 16-byte chunks of a K tile
  // (key, 8-channel group) and of a V^T tile (channel, 8-key group) it moves.  The page size is
  // a power of two (host-checked), so a key's page and offset are a shift and a mask.
  constexpr int KC = (kKeys * ND * 2 + 255) / 256;
  constexpr int VC = (NV * 32 * 4 + 255) / 256;
  const int bshift = a.bs_shift, bmask = bs - 1;
  const int kchunks = kKeys * (dim >> 3), vchunks = vdim * (kKeys >> 3);
  int k_key[KC], k_src[KC], k_dst[KC];
#pragma unroll
  for (int c = 0; c < KC; ++c) {
    const int i = tid + c * 256;
    const int key = i / (dim >> 3), c8 = i - key * (dim >> 3);
    k_key[c] = i < kchunks ? key : -1;
    k_src[c] = c8 * 8;
    k_dst[c] = key * KS + c8 * 8;
  }
  const __bf16* kbase = k_cache + static_cast<int64_t>(g) * bs * dim;
  const __bf16* vbase = v_cache + static_cast<int64_t>(g) * vdim * bs;
  const int64_t kpage = static_cast<int64_t>(G) * bs * dim, vpage = static_cast<int64_t>(G) * vdim * bs;
  for (int k0 = kbeg; k0 < kend; k0 += kKeys) {
    __syncthreads();
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      if (k_key[c] < 0) continue;
      const int tk = k0 + k_key[c];
      u32x4 z = {0u, 0u, 0u, 0u};
      if (tk < kend)
        z = *reinterpret_cast<const u32x4*>(kbase + page_of(tk >> bshift) * kpage +
                                            (tk & bmask) * dim + k_src[c]);
      *reinterpret_cast<u32x4*>(lds_k + k_dst[c]) = z;
    }
#pragma unroll
    for (int c = 0; c < VC; ++c) {
      const int i = tid + c * 256;
      if (i >= vchunks) continue;
      const int ch = i >> 2, kg = i & 3;
      const int t8 = k0 + kg * 8;
      u32x4 z = {0u, 0u, 0u, 0u};
      if (t8 < kend) {
        z = *reinterpret_cast<const u32x4*>(vbase + page_of(t8 >> bshift) * vpage + ch * bs +
                                            (t8 & bmask));
        if (t8 + 8 > kend) {   // keys past the end: their V must be exactly zero
          bf16x8 e = __builtin_bit_cast(bf16x8, z);
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (t8 + j >= kend) e[j] = static_cast<__bf16>(0.f);
          z = __builtin_bit_cast(u32x4, e);
        }
      }
      // key-permuted image: inside each 16-key step, key 8 a + 4 h + b sits at 8 h + 4 a + b, so
      // the 8 keys a lane half needs for a P.V fragment are one 16-byte read
      typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;
      __bf16* vrow = lds_v + ch * kVStride + (kg >> 1) * 16 + (kg & 1) * 4;
      *reinterpret_cast<u32x2*>(vrow) = u32x2{z[0], z[1]};
      *reinterpret_cast<u32x2*>(vrow + 8) = u32x2{z[2], z[3]};
    }
    __syncthreads();
    if (!wave_on) continue;
    f32x16 S;
#pragma unroll
    for (int i = 0; i < 16; ++i) S[i] = 0.f;
#pragma unroll
    for (int st = 0; st < ND; ++st) {
      if (st < nd) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(lds_k + r * KS + st * 16 + 8 * h);
        S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[st], S, 0, 0, 0);
      }
    }
    // scores in log2 units (scale * log2 e folded into one multiply; the sink's score 0 stays 0);
    // only tiles that reach the wave's causal edge or the end of the keys are masked
    float tmax = kNegBig;
    // (a masked score is -inf, the running maximum starts at the finite kNegBig: a column whose
    // window has not begun yet keeps weight exp2(-inf) = 0 on every key of the tile)
    if (k0 + kKeys - 1 > qpos_first || k0 + kKeys > kend || k0 <= edge_lo) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = k0 + 8 * (i >> 2) + 4 * h + (i & 3);
        S[i] = (key <= qpos && key >= qlow && key < kend) ? S[i] * scale2 : -INFINITY;
        tmax = fmaxf(tmax, S[i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        S[i] *= scale2;
        tmax = fmaxf(tmax, S[i]);
      }
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
    const float m_new = fmaxf(m, tmax);
    const float alpha = __builtin_amdgcn_exp2f(m - m_new);
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      S[i] = __builtin_amdgcn_exp2f(S[i] - m_new);   // masked scores: exp2(-inf) = 0
      psum += S[i];
    }
    psum += __shfl_xor(psum, 32, kWave);
    l = l * alpha + psum;
    m = m_new;
    bf16x8 pk[2];
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int j = 0; j < 8; ++j) pk[st][j] = static_cast<__bf16>(S[8 * st + j]);
#pragma unroll
    for (int vt = 0; vt < NV; ++vt) {
      if (vt < nv) {
#pragma unroll
        for (int i = 0; i < 16; ++i) O[vt][i] *= alpha;
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          const bf16x8 vf = *reinterpret_cast<const bf16x8*>(lds_v + (vt * 32 + r) * kVStride +
                                                             16 * st + 8 * h);
          O[vt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pk[st], O[vt], 0, 0, 0);
        }
      }
    }
  }
  if (!valid) return;
  if (DECODE) {
    float* po = a.part + ((static_cast<int64_t>(s) * H + head) * a.max_parts + blockIdx.z) *
                             (vdim + 2);
#pragma unroll
    for (int vt = 0; vt < NV; ++vt)
      if (vt < nv)
#pragma unroll
        for (int i = 0; i < 16; ++i) po[vt * 32 + 8 * (i >> 2) + 4 * h + (i & 3)] = O[vt][i];
    if (h == 0) {
      po[vdim] = m * 0.693147180559945309f;   // the combine kernel works in natural-log units
      po[vdim + 1] = l;
    }
    return;
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  __bf16* o = out + (qrow * H + head) * vdim;
#pragma unroll
  for (int vt = 0; vt < NV; ++vt) {
    if (vt < nv) {
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        bf16x4 e;
#pragma unroll
        for (int j = 0; j < 4; ++j) e[j] = static_cast<__bf16>(O[vt][4 * i4 + j] * inv);
        *reinterpret_cast<bf16x4*>(o + vt * 32 + 8 * i4 + 4 * h) = e;
      }
    }
  }
}

size_t rows_smem(int kt, int dim, int vdim) {
  return sizeof(float) * (static_cast<size_t>(kRows) * dim + static_cast<size_t>(kt) * (dim + 1) +
                          static_cast<size_t>(kt) * (vdim + 1) + static_cast<size_t>(kRows) * kt);
}

template <typename K>
int opt_in_smem(K kernel, size_t smem, size_t* opted) {
  if (smem > 48 * 1024 && smem > *opted) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       static_cast<int>(smem));
    if (e != hipSuccess) return static_cast<int>(e);
    *opted = smem;
  }
  return 0;
}

// partitions a decode row can touch: all of its context, or the ones its window overlaps
int decode_parts(int max_decode_kv, int window) {
  const int all = (max_decode_kv + kPartTokens - 1) / kPartTokens;
  return window > 0 ? min(all, (window + kPartTokens - 1) / kPartTokens + 1) : all;
}

template <typename T>
int launch_rows(void* out, const void* q, const void* k_cache, const void* v_cache, AttnArgs a,
                int num_tiles, int num_decode, int max_decode_kv, hipStream_t st) {
  int KT = 64;
  while (KT > 16 && rows_smem(KT, a.dim, a.vdim) > 96 * 1024) KT >>= 1;
  const size_t smem = rows_smem(KT, a.dim, a.vdim);
  if (smem > 150 * 1024) return -1;
  a.KT = KT;
  static size_t opted_p = 0, opted_d = 0;
  if (num_tiles > 0) {
    if (int rc = opt_in_smem(sink_attention_rows_kernel<T, false>, smem, &opted_p)) return rc;
    hipLaunchKernelGGL((sink_attention_rows_kernel<T, false>), dim3(num_tiles * 4, a.H), dim3(256),
                       smem, st, static_cast<T*>(out), static_cast<const T*>(q),
                       static_cast<const T*>(k_cache), static_cast<const T*>(v_cache), a);
  }
  if (num_decode > 0) {
    if (int rc = opt_in_smem(sink_attention_rows_kernel<T, true>, smem, &opted_d)) return rc;
    const int parts = decode_parts(max_decode_kv, a.window);
    if (parts > a.max_parts || parts < 1) return -1;
    const int head_blocks = (a.H / a.G + kRows - 1) / kRows;
    hipLaunchKernelGGL((sink_attention_rows_kernel<T, true>),
                       dim3(num_decode, a.G * head_blocks, parts),
                       dim3(256), smem, st, static_cast<T*>(out), static_cast<const T*>(q),
                       static_cast<const T*>(k_cache), static_cast<const T*>(v_cache), a);
    hipLaunchKernelGGL(sink_attention_combine_kernel<T>, dim3(num_decode, a.H), dim3(kWave), 0, st,
                       static_cast<T*>(out), a);
  }
  return static_cast<int>(hipGetLastError());
}

template <int ND, int NV>
void launch_mfma(void* out, const void* q, const void* k_cache, const void* v_cache, AttnArgs a,
                 int num_tiles, int num_decode, int parts, hipStream_t st) {
  const int chunks = (kTileTokens * (a.H / a.G) + 127) / 128;
  if (num_tiles > 0)
    hipLaunchKernelGGL((sink_attention_mfma_kernel<ND, NV, false>), dim3(num_tiles, a.G, chunks),
                       dim3(256), 0, st, static_cast<__bf16*>(out), static_cast<const __bf16*>(q),
                       static_cast<const __bf16*>(k_cache), static_cast<const __bf16*>(v_cache), a);
  if (num_decode > 0) {
    hipLaunchKernelGGL((sink_attention_mfma_kernel<ND, NV, true>), dim3(num_decode, a.G, parts),
                       dim3(256), 0, st, static_cast<__bf16*>(out), static_cast<const __bf16*>(q),
                       static_cast<const __bf16*>(k_cache), static_cast<const __bf16*>(v_cache), a);
    hipLaunchKernelGGL(sink_attention_combine_kernel<__bf16>, dim3(num_decode, a.H), dim3(kWave),
                       0, st, static_cast<__bf16*>(out), a);
  }
}

}  // namespace mixk

using namespace mixk;

// Prefill tiles (64 query tokens each: tile_seq / tile_qoff) and decode sequences
// [0, num_decode) (one query row each, row = seq_qstart[s]; partials in `part`
// [num_decode, H, max_parts, vdim + 2] fp32).  use_mfma: bf16 matrix-core prefill kernel.
extern "C" int mixk_sink_attention(void* out, const void* q, const void* k_cache,
                                   const void* v_cache, const int* block_tables, int bt_width,
                                   const int* seq_kvlen, const int* seq_qstart,
                                   const int* tile_seq, const int* tile_qoff, int num_tiles,
                                   int num_decode, int max_decode_kv, float* part, int max_parts,
                                   int H, int G, int dim, int vdim, int block_size, float scale,
                                   int sink, const float* sink_val, int window, int use_mfma,
                                   int dtype, hipStream_t st) {
  if (num_tiles <= 0 && num_decode <= 0) return 0;
  if (vdim > 16 * kMaxVPer || G <= 0 || H % G != 0) return -1;
  int bs_shift = 0;
  while ((1 << bs_shift) < block_size) ++bs_shift;
  AttnArgs a{block_tables, seq_kvlen, seq_qstart, tile_seq, tile_qoff, part, sink ? sink_val : nullptr,
             bt_width, H, G, dim, vdim, block_size, sink, 0, max_parts, bs_shift, scale,
             window > 0 ? window : 0};
  int rc = 0;
  if (use_mfma) {
    if (dtype != 0 || dim % 16 || vdim % 32 || dim > 256 || vdim > 256 || block_size < 8 ||
        (block_size & (block_size - 1)))
      return -1;
    // decode columns = the query heads of one KV head: they must fit one workgroup
    const int nd_mfma = (H / G <= 128) ? num_decode : 0;
    const int parts = decode_parts(max_decode_kv, a.window);
    if (nd_mfma > 0 && (parts > max_parts || parts < 1)) return -1;
    if (dim <= 64 && vdim <= 64)
      launch_mfma<4, 2>(out, q, k_cache, v_cache, a, num_tiles, nd_mfma, parts, st);
    else if (dim <= 128 && vdim <= 128)
      launch_mfma<8, 4>(out, q, k_cache, v_cache, a, num_tiles, nd_mfma, parts, st);
    else
      launch_mfma<16, 8>(out, q, k_cache, v_cache, a, num_tiles, nd_mfma, parts, st);
    rc = static_cast<int>(hipGetLastError());
    if (rc) return rc;
    num_tiles = 0;
    if (nd_mfma > 0) num_decode = 0;
    if (num_decode <= 0) return 0;
  }
  MIXK_DISPATCH(dtype, rc = launch_rows<T>(out, q, k_cache, v_cache, a, num_tiles, num_decode,
                                           max_decode_kv, st));
  return rc;
}
