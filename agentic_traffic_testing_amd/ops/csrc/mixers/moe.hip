// Routed experts: top-k routing (sigmoid or softmax scores, optional choice correction and
// group-limited choice, optional renormalisation), an on-device plan that sorts the (row, choice) pairs by
// expert into tiles, and grouped matrix products over the tiles - no host round trip, so a step
// can be recorded in a graph.
//
// * moe_route: one wave per row of fp32 router logits [T, E]; scores = sigmoid, or softmax over
//   the row; choice scores = scores (+ correction[e]); with groups > 1 a group (E / groups
//   neighbouring experts) scores its largest choice score, `keep` rounds of wave-wide arg-max
//   pick the groups whose experts stay eligible; `top` rounds of wave-wide arg-max over the
//   eligible choice scores (ties: lowest index) give idx [T, top]; wts [T, top] are the plain
//   scores of the chosen, optionally divided by their sum + 1e-20.
// * moe_plan (one workgroup): histogram of the P = T * top pairs over the experts, prefix sums,
//   the tile table (expert, first sorted position, rows <= rows_per_tile), and the pairs scattered
//   into expert order.  plan = [ntiles, 0, tile_expert[max_tiles], tile_start[max_tiles],
//   tile_rows[max_tiles], sorted_pair[P]].  The order inside an expert is arbitrary; a row's
//   result does not depend on its place in a tile.
// * moe_gemm: out = rows . W[e]^T per tile.
//   GLU form (first product): rows are gathered from h by the pair's row, two weight tiles (gate,
//   up) share the row tile, and the epilogue applies the router weight w and the clamped GLU:
//   g = min(w acc_g, limit), u = clamp(w acc_u, -limit, limit), act = g sigmoid(alpha g) (u + 1),
//   stored in sorted order.  Plain form (second product): rows are the activations in sorted
//   order, results go to the pair's own row of y [P, W]; with `split` > 1 a tile's K range is
//   cut over that many workgroups (a decode step has few tiles and a long K) and the fp32
//   partials go to rows pair * split + z of y [P * split, W], summed by pair_sum together with
//   the row's choices.
//   Matrix-core kernel (bf16, K % 8 == 0): mfma_f32_32x32x16_bf16 with the weights as the A operand
//   (features = accumulator rows, so a lane holds 4 consecutive features of one row of the
//   output), 4 waves = 2 x 2, K in steps of 64 through LDS with the next step's loads in flight;
//   tiles of 64 features x 64 rows for steps of few rows (they stream the weights once); for
//   prefill-sized steps, where the operand traffic per product decides, 128 rows x 128 features
//   (four 32 x 32 blocks per wave) in the plain form and 128 rows x 64 features of gate and of
//   up in the GLU form (the same four blocks per wave and LDS per workgroup).  Rows kernel (any dtype and sizes): fp32 FMA, 4 x 4 outputs per thread from fp32
//   LDS tiles of 64 rows x 64 features.
//   With glu = 1 the first product's epilogue is the plain SiLU GLU, silu(acc_g) acc_u, without
//   the router weight (moe_combine applies it to the expert's output).
// * clamped_glu (rows of [gate | up] products from library GEMMs), pair_sum (a row's choices and
//   split partials added in fp32), moe_combine (out[t] = sum_j w[t, j] y[t, j] (+ addend[t]) in
//   fp32, where an index >= E is an identity expert whose output is the row of h itself).
#include "mix_common.h"
#include "mixers.h"

namespace mixk {

constexpr int kMoeRows = 64;        // rows per tile
constexpr int kMoeFeat = 64;        // output features per workgroup
constexpr int kMaxExperts = 1024;

__device__ __forceinline__ void wave_argmax(float& best, int& be) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ob = __shfl_xor(best, o, kWave);
    const int oe = __shfl_xor(be, o, kWave);
    if (ob > best || (ob == best && oe < be)) {
      best = ob;
      be = oe;
    }
  }
}

// Every wave runs to the end (rows past T_ recompute the last row and write nothing), so the
// workgroup barriers around the LDS exchange of the grouped form are reached by all of them.
// PER: experts per lane (64 PER >= E), so few experts cost few registers, LDS and instructions.
template <int PER>
__global__ void __launch_bounds__(256)
moe_route_kernel(int* __restrict__ idx, float* __restrict__ wts, const float* __restrict__ logits,
                 const float* __restrict__ correction, int T_, int E, int top, int softmax,
                 int groups, int keep, int renorm) {
  __shared__ float s_choice[4][PER * kWave];
  __shared__ unsigned char s_kept[4][PER * kWave];
  const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t_raw = blockIdx.x * 4 + wv;
  const bool live = t_raw < T_;
  const int t = live ? t_raw : T_ - 1;
  const float* row = logits + static_cast<int64_t>(t) * E;
  float sc[PER], ch[PER];
  int pick[PER];
  float zmax = -INFINITY;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int e = lane + j * kWave;
    sc[j] = e < E ? row[e] : -INFINITY;
    zmax = fmaxf(zmax, sc[j]);
    pick[j] = -1;
  }
  if (softmax) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) zmax = fmaxf(zmax, __shfl_xor(zmax, o, kWave));
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      sc[j] = lane + j * kWave < E ? expf(sc[j] - zmax) : 0.f;
      sum += sc[j];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int j = 0; j < PER; ++j) sc[j] = sc[j] / sum;
  } else {
#pragma unroll
    for (int j = 0; j < PER; ++j) sc[j] = sigmoidf_(sc[j]);
  }
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int e = lane + j * kWave;
    ch[j] = e < E ? sc[j] + (correction != nullptr ? correction[e] : 0.f) : -INFINITY;
  }
  if (groups > 1) {   // uniform over the launch
    const int gs = E / groups;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lane + j * kWave;
      if (e < E) s_choice[wv][e] = ch[j];
      if (e < groups) s_kept[wv][e] = 0;
    }
    __syncthreads();
    float gm[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int g = lane + j * kWave;
      gm[j] = -INFINITY;
      if (g < groups)
        for (int i = 0; i < gs; ++i) gm[j] = fmaxf(gm[j], s_choice[wv][g * gs + i]);
    }
    for (int k = 0; k < keep; ++k) {
      float best = -INFINITY;
      int be = 0x7fffffff;
#pragma unroll
      for (int j = 0; j < PER; ++j)
        if (gm[j] > best) {
          best = gm[j];
          be = lane + j * kWave;
        }
      wave_argmax(best, be);
#pragma unroll
      for (int j = 0; j < PER; ++j)
        if (lane + j * kWave == be) {
          gm[j] = -INFINITY;
          s_kept[wv][be] = 1;
        }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lane + j * kWave;
      if (e < E && !s_kept[wv][e / gs]) ch[j] = -INFINITY;
    }
  }
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int be = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (ch[j] > best) {   // ascending e inside a lane: the first of equals wins
        best = ch[j];
        be = lane + j * kWave;
      }
    wave_argmax(best, be);
    if (be == 0x7fffffff) {   // nothing eligible is left (non-finite scores): a zero weight
      if (live && lane == 0) {
        idx[static_cast<int64_t>(t) * top + k] = 0;
        wts[static_cast<int64_t>(t) * top + k] = 0.f;
      }
      continue;
    }
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (lane + j * kWave == be) {
        ch[j] = -INFINITY;
        pick[j] = k;
      }
  }
  float tot = 0.f;
#pragma unroll
  for (int j = 0; j < PER; ++j)
    if (pick[j] >= 0) tot += sc[j];
  tot = wave_sum(tot);
  if (!live) return;
#pragma unroll
  for (int j = 0; j < PER; ++j)
    if (pick[j] >= 0) {
      idx[static_cast<int64_t>(t) * top + pick[j]] = lane + j * kWave;
      wts[static_cast<int64_t>(t) * top + pick[j]] = renorm ? sc[j] / (tot + 1e-20f) : sc[j];
    }
}

__global__ void __launch_bounds__(1024)
moe_plan_kernel(int* __restrict__ plan, const int* __restrict__ idx, int P, int E, int max_tiles,
                int rows_per_tile) {
  __shared__ int cnt[kMaxExperts], cur[kMaxExperts];
  int* tile_expert = plan + 2;
  int* tile_start = tile_expert + max_tiles;
  int* tile_rows = tile_start + max_tiles;
  int* sorted = tile_rows + max_tiles;
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = idx[p];
    if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int off = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      cur[e] = off;
      for (int r = 0; r < cnt[e] && nt < max_tiles; r += rows_per_tile, ++nt) {
        tile_expert[nt] = e;
        tile_start[nt] = off + r;
        tile_rows[nt] = min(rows_per_tile, cnt[e] - r);
      }
      off += cnt[e];
    }
    plan[0] = nt;
    plan[1] = 0;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = idx[p];
    if (e >= 0 && e < E) sorted[atomicAdd(&cur[e], 1)] = p;
  }
}

struct MoeArgs {
  const int* plan;
  const float* wts;   // GLU: router weight of every pair [P]
  int max_tiles, top, N, K;
  int64_t x_stride;
  int64_t w_estride;   // elements between two experts' matrices
  float limit, alpha;
  int glu;             // GLU form: 0 clamped GLU of the weighted products, 1 silu(g) u, no weight
  int split, k_chunk;  // plain form: blockIdx.z takes K range [z k_chunk, (z + 1) k_chunk) and
                       // writes its fp32 partial to row pair * split + z
};

__device__ __forceinline__ float clamped_glu(float g, float u, float wt, float limit, float alpha) {
  g = fminf(g * wt, limit);
  u = fminf(fmaxf(u * wt, -limit), limit);
  return g * sigmoidf_(alpha * g) * (u + 1.0f);
}

__device__ __forceinline__ float glu_act(float g, float u, float wt, const MoeArgs& a) {
  return a.glu == 1 ? siluf_(g) * u : clamped_glu(g, u, wt, a.limit, a.alpha);
}

typedef __attribute__((ext_vector_type(8))) __bf16 mbf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 mbf16x4;
typedef __attribute__((ext_vector_type(16))) float mf32x16;
typedef __attribute__((ext_vector_type(4))) unsigned int mu32x4;

__device__ __forceinline__ void st4(__bf16* p, const float* o) {
  mbf16x4 v;
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = static_cast<__bf16>(o[i]);
  *reinterpret_cast<mbf16x4*>(p) = v;
}
__device__ __forceinline__ void st4(float* p, const float* o) {
  *reinterpret_cast<f32x4v*>(p) = f32x4v{o[0], o[1], o[2], o[3]};
}

constexpr int kMoeBK = 64;
constexpr int kMoeLds = kMoeBK + 8;   // padded row of a staged tile (bf16 elements)

// Workgroup = 2 x 2 waves, a wave = MF x MR blocks of 32 features x 32 rows: tiles of 64 MF features
// x 64 MR rows.  The next K step's global loads are issued into registers before the current
// step's products and written to LDS after them.
template <bool GLU, int MF, int MR, typename OutT>
__global__ void __launch_bounds__(256)
moe_gemm_mfma_kernel(OutT* __restrict__ out, const __bf16* __restrict__ x,
                     const __bf16* __restrict__ w1, const __bf16* __restrict__ w2, MoeArgs a) {
  constexpr int FT = 64 * MF, RT = 64 * MR, WCH = 2 * MF, XCH = 2 * MR;
  __shared__ __attribute__((aligned(16))) __bf16 lds_w1[FT * kMoeLds];
  __shared__ __attribute__((aligned(16))) __bf16 lds_w2[GLU ? FT * kMoeLds : 8];
  __shared__ __attribute__((aligned(16))) __bf16 lds_x[RT * kMoeLds];
  __shared__ int src_row[RT];
  // Workgroups go to the 8 XCDs round robin by their linear id; the tiles of one expert that
  // share a block of features read the same weights, so ids are remapped to give every XCD a
  // contiguous run of (feature block, tile) pairs and the weights pass through one L2 only.
  int lin = blockIdx.y * gridDim.x + blockIdx.x;
  const int full = static_cast<int>(gridDim.x * gridDim.y) / 8 * 8;
  if (lin < full) lin = (lin % 8) * (full / 8) + lin / 8;
  const int tile = lin % static_cast<int>(gridDim.x), fblock = lin / static_cast<int>(gridDim.x);
  if (tile >= a.plan[0]) return;
  const int* tile_expert = a.plan + 2;
  const int* tile_start = tile_expert + a.max_tiles;
  const int* tile_rows = tile_start + a.max_tiles;
  const int* sorted = tile_rows + a.max_tiles;
  const int e = tile_expert[tile], start = tile_start[tile], nrows = tile_rows[tile];
  const int N = a.N, K = a.K, f0 = fblock * FT;
  const int k_begin = blockIdx.z * a.k_chunk, k_end = min(K, k_begin + a.k_chunk);
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int r = lane & 31, h = lane >> 5, fm = w & 1, rn = w >> 1;
  for (int i = tid; i < RT; i += 256)
    src_row[i] = i < nrows ? (GLU ? sorted[start + i] / a.top : start + i) : -1;
  __syncthreads();
  const __bf16* w1e = w1 + e * a.w_estride;
  const __bf16* w2e = GLU ? w2 + e * a.w_estride : nullptr;
  // this thread's 16-byte chunks of a staged K step: (row, 8-channel group) of each tile
  int w_off[WCH], l_off[WCH > XCH ? WCH : XCH];
  int64_t x_off[XCH];
#pragma unroll
  for (int c = 0; c < (WCH > XCH ? WCH : XCH); ++c) {
    const int ch = tid + c * 256, row = ch >> 3, kc = (ch & 7) * 8;
    l_off[c] = row * kMoeLds + kc;
    if (c < WCH) w_off[c] = f0 + row < N ? (f0 + row) * K + kc : -1;
    if (c < XCH) x_off[c] = src_row[row] >= 0 ? src_row[row] * a.x_stride + kc : -1;
  }
  mu32x4 p1[WCH], p2[GLU ? WCH : 1], px[XCH];
  auto fetch = [&](int k0) {
    const int kc = (tid & 7) * 8;
    const bool kin = k0 + kc < k_end;
#pragma unroll
    for (int c = 0; c < WCH; ++c) {
      p1[c] = mu32x4{0u, 0u, 0u, 0u};
      if (GLU) p2[c] = mu32x4{0u, 0u, 0u, 0u};
      if (kin && w_off[c] >= 0) {
        p1[c] = *reinterpret_cast<const mu32x4*>(w1e + w_off[c] + k0);
        if (GLU) p2[c] = *reinterpret_cast<const mu32x4*>(w2e + w_off[c] + k0);
      }
    }
#pragma unroll
    for (int c = 0; c < XCH; ++c) {
      px[c] = mu32x4{0u, 0u, 0u, 0u};
      if (kin && x_off[c] >= 0) px[c] = *reinterpret_cast<const mu32x4*>(x + x_off[c] + k0);
    }
  };
  mf32x16 acc1[MF][MR], acc2[GLU ? MF : 1][GLU ? MR : 1];
#pragma unroll
  for (int i = 0; i < MF; ++i)
#pragma unroll
    for (int j = 0; j < MR; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        acc1[i][j][q] = 0.f;
        if (GLU) acc2[i][j][q] = 0.f;
      }
  fetch(k_begin);
  for (int k0 = k_begin; k0 < k_end; k0 += kMoeBK) {
    if (k0 > k_begin) __syncthreads();   // the previous step's reads of LDS are done
#pragma unroll
    for (int c = 0; c < WCH; ++c) {
      *reinterpret_cast<mu32x4*>(lds_w1 + l_off[c]) = p1[c];
      if (GLU) *reinterpret_cast<mu32x4*>(lds_w2 + l_off[c]) = p2[c];
    }
#pragma unroll
    for (int c = 0; c < XCH; ++c) *reinterpret_cast<mu32x4*>(lds_x + l_off[c]) = px[c];
    __syncthreads();
    if (k0 + kMoeBK < k_end) fetch(k0 + kMoeBK);
#pragma unroll
    for (int ks = 0; ks < kMoeBK / 16; ++ks) {
      mbf16x8 xf[MR];
#pragma unroll
      for (int j = 0; j < MR; ++j)
        xf[j] = *reinterpret_cast<const mbf16x8*>(lds_x + ((rn * MR + j) * 32 + r) * kMoeLds +
                                                  ks * 16 + 8 * h);
#pragma unroll
      for (int i = 0; i < MF; ++i) {
        const int wrow = ((fm * MF + i) * 32 + r) * kMoeLds + ks * 16 + 8 * h;
        const mbf16x8 a1 = *reinterpret_cast<const mbf16x8*>(lds_w1 + wrow);
#pragma unroll
        for (int j = 0; j < MR; ++j)
          acc1[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, xf[j], acc1[i][j], 0, 0, 0);
        if (GLU) {
          const mbf16x8 a2 = *reinterpret_cast<const mbf16x8*>(lds_w2 + wrow);
#pragma unroll
          for (int j = 0; j < MR; ++j)
            acc2[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a2, xf[j], acc2[i][j], 0, 0, 0);
        }
      }
    }
  }
  // lane (r, h) of block (i, j) holds output row (rn MR + j) 32 + r and features
  // (fm MF + i) 32 + 8 (q / 4) + 4 h + (q % 4)
#pragma unroll
  for (int j = 0; j < MR; ++j) {
    const int lrow = (rn * MR + j) * 32 + r;
    if (lrow >= nrows) continue;
    const int pair = sorted[start + lrow];
    const float wt = GLU ? a.wts[pair] : 1.f;
    OutT* orow = out + (GLU ? static_cast<int64_t>(start + lrow)
                            : static_cast<int64_t>(pair) * a.split + blockIdx.z) * N;
#pragma unroll
    for (int i = 0; i < MF; ++i)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int f = f0 + (fm * MF + i) * 32 + 8 * i4 + 4 * h;
        float v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
          v[q] = GLU ? glu_act(acc1[i][j][4 * i4 + q], acc2[GLU ? i : 0][GLU ? j : 0][4 * i4 + q],
                               wt, a)
                     : acc1[i][j][4 * i4 + q];
        if (f + 3 < N && (N & 3) == 0) {
          st4(orow + f, v);
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (f + q < N) orow[f + q] = static_cast<OutT>(v[q]);
        }
      }
  }
}

constexpr int kRowsBK = 16;

template <typename T, bool GLU>
__global__ void __launch_bounds__(256)
moe_gemm_rows_kernel(T* __restrict__ out, const T* __restrict__ x, const T* __restrict__ w1,
                     const T* __restrict__ w2, MoeArgs a) {
  __shared__ float s_x[kMoeRows][kRowsBK + 1], s_w1[kMoeFeat][kRowsBK + 1];
  __shared__ float s_w2[GLU ? kMoeFeat : 1][kRowsBK + 1];
  __shared__ int src_row[kMoeRows];
  const int tile = blockIdx.x;
  if (tile >= a.plan[0]) return;
  const int* tile_expert = a.plan + 2;
  const int* tile_start = tile_expert + a.max_tiles;
  const int* tile_rows = tile_start + a.max_tiles;
  const int* sorted = tile_rows + a.max_tiles;
  const int e = tile_expert[tile], start = tile_start[tile], nrows = tile_rows[tile];
  const int N = a.N, K = a.K, f0 = blockIdx.y * kMoeFeat;
  const int tid = threadIdx.x, tr = tid >> 4, tc = tid & 15;   // rows 4 tr .., features tc + 16 j
  if (tid < kMoeRows)
    src_row[tid] = tid < nrows ? (GLU ? sorted[start + tid] / a.top : start + tid) : -1;
  __syncthreads();
  const T* w1e = w1 + e * a.w_estride;
  const T* w2e = GLU ? w2 + e * a.w_estride : nullptr;
  float acc1[4][4], acc2[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc1[i][j] = acc2[i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += kRowsBK) {
    if (k0 > 0) __syncthreads();
    for (int i = tid; i < kMoeRows * kRowsBK; i += 256) {
      const int row = i / kRowsBK, kk = i - row * kRowsBK;
      const bool kin = k0 + kk < K;
      const int sr = src_row[row];
      s_x[row][kk] = (kin && sr >= 0) ? ldf(x + sr * a.x_stride + k0 + kk) : 0.f;
      const bool fin = kin && f0 + row < N;
      s_w1[row][kk] = fin ? ldf(w1e + static_cast<int64_t>(f0 + row) * K + k0 + kk) : 0.f;
      if (GLU) s_w2[row][kk] = fin ? ldf(w2e + static_cast<int64_t>(f0 + row) * K + k0 + kk) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kRowsBK; ++kk) {
      float xv[4], wa[4], wb[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) xv[i] = s_x[4 * tr + i][kk];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        wa[j] = s_w1[tc + 16 * j][kk];
        wb[j] = GLU ? s_w2[tc + 16 * j][kk] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc1[i][j] += xv[i] * wa[j];
          if (GLU) acc2[i][j] += xv[i] * wb[j];
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int lrow = 4 * tr + i;
    if (lrow >= nrows) continue;
    const int pair = sorted[start + lrow];
    const float wt = GLU ? a.wts[pair] : 1.f;
    T* orow = out + static_cast<int64_t>(GLU ? start + lrow : pair) * N;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int f = f0 + tc + 16 * j;
      if (f < N)
        stf(orow + f, GLU ? glu_act(acc1[i][j], acc2[i][j], wt, a) : acc1[i][j]);
    }
  }
}

// Clamped GLU over rows of [gate | up] products (the library path of prefill-sized steps): one
// thread per output element, the row's router weight applied to both products first.
template <typename T>
__global__ void clamped_glu_kernel(T* __restrict__ out, const T* __restrict__ gu,
                                   const float* __restrict__ wts, int ff, float limit,
                                   float alpha) {
  const int f = blockIdx.y * blockDim.x + threadIdx.x;
  if (f >= ff) return;
  const int64_t r = blockIdx.x;
  const T* row = gu + r * 2 * ff;
  stf(out + r * ff + f, clamped_glu(ldf(row + f), ldf(row + ff + f), wts[r], limit, alpha));
}

// out[t] = sum_j y[t, j] over a row's `top` summands, accumulated in fp32 in the order of j.
template <typename T, typename TI>
__global__ void pair_sum_kernel(T* __restrict__ out, const TI* __restrict__ y, int top, int W) {
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= W) return;
  const TI* src = y + static_cast<int64_t>(blockIdx.x) * top * W + i;
  float a = 0.f;
  for (int j = 0; j < top; ++j) a += ldf(src + static_cast<int64_t>(j) * W);
  stf(out + static_cast<int64_t>(blockIdx.x) * W + i, a);
}

template <typename T, typename TI>   // W % 8 == 0: eight adjacent features per thread
__global__ void pair_sum_vec_kernel(T* __restrict__ out, const TI* __restrict__ y, int top, int W) {
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (i >= W) return;
  const TI* src = y + static_cast<int64_t>(blockIdx.x) * top * W + i;
  float a[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int j = 0; j < top; ++j) {
    float v[8];
    ld8(src + static_cast<int64_t>(j) * W, v);
#pragma unroll
    for (int e = 0; e < 8; ++e) a[e] += v[e];
  }
  st8(out + static_cast<int64_t>(blockIdx.x) * W + i, a);
}

// out[t] = sum_j wts[t, j] * v_j (+ addend[t]) in fp32, j in order; v_j = the sum of the pair's
// `split` adjacent rows of y, or the row of h when idx[t, j] >= E (an identity expert).
template <typename T, typename TY, bool VEC>
__global__ void moe_combine_kernel(T* __restrict__ out, const TY* __restrict__ y,
                                   const int* __restrict__ idx, const float* __restrict__ wts,
                                   const T* __restrict__ h, const T* __restrict__ addend, int top,
                                   int split, int E, int W) {
  constexpr int N = VEC ? 8 : 1;
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * N;
  if (i >= W) return;
  const int64_t t = blockIdx.x;
  float acc[N];
#pragma unroll
  for (int e = 0; e < N; ++e) acc[e] = 0.f;
  for (int j = 0; j < top; ++j) {
    const int ex = idx[t * top + j];
    const float w = wts[t * top + j];
    float v[N];
    if (ex >= E) {
      if (VEC) ld8(h + t * W + i, v); else v[0] = ldf(h + t * W + i);
    } else {
#pragma unroll
      for (int e = 0; e < N; ++e) v[e] = 0.f;
      const TY* src = y + (t * top + j) * split * W + i;
      for (int z = 0; z < split; ++z) {
        float u[N];
        if (VEC) ld8(src + static_cast<int64_t>(z) * W, u); else u[0] = ldf(src + static_cast<int64_t>(z) * W);
#pragma unroll
        for (int e = 0; e < N; ++e) v[e] += u[e];
      }
    }
#pragma unroll
    for (int e = 0; e < N; ++e) acc[e] += w * v[e];
  }
  if (addend != nullptr) {
    float u[N];
    if (VEC) ld8(addend + t * W + i, u); else u[0] = ldf(addend + t * W + i);
#pragma unroll
    for (int e = 0; e < N; ++e) acc[e] += u[e];
  }
  if (VEC) st8(out + t * W + i, acc); else stf(out + t * W + i, acc[0]);
}

}  // namespace mixk

using namespace mixk;

extern "C" int mixk_moe_combine(void* out, const void* y, int y_f32, const int* idx,
                                const float* wts, const void* h, const void* addend, int T_,
                                int top, int split, int E, int W, int dtype, hipStream_t st) {
  if (T_ <= 0 || W <= 0) return 0;
  if (top < 1 || split < 1) return -1;
  auto al = [](const void* p, uintptr_t m) { return (reinterpret_cast<uintptr_t>(p) & m) == 0; };
  const uintptr_t am = dtype == 2 ? 31 : 15;
  const bool vec = W % 8 == 0 && al(out, am) && al(h, am) && al(y, y_f32 ? 31 : am) &&
                   (addend == nullptr || al(addend, am));
  const dim3 grid(T_, vec ? (W / 8 + 127) / 128 : (W + 255) / 256), block(vec ? 128 : 256);
#define MIXK_COMBINE(TY, VEC)                                                                     \
  hipLaunchKernelGGL((moe_combine_kernel<T, TY, VEC>), grid, block, 0, st, static_cast<T*>(out),  \
                     static_cast<const TY*>(y), idx, wts, static_cast<const T*>(h),               \
                     static_cast<const T*>(addend), top, split, E, W)
  MIXK_DISPATCH(dtype, {
    if (y_f32 && vec)
      MIXK_COMBINE(float, true);
    else if (y_f32)
      MIXK_COMBINE(float, false);
    else if (vec)
      MIXK_COMBINE(T, true);
    else
      MIXK_COMBINE(T, false);
  });
#undef MIXK_COMBINE
  return static_cast<int>(hipGetLastError());
}

// y_f32: the summands are fp32 (split-K partials) whatever the output dtype.
extern "C" int mixk_pair_sum(void* out, const void* y, int y_f32, int T_, int top, int W,
                             int dtype, hipStream_t st) {
  if (T_ <= 0 || W <= 0) return 0;
  const bool vec = W % 8 == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(y) & 31) == 0;
  const dim3 grid(T_, vec ? (W / 8 + 127) / 128 : (W + 255) / 256), block(vec ? 128 : 256);
  MIXK_DISPATCH(dtype, {
    if (y_f32 && vec)
      hipLaunchKernelGGL((pair_sum_vec_kernel<T, float>), grid, block, 0, st, static_cast<T*>(out),
                         static_cast<const float*>(y), top, W);
    else if (y_f32)
      hipLaunchKernelGGL((pair_sum_kernel<T, float>), grid, block, 0, st, static_cast<T*>(out),
                         static_cast<const float*>(y), top, W);
    else if (vec)
      hipLaunchKernelGGL((pair_sum_vec_kernel<T, T>), grid, block, 0, st, static_cast<T*>(out),
                         static_cast<const T*>(y), top, W);
    else
      hipLaunchKernelGGL((pair_sum_kernel<T, T>), grid, block, 0, st, static_cast<T*>(out),
                         static_cast<const T*>(y), top, W);
  });
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_clamped_glu(void* out, const void* gu, const float* wts, int R, int ff,
                                float limit, float alpha, int dtype, hipStream_t st) {
  if (R <= 0 || ff <= 0) return 0;
  MIXK_DISPATCH(dtype, hipLaunchKernelGGL(clamped_glu_kernel<T>, dim3(R, (ff + 255) / 256),
                                          dim3(256), 0, st, static_cast<T*>(out),
                                          static_cast<const T*>(gu), wts, ff, limit, alpha));
  return static_cast<int>(hipGetLastError());
}

extern "C" int mixk_moe_route(int* idx, float* wts, const float* logits, const float* correction,
                              int T_, int E, int top, int softmax, int groups, int keep,
                              int renorm, hipStream_t st) {
  if (T_ <= 0) return 0;
  if (E < 1 || E > kMaxExperts || top < 1 || top > E || groups < 1 || E % groups != 0 ||
      keep < 1 || keep > groups || top > keep * (E / groups))
    return -1;
#define MIXK_ROUTE(PER)                                                                          \
  hipLaunchKernelGGL(moe_route_kernel<PER>, dim3((T_ + 3) / 4), dim3(256), 0, st, idx, wts,      \
                     logits, correction, T_, E, top, softmax, groups, keep, renorm)
  if (E <= kWave)
    MIXK_ROUTE(1);
  else if (E <= 4 * kWave)
    MIXK_ROUTE(4);
  else
    MIXK_ROUTE(kMaxExperts / kWave);
#undef MIXK_ROUTE
  return static_cast<int>(hipGetLastError());
}

// y [T * top, W] (a pair's row), act [T * top, ff] (sorted order), plan [2 + 3 max_tiles + T * top].
// tile_rows: 64, or 128 for the large matrix-core tiles (bf16, widths % 8 == 0 only).
// split > 1 (matrix-core kernel with 64-row tiles only): the down product's K range is cut in
// `split` parts and y is fp32 [T * top * split, W], a pair's partials in adjacent rows.
extern "C" int mixk_moe_experts(void* y, void* act, int* plan, const void* h, const int* idx,
                                const float* wts, const void* w_gate, const void* w_up,
                                const void* w_down, int T_, int top, int E, int ff, int W,
                                int64_t gu_estride, int max_tiles, int tile_rows, int split,
                                float limit, float alpha, int glu, int dtype, hipStream_t st) {
  if (T_ <= 0) return 0;
  if (glu != 0 && glu != 1) return -1;
  const int P = T_ * top;
  const bool mfma = dtype == 0 && W % 8 == 0 && ff % 8 == 0;
  if (E < 1 || E > kMaxExperts || (tile_rows != 64 && !(tile_rows == 128 && mfma)) ||
      max_tiles < P / tile_rows + min(E, P) || split < 1 ||
      (split > 1 && !(mfma && tile_rows == 64)))
    return -1;
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), 0, st, plan, idx, P, E, max_tiles,
                     tile_rows);
  MoeArgs a1{plan, wts, max_tiles, top, ff, W, static_cast<int64_t>(W), gu_estride, limit, alpha,
             glu, 1, W};
  // the down product's K range per workgroup: a multiple of the staged K step
  const int k_chunk = split > 1 ? ((ff + split - 1) / split + kMoeBK - 1) / kMoeBK * kMoeBK : ff;
  MoeArgs a2{plan, wts, max_tiles, top, W, ff, static_cast<int64_t>(ff),
             static_cast<int64_t>(W) * ff, limit, alpha, glu, split, k_chunk};
  // feature blocks: 64 for the gate | up form (two weight tiles per block), 128 for the down form
  // of the large tiles
  const int ft2 = tile_rows == 128 && mfma ? 128 : kMoeFeat;
  const dim3 g1(max_tiles, (ff + kMoeFeat - 1) / kMoeFeat), g2(max_tiles, (W + ft2 - 1) / ft2);
#define MIXK_MOE_MFMA(MF, MR, YT, GZ)                                                             \
  do {                                                                                            \
    hipLaunchKernelGGL((moe_gemm_mfma_kernel<true, 1, MR, __bf16>), g1, dim3(256), 0, st,         \
                       static_cast<__bf16*>(act), static_cast<const __bf16*>(h),                  \
                       static_cast<const __bf16*>(w_gate), static_cast<const __bf16*>(w_up), a1); \
    hipLaunchKernelGGL((moe_gemm_mfma_kernel<false, MF, MR, YT>), dim3(g2.x, g2.y, GZ), dim3(256), \
                       0, st, static_cast<YT*>(y), static_cast<const __bf16*>(act),               \
                       static_cast<const __bf16*>(w_down), static_cast<const __bf16*>(nullptr),   \
                       a2);                                                                       \
  } while (0)
  if (mfma) {
    if (tile_rows == 128)
      MIXK_MOE_MFMA(2, 2, __bf16, 1);
    else if (split > 1)
      MIXK_MOE_MFMA(1, 1, float, split);
    else
      MIXK_MOE_MFMA(1, 1, __bf16, 1);
    return static_cast<int>(hipGetLastError());
  }
#undef MIXK_MOE_MFMA
  MIXK_DISPATCH(dtype, {
    hipLaunchKernelGGL((moe_gemm_rows_kernel<T, true>), g1, dim3(256), 0, st, static_cast<T*>(act),
                       static_cast<const T*>(h), static_cast<const T*>(w_gate),
                       static_cast<const T*>(w_up), a1);
    hipLaunchKernelGGL((moe_gemm_rows_kernel<T, false>), g2, dim3(256), 0, st, static_cast<T*>(y),
                       static_cast<const T*>(act), static_cast<const T*>(w_down),
                       static_cast<const T*>(nullptr), a2);
  });
  return static_cast<int>(hipGetLastError());
}
