// Mixture-of-experts feed-forward with device-side routing (no host synchronisation):
//
//   route   : fp32 logits z = R h + b, the `top` largest (ties: lowest index), softmax over
//             those only; also the fp32 logit of the always-on expert's gate.  Scored form:
//             s = sigmoid(z); the choice goes by s + correction, limited to the `keep` best of
//             `groups` equal groups of neighbouring experts (a group's score: the sum of its two
//             largest choice scores); weights s / (sum of the chosen s + 1e-20) * scale
//   align   : slots (token, j) bucketed by expert into tile-aligned position ranges
//   gemm    : per position tile (one expert) C = A W_e^T on 16 x 16 MFMAs; "up" gathers token
//             rows and applies the activation, "down" scatters rows back to their slots
//   combine : out32[t] = sum_j weight[t, j] * y[slot(t, j)]   (fp32, fixed order)
//
// Position tiles are TM rows; a tile belongs to one expert (tile_expert, -1 = unused).
#include <algorithm>

#include "seqmix_common.h"

namespace {

constexpr int TM = 64, TN = 256, MAX_E = 256;  // position tile rows, output columns per workgroup (4 waves x 64)

// One workgroup per token: the four waves share the experts (and the gate row), a wave's lanes
// stride over the width with 16-byte loads of the fp32 router rows; thread 0 then picks the top-k.
template <typename T>
__global__ __launch_bounds__(256) void route_kernel(const T* __restrict__ h, const float* __restrict__ rw,
                                                    const float* __restrict__ rb, const float* __restrict__ gw,
                                                    int* __restrict__ idx, float* __restrict__ wts,
                                                    float* __restrict__ gate, int W, int E, int top, int scored,
                                                    const float* __restrict__ corr, int groups, int keep, float wscale) {
  __shared__ float z[MAX_E + 1], sc[MAX_E], gs[MAX_E];   // logits / choice scores, sigmoid scores, group scores
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* row = h + static_cast<size_t>(t) * W;
  const int rows = E + (gw != nullptr ? 1 : 0);
  const bool vec = (W & 3) == 0;
  for (int e = wave; e < rows; e += 4) {
    const float* wrow = e < E ? rw + static_cast<size_t>(e) * W : gw;
    float d = 0.f;
    if (vec) {
      for (int i = 4 * lane; i < W; i += 256) {
        const f32x4 wv = *reinterpret_cast<const f32x4*>(wrow + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) d += Elem<T>::ld(row[i + j]) * wv[j];
      }
    } else {
      for (int i = lane; i < W; i += 64) d += Elem<T>::ld(row[i]) * wrow[i];
    }
    d = wave_sum(d);
    if (lane == 0) z[e] = d + ((e < E && rb) ? rb[e] : 0.f);
  }
  __syncthreads();
  if (threadIdx.x == 0 && scored) {
    for (int e = 0; e < E; ++e) {
      sc[e] = 1.0f / (1.0f + expf(-z[e]));
      z[e] = sc[e] + (corr != nullptr ? corr[e] : 0.f);
    }
    if (groups > 1 && keep < groups) {
      const int per = E / groups;
      for (int g = 0; g < groups; ++g) {
        float a = -INFINITY, b = -INFINITY;   // the two largest of the group
        for (int e = g * per; e < (g + 1) * per; ++e) {
          const float v = z[e];
          if (v > a) { b = a; a = v; } else if (v > b) { b = v; }
        }
        gs[g] = per > 1 ? a + b : a;
      }
      for (int g = 0; g < groups; ++g) {      // a group stays if fewer than `keep` groups come before it
        int ahead = 0;
        for (int o = 0; o < groups; ++o) ahead += (gs[o] > gs[g] || (gs[o] == gs[g] && o < g)) ? 1 : 0;
        if (ahead >= keep)
          for (int e = g * per; e < (g + 1) * per; ++e) z[e] = -INFINITY;
      }
    }
    float den = 0.f;
    for (int j = 0; j < top; ++j) {
      int be = 0;   // (the host checked that `top` experts are allowed)
      float bv = -INFINITY;
      for (int e = 0; e < E; ++e)
        if (z[e] > bv) { bv = z[e]; be = e; }
      z[be] = -INFINITY;
      idx[t * top + j] = be;
      wts[t * top + j] = sc[be];
      den += sc[be];
    }
    for (int j = 0; j < top; ++j) wts[t * top + j] = wts[t * top + j] / (den + 1e-20f) * wscale;
  } else if (threadIdx.x == 0) {
    if (gw != nullptr) gate[t] = z[E];
    float best0 = 0.f, den = 0.f;
    for (int j = 0; j < top; ++j) {
      int be = 0;
      float bv = -INFINITY;
      for (int e = 0; e < E; ++e)
        if (z[e] > bv) { bv = z[e]; be = e; }
      z[be] = -INFINITY;
      if (j == 0) best0 = bv;
      const float p = expf(bv - best0);
      idx[t * top + j] = be;
      wts[t * top + j] = p;
      den += p;
    }
    for (int j = 0; j < top; ++j) wts[t * top + j] /= den;
  }
}

__global__ __launch_bounds__(1024) void align_kernel(const int* __restrict__ idx, int n_slots, int E,
                                                     int* __restrict__ sorted, int cap, int* __restrict__ tile_expert,
                                                     int n_tiles) {
  __shared__ int cnt[MAX_E], off[MAX_E + 1];
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n_slots; i += blockDim.x) {
    const int e = idx[i];
    if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
  }
  for (int i = threadIdx.x; i < cap; i += blockDim.x) sorted[i] = -1;
  __syncthreads();
  if (threadIdx.x == 0) {
    off[0] = 0;
    for (int e = 0; e < E; ++e) off[e + 1] = off[e] + (cnt[e] + TM - 1) / TM * TM;
  }
  __syncthreads();
  for (int t = threadIdx.x; t < n_tiles; t += blockDim.x) {
    int who = -1;
    for (int e = 0; e < E; ++e)
      if (t * TM >= off[e] && t * TM < off[e + 1]) who = e;
    tile_expert[t] = who;
  }
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n_slots; i += blockDim.x) {
    const int e = idx[i];
    if (e >= 0 && e < E) sorted[off[e] + atomicAdd(&cnt[e], 1)] = i;
  }
}

// Epilogue of a gated expert's first product (act 2).  The N rows of the expert's weight are its
// gate and up rows in alternating groups of 16 ([gate 0..15 | up 0..15 | gate 16..31 | ...]), so a
// wave's n tiles 0 / 2 hold gate columns and tiles 1 / 3 the up columns of the SAME features:
// out[r, f] = silu(gate_f) * up_f with f = n / 2 (N / 2 output columns), both factors and the
// activation rounded to T like a projection's output.
template <typename T>
__device__ __forceinline__ void store_gated(const f32x4 (&acc)[4][4], const int (&slot)[4], T* __restrict__ out,
                                            int64_t out_stride, int scatter, int p0, int n0, int N, int col, int grp) {
  auto rnd = [](float v) { return Elem<T>::ld(Elem<T>::st(v)); };
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (slot[j] < 0) continue;
    const int64_t r = scatter ? slot[j] : p0 + 16 * j + col;
#pragma unroll
    for (int i2 = 0; i2 < 2; ++i2)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (n0 + 32 * i2 + 16 + 4 * grp + q < N) {
          const float g = rnd(acc[2 * i2][j][q]), u = rnd(acc[2 * i2 + 1][j][q]);
          out[r * out_stride + (n0 >> 1) + 16 * i2 + 4 * grp + q] = Elem<T>::st(rnd(g / (1.0f + expf(-g))) * u);
        }
      }
  }
}

// Position p of tile blockIdx.x: slot = sorted[p] (-1: padding).  gather: A row = a[(slot / top)]
// (token rows), else a[p].  scatter: output row = slot, else p.  act 1: relu squared; act 2: `store_gated`.
template <typename T, bool FULL>
__global__ __launch_bounds__(256) void moe_gemm_kernel(const T* __restrict__ a, int64_t a_stride, const T* __restrict__ w,
                                                       T* __restrict__ out, int64_t out_stride,
                                                       const int* __restrict__ sorted,
                                                       const int* __restrict__ tile_expert, int N, int K, int top,
                                                       int gather, int scatter, int act, int vec) {
  typedef typename Elem<T>::frag F;
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int p0 = blockIdx.x * TM, n0 = blockIdx.y * TN + 64 * wave;   // a wave: all 64 rows x 64 columns
  if (n0 >= N) return;
  const T* we = w + static_cast<size_t>(e) * N * K;
  const T* arow[4];
  int slot[4];
  const T* wrow[4];
  bool wok[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int p = p0 + 16 * i + col;
    slot[i] = sorted[p];
    const int64_t r = gather ? (slot[i] < 0 ? 0 : slot[i] / top) : p;
    arow[i] = a + r * a_stride;
    const int n = n0 + 16 * i + col;
    wok[i] = n < N;
    wrow[i] = we + static_cast<size_t>(wok[i] ? n : 0) * K;
  }
  f32x4 acc[4][4];  // [n tile][m tile]: lane holds C[m = col][n = 4 grp + i]
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
  for (int k = 4 * grp; k < K; k += 16) {
    F af[4], wf[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      af[i] = slot[i] >= 0 ? load_frag_t<T, FULL>(arow[i] + k, K - k, vec) : zero_frag<T>();
      wf[i] = wok[i] ? load_frag_t<T, FULL>(wrow[i] + k, K - k, vec) : zero_frag<T>();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = mma16(wf[i], af[j], acc[i][j]);
  }
  if (act == 2) {
    store_gated<T>(acc, slot, out, out_stride, scatter, p0, n0, N, col, grp);
    return;
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (slot[j] < 0) continue;
    const int64_t r = scatter ? slot[j] : p0 + 16 * j + col;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + 16 * i + 4 * grp + q;
        if (n < N) {
          float v = acc[i][j][q];
          if (act == 1) { v = fmaxf(v, 0.f); v *= v; }
          out[r * out_stride + n] = Elem<T>::st(v);
        }
      }
  }
}

// The same product with both operands staged through LDS (K a multiple of 32, 16-byte aligned
// rows): a workgroup loads its 64 x 32 slice of A and 256 x 32 slice of W_e with 16-byte row-wise
// loads (the next slice is in flight in registers while the current one is multiplied), and the
// waves read their MFMA fragments from LDS (rows padded by 8 elements).  bf16 uses the 32-deep
// v_mfma_f32_16x16x32_bf16 (a lane holds 8 consecutive k of its row), fp32 the 4-deep fp32 MFMA.
template <typename T>
__global__ __launch_bounds__(256) void moe_gemm_lds_kernel(const T* __restrict__ a, int64_t a_stride, const T* __restrict__ w,
                                                           T* __restrict__ out, int64_t out_stride,
                                                           const int* __restrict__ sorted,
                                                           const int* __restrict__ tile_expert, int N, int K, int top,
                                                           int gather, int scatter, int act) {
  typedef typename Elem<T>::frag F;
  constexpr int BK = 32, LDK = BK + 8;   // rows stay 16-byte aligned for the 8-element fragment reads
  typedef T Chunk __attribute__((ext_vector_type(8)));   // 8 consecutive elements (16 or 32 bytes)
  __shared__ __attribute__((aligned(16))) T As[TM * LDK];
  __shared__ __attribute__((aligned(16))) T Ws[TN * LDK];
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int p0 = blockIdx.x * TM, nb = blockIdx.y * TN;
  const T* we = w + static_cast<size_t>(e) * N * K;
  // staging role: row tid / 4 of the slice, 8 elements at k = 8 (tid % 4)
  const int s_row = tid >> 2, s_k = (tid & 3) * 8;
  const int a_slot = sorted[p0 + s_row];
  const T* a_src = a + (gather ? static_cast<int64_t>(a_slot < 0 ? 0 : a_slot / top) : static_cast<int64_t>(p0 + s_row)) * a_stride + s_k;
  const T* w_src[4];
  bool w_ok[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = nb + s_row + 64 * i;
    w_ok[i] = n < N;
    w_src[i] = we + static_cast<size_t>(w_ok[i] ? n : 0) * K + s_k;
  }
  Chunk ra, rw0, rw1, rw2, rw3;
  auto get = [&](const T* p, bool ok) {
    Chunk c = Chunk(T(0));
    if (ok) c = *reinterpret_cast<const Chunk*>(p);
    return c;
  };
  auto fetch = [&](int k0) {
    ra = get(a_src + k0, a_slot >= 0);
    rw0 = get(w_src[0] + k0, w_ok[0]);
    rw1 = get(w_src[1] + k0, w_ok[1]);
    rw2 = get(w_src[2] + k0, w_ok[2]);
    rw3 = get(w_src[3] + k0, w_ok[3]);
  };
  int slot[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) slot[j] = sorted[p0 + 16 * j + col];
  f32x4 acc[4][4];  // [n tile][m tile]: lane holds C[m = col][n = 4 grp + i]
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();   // the previous slice has been read
    *reinterpret_cast<Chunk*>(&As[s_row * LDK + s_k]) = ra;
    *reinterpret_cast<Chunk*>(&Ws[(s_row + 0) * LDK + s_k]) = rw0;
    *reinterpret_cast<Chunk*>(&Ws[(s_row + 64) * LDK + s_k]) = rw1;
    *reinterpret_cast<Chunk*>(&Ws[(s_row + 128) * LDK + s_k]) = rw2;
    *reinterpret_cast<Chunk*>(&Ws[(s_row + 192) * LDK + s_k]) = rw3;
    __syncthreads();
    if (k0 + BK < K) fetch(k0 + BK);
    if constexpr (sizeof(T) == 2) {
      bf16x8 af[4], wf[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        af[i] = *reinterpret_cast<const bf16x8*>(&As[(16 * i + col) * LDK + 8 * grp]);
        wf[i] = *reinterpret_cast<const bf16x8*>(&Ws[(64 * wave + 16 * i + col) * LDK + 8 * grp]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i], af[j], acc[i][j], 0, 0, 0);
    } else {
#pragma unroll
    for (int ks = 0; ks < BK; ks += 16) {
      F af[4], wf[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        af[i] = *reinterpret_cast<const F*>(&As[(16 * i + col) * LDK + ks + 4 * grp]);
        wf[i] = *reinterpret_cast<const F*>(&Ws[(64 * wave + 16 * i + col) * LDK + ks + 4 * grp]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = mma16(wf[i], af[j], acc[i][j]);
    }
    }
  }
  const int n0 = nb + 64 * wave;
  if (act == 2) {
    store_gated<T>(acc, slot, out, out_stride, scatter, p0, n0, N, col, grp);
    return;
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (slot[j] < 0) continue;
    const int64_t r = scatter ? slot[j] : p0 + 16 * j + col;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + 16 * i + 4 * grp + q;
        if (n < N) {
          float v = acc[i][j][q];
          if (act == 1) { v = fmaxf(v, 0.f); v *= v; }
          out[r * out_stride + n] = Elem<T>::st(v);
        }
      }
  }
}

// The LDS-staged product for small steps: a workgroup covers 64 columns instead of 256 (wave w takes
// the 16 rows of m-tile w times all 64 columns), so a decode step's few position tiles become four
// times as many workgroups; the staging and the fragment layout are those of `moe_gemm_lds_kernel`.
template <typename T>
__global__ __launch_bounds__(256) void moe_gemm_lds_narrow_kernel(const T* __restrict__ a, int64_t a_stride,
                                                                  const T* __restrict__ w, T* __restrict__ out,
                                                                  int64_t out_stride, const int* __restrict__ sorted,
                                                                  const int* __restrict__ tile_expert, int N, int K, int top,
                                                                  int gather, int scatter, int act) {
  typedef typename Elem<T>::frag F;
  constexpr int BK = 32, LDK = BK + 8, TNN = 64;
  typedef T Chunk __attribute__((ext_vector_type(8)));
  __shared__ __attribute__((aligned(16))) T As[TM * LDK];
  __shared__ __attribute__((aligned(16))) T Ws[TNN * LDK];
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int p0 = blockIdx.x * TM, nb = blockIdx.y * TNN;
  const T* we = w + static_cast<size_t>(e) * N * K;
  const int s_row = tid >> 2, s_k = (tid & 3) * 8;
  const int a_slot = sorted[p0 + s_row];
  const T* a_src = a + (gather ? static_cast<int64_t>(a_slot < 0 ? 0 : a_slot / top) : static_cast<int64_t>(p0 + s_row)) * a_stride + s_k;
  const bool w_ok = nb + s_row < N;
  const T* w_src = we + static_cast<size_t>(w_ok ? nb + s_row : 0) * K + s_k;
  Chunk ra, rw;
  auto get = [&](const T* p, bool ok) {
    Chunk c = Chunk(T(0));
    if (ok) c = *reinterpret_cast<const Chunk*>(p);
    return c;
  };
  auto fetch = [&](int k0) {
    ra = get(a_src + k0, a_slot >= 0);
    rw = get(w_src + k0, w_ok);
  };
  const int slot = sorted[p0 + 16 * wave + col];
  f32x4 acc[4];  // [n tile]: lane holds C[m = col of m-tile `wave`][n = 4 grp + i]
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();   // the previous slice has been read
    *reinterpret_cast<Chunk*>(&As[s_row * LDK + s_k]) = ra;
    *reinterpret_cast<Chunk*>(&Ws[s_row * LDK + s_k]) = rw;
    __syncthreads();
    if (k0 + BK < K) fetch(k0 + BK);
    if constexpr (sizeof(T) == 2) {
      const bf16x8 af = *reinterpret_cast<const bf16x8*>(&As[(16 * wave + col) * LDK + 8 * grp]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bf16x8 wf = *reinterpret_cast<const bf16x8*>(&Ws[(16 * i + col) * LDK + 8 * grp]);
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, af, acc[i], 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < BK; ks += 16) {
        const F af = *reinterpret_cast<const F*>(&As[(16 * wave + col) * LDK + ks + 4 * grp]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const F wf = *reinterpret_cast<const F*>(&Ws[(16 * i + col) * LDK + ks + 4 * grp]);
          acc[i] = mma16(wf, af, acc[i]);
        }
      }
    }
  }
  if (slot < 0) return;
  const int64_t r = scatter ? slot : p0 + 16 * wave + col;
  if (act == 2) {   // gate / up column pairs, as `store_gated`
    auto rnd = [](float v) { return Elem<T>::ld(Elem<T>::st(v)); };
#pragma unroll
    for (int i2 = 0; i2 < 2; ++i2)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (nb + 32 * i2 + 16 + 4 * grp + q < N) {
          const float g = rnd(acc[2 * i2][q]), u = rnd(acc[2 * i2 + 1][q]);
          out[r * out_stride + (nb >> 1) + 16 * i2 + 4 * grp + q] = Elem<T>::st(rnd(g / (1.0f + expf(-g))) * u);
        }
      }
    return;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = nb + 16 * i + 4 * grp + q;
      if (n < N) {
        float v = acc[i][q];
        if (act == 1) { v = fmaxf(v, 0.f); v *= v; }
        out[r * out_stride + n] = Elem<T>::st(v);
      }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void combine_kernel(const T* __restrict__ y, const float* __restrict__ wts,
                                                      float* __restrict__ out, int W, int top) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += 256) {
    float s = 0.f;
    for (int j = 0; j < top; ++j) s += wts[t * top + j] * Elem<T>::ld(y[(static_cast<size_t>(t) * top + j) * W + c]);
    out[static_cast<size_t>(t) * W + c] = s;
  }
}

}  // namespace

BCG_API int bcg_moe_tile_rows() { return TM; }

BCG_API int bcg_moe_route_scored(const void* h, const void* rw, const void* corr, void* idx, void* wts, int T_, int W, int E,
                                 int top, int groups, int keep, float wscale, int is_f32, void* stream) {
  if (T_ <= 0) return 0;
  if (E < 1 || E > MAX_E || top < 1 || top > E || groups < 1 || E % groups || keep < 1 || keep > groups ||
      top > keep * (E / groups)) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (is_f32)
    route_kernel<float><<<T_, 256, 0, s>>>(static_cast<const float*>(h), static_cast<const float*>(rw), nullptr, nullptr,
                                          static_cast<int*>(idx), static_cast<float*>(wts), nullptr, W, E, top, 1,
                                          static_cast<const float*>(corr), groups, keep, wscale);
  else
    route_kernel<bf16_t><<<T_, 256, 0, s>>>(static_cast<const bf16_t*>(h), static_cast<const float*>(rw), nullptr, nullptr,
                                           static_cast<int*>(idx), static_cast<float*>(wts), nullptr, W, E, top, 1,
                                           static_cast<const float*>(corr), groups, keep, wscale);
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_moe_route(const void* h, const void* rw, const void* rb, const void* gw, void* idx, void* wts, void* gate,
                          int T_, int W, int E, int top, int is_f32, void* stream) {
  if (T_ <= 0) return 0;
  if (E < 1 || E > MAX_E || top < 1 || top > E) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (is_f32)
    route_kernel<float><<<T_, 256, 0, s>>>(static_cast<const float*>(h), static_cast<const float*>(rw), static_cast<const float*>(rb),
                                         static_cast<const float*>(gw), static_cast<int*>(idx), static_cast<float*>(wts),
                                         static_cast<float*>(gate), W, E, top, 0, nullptr, 1, 1, 1.0f);
  else
    route_kernel<bf16_t><<<T_, 256, 0, s>>>(static_cast<const bf16_t*>(h), static_cast<const float*>(rw), static_cast<const float*>(rb),
                                          static_cast<const float*>(gw), static_cast<int*>(idx), static_cast<float*>(wts),
                                          static_cast<float*>(gate), W, E, top, 0, nullptr, 1, 1, 1.0f);
  return BCG_CHECK_LAUNCH();
}

// sorted: [cap] with cap = n_tiles * TM >= n_slots + E (TM - 1); tile_expert: [n_tiles].
BCG_API int bcg_moe_align(const void* idx, int n_slots, int E, void* sorted, int cap, void* tile_expert, int n_tiles,
                          void* stream) {
  if (n_slots <= 0) return 0;
  if (E < 1 || E > MAX_E || cap != n_tiles * TM || cap < n_slots + E * (TM - 1)) return -2;
  align_kernel<<<1, 1024, 0, static_cast<hipStream_t>(stream)>>>(static_cast<const int*>(idx), n_slots, E,
                                                                 static_cast<int*>(sorted), cap,
                                                                 static_cast<int*>(tile_expert), n_tiles);
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_moe_gemm(const void* a, int64_t a_stride, const void* w, void* out, int64_t out_stride, const void* sorted,
                         const void* tile_expert, int n_tiles, int N, int K, int top, int gather, int scatter, int act,
                         int is_f32, void* stream) {
  if (n_tiles <= 0) return 0;
  if (N < 1 || K < 1 || n_tiles > (1 << 24) || (N + TN - 1) / TN > 65535 || (act == 2 && N % 32)) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(n_tiles, (N + TN - 1) / TN);
  const int vec = (K % 4 == 0 && a_stride % 4 == 0) ? 1 : 0;
#define BCG_MOE_GEMM(TYPE, FULL_)                                                                                    \
  moe_gemm_kernel<TYPE, FULL_><<<grid, 256, 0, s>>>(static_cast<const TYPE*>(a), a_stride, static_cast<const TYPE*>(w), \
                                                    static_cast<TYPE*>(out), out_stride, static_cast<const int*>(sorted), \
                                                    static_cast<const int*>(tile_expert), N, K, top, gather, scatter, act, vec)
  const bool full = vec && K % 16 == 0;   // whole, aligned fragments only
  const int esz = is_f32 ? 4 : 2;
  if (K % 32 == 0 && (a_stride * esz) % 16 == 0 && (reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(w)) % 16 == 0) {
    if (static_cast<int64_t>(n_tiles) * grid.y < 512 && (N + 63) / 64 <= 65535) {   // a small step: 64-column workgroups
      const dim3 ngrid(n_tiles, (N + 63) / 64);
      if (is_f32)
        moe_gemm_lds_narrow_kernel<float><<<ngrid, 256, 0, s>>>(static_cast<const float*>(a), a_stride, static_cast<const float*>(w),
                                                               static_cast<float*>(out), out_stride, static_cast<const int*>(sorted),
                                                               static_cast<const int*>(tile_expert), N, K, top, gather, scatter, act);
      else
        moe_gemm_lds_narrow_kernel<bf16_t><<<ngrid, 256, 0, s>>>(static_cast<const bf16_t*>(a), a_stride, static_cast<const bf16_t*>(w),
                                                                static_cast<bf16_t*>(out), out_stride, static_cast<const int*>(sorted),
                                                                static_cast<const int*>(tile_expert), N, K, top, gather, scatter, act);
      return BCG_CHECK_LAUNCH();
    }
    if (is_f32)
      moe_gemm_lds_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(a), a_stride, static_cast<const float*>(w),
                                                     static_cast<float*>(out), out_stride, static_cast<const int*>(sorted),
                                                     static_cast<const int*>(tile_expert), N, K, top, gather, scatter, act);
    else
      moe_gemm_lds_kernel<bf16_t><<<grid, 256, 0, s>>>(static_cast<const bf16_t*>(a), a_stride, static_cast<const bf16_t*>(w),
                                                      static_cast<bf16_t*>(out), out_stride, static_cast<const int*>(sorted),
                                                      static_cast<const int*>(tile_expert), N, K, top, gather, scatter, act);
    return BCG_CHECK_LAUNCH();
  }
  if (is_f32) {
    if (full) BCG_MOE_GEMM(float, true); else BCG_MOE_GEMM(float, false);
  } else {
    if (full) BCG_MOE_GEMM(bf16_t, true); else BCG_MOE_GEMM(bf16_t, false);
  }
#undef BCG_MOE_GEMM
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_moe_combine(const void* y, const void* wts, void* out, int T_, int W, int top, int is_f32, void* stream) {
  if (T_ <= 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (is_f32)
    combine_kernel<float><<<T_, 256, 0, s>>>(static_cast<const float*>(y), static_cast<const float*>(wts), static_cast<float*>(out), W, top);
  else
    combine_kernel<bf16_t><<<T_, 256, 0, s>>>(static_cast<const bf16_t*>(y), static_cast<const float*>(wts), static_cast<float*>(out), W, top);
  return BCG_CHECK_LAUNCH();
}
