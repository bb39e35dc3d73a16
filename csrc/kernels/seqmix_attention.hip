// Multi-map (differential) causal GQA attention over a paged KV cache, fp32 scores and softmax.
//
//   head h, map m:  a_m = softmax(scale q_m K_m^T) V      (every map over the SAME values)
//   o = a_0 - lam a_1   (maps = 2;  maps = 1: a_0),   o <- o / sqrt(mean(o^2) + eps) * out_scale
//
// Cache of one layer run: K [NB, G, BS, maps dim], V [NB, G, vdim, BS] logically.  With `swz`
// (maps dim a multiple of 4) a (page, KV head) slab is stored fragment-major, so that the 64
// lanes of one MFMA operand load read 512 contiguous bytes instead of 64 scattered 8-byte pieces:
//   K slab [maps dim / 4][BS][4]  (4 features of one key, key after key, feature group after group)
//   V slab [BS / 4][vdim][4]      (4 keys of one value feature, feature after feature, key group after group)
// BS is a multiple of 16.
//
// prefill_kernel: a work tile is <= 64 query rows of one sequence (4 waves x 16 rows) for one
// query head.  Per 16 keys a wave computes S^T = K Q^T (keys x queries) with 16 x 16 MFMAs, so
// the C registers of S^T are already the B operand (keys x queries) of O^T = V^T P^T: no
// shuffle between the two products; softmax statistics are per query = per lane column
// (reduced over the 4 lane groups).  K / V^T fragments are read straight from the cache
// (a lane's share of an operand is 4 consecutive elements of one cache row).
//
// The bf16 instance for heads up to 64 / 128 wide takes 32 keys per iteration and prefetches
// the next iteration's K fragments in registers.
//
// decode_mfma_kernel: single-token rows.  The 16 MFMA columns hold the query heads that share
// one KV head (GQA packing), so the cache is read once per KV head; one wave per 128-key split.
// The split size is fixed, so a row's result does not depend on what else is in the batch.
// decode_merge_kernel merges the splits and applies the map combination + head norm.
//
// Optional, for one-map heads: a sliding window (a query at position i sees keys j with
// i - j < window) or a chunk mask (position i sees j <= i of its own chunk, floor(i / chunk) ==
// floor(j / chunk), chunks counted from position 0), and a per-head sink, a learned logit that takes part in the softmax denominator
// only (no key, no value, not scaled).  The key loop starts at the window's (chunk's) first 16-key
// tile; decode splits are counted from the window's (chunk's) first split.
#include <algorithm>

#include "seqmix_common.h"

namespace {

constexpr int SPLIT_KEYS = 128;
constexpr float MAX_FLOOR = -1.0e30f;   // running maxima start finite: a tile may be hidden as a whole
constexpr float LOG2E = 1.4426950408889634f;

struct AttnArgs {
  const void* q;            // [T, H, maps dim]
  const void* k_cache;
  const void* v_cache;
  const int* block_tables;  // [B, max_blocks]
  const int* q_start;       // [B + 1] (prefill)
  const int* seq_lens;      // [B]
  const int* work;          // prefill: tiles [n, 3] {seq, row0, row_end}; decode: items [n, 2] {row, seq} or null
  void* out;                // [T, H vdim]
  float* ws;                // decode partials
  int max_blocks, H, G, maps, dim, vdim, BS, num_blocks, n_splits;
  float scale, lam, head_eps, out_scale;
  int vec_k, vec_v;         // rows of K / V^T are aligned for 4-element vector loads
  int window;               // > 0: keys below position - window + 1 are hidden
  int chunk;                // > 0: keys below position - position % chunk are hidden (chunks count from position 0)
  const float* sink;        // [H] or null
  int swz;                  // fragment-major slabs (see the top of the file)
};

// First key that a query at position `pos` sees: the window's or the chunk's first, else 0.
__device__ __forceinline__ int first_key(const AttnArgs& a, int pos) {
  if (a.window > 0) return max(0, pos - a.window + 1);
  if (a.chunk > 0) return pos - pos % a.chunk;
  return 0;
}

// The key loop shared by both kernels: keys [k_begin, k_last] of one sequence for the 16 query
// columns of a wave (column = a query row of one head, or a query head of one token).
//   limit      per lane: the last key its column may see;  limit_min: the smallest over the wave
//   lo         per lane: the first key its column may see;  lo_max: the largest over the wave
//   KT         16-key tiles per iteration (one softmax update and one rescale per iteration)
//   PF         this iteration's V^T fragments are loaded before its QK^T products and the next
//              iteration's K fragments right after them (loads fly under the MFMAs and the softmax)
//   FULL       whole, aligned fragments only (no branch around any load)
// Everything that does not depend on the lane stays scalar: the page lookup and the slab base go
// to SGPRs, a lane adds a 32-bit offset that is fixed for the whole loop.  Scores are kept in the
// log2 domain (scale * log2 e folded into one multiply, v_exp_f32 directly).
template <typename T, int KC, int VT, int KT, bool PF, bool FULL, int EXACT, int NM>
__device__ __forceinline__ void attend_range(const AttnArgs& a_, int g, const typename Elem<T>::frag (&qf)[NM][KC],
                                             int limit, int limit_min, int lo, int lo_max, int k_begin, int k_last,
                                             const int* __restrict__ table, f32x4 (&acc)[NM][VT], float (&mx)[NM],
                                             float (&den)[NM]) {
  typedef typename Elem<T>::frag F;
  // EXACT (1 or 2 = the number of maps): dim = 16 KC, vdim = 16 VT, 16-token pages, fragment-major slabs -- every guard
  // below is a compile-time constant, fragment offsets are immediates, the loop body is straight-line
  struct Shape {
    const AttnArgs& r;
    int maps, dim, vdim, swz, BS, G, max_blocks, num_blocks, vec_k, vec_v;
    float scale;
    const void *k_cache, *v_cache;
  };
  const Shape a{a_, EXACT ? EXACT : a_.maps, EXACT ? 16 * KC : a_.dim, EXACT ? 16 * VT : a_.vdim, EXACT ? 1 : a_.swz, EXACT ? 16 : a_.BS, a_.G,
                a_.max_blocks, a_.num_blocks, EXACT ? 1 : a_.vec_k, EXACT ? 1 : a_.vec_v, a_.scale, a_.k_cache, a_.v_cache};
  const int lane = threadIdx.x & 63, col = lane & 15, grp = lane >> 4;
  const int KD = a.maps * a.dim;
  const int kc = EXACT ? KC : (a.dim + 15) >> 4, vt = EXACT ? VT : (a.vdim + 15) >> 4;
  const bool vec_k = a.vec_k && (a.dim & 3) == 0;
  const float sc = a.scale * 1.4426950408889634f;
  // offsets inside a (page, KV head) slab = one lane offset (fixed for the whole loop) + a
  // wave-uniform offset per fragment; the slab base and the tile's key offset are uniform too
  const uint32_t k_lane = a.swz ? (grp * a.BS + col) * 4 : col * KD + 4 * grp;
  const uint32_t v_lane = a.swz ? (grp * a.vdim + col) * 4 : col * a.BS + 4 * grp;
  auto k_uni = [&](int m, int c) { return a.swz ? ((m * a.dim + 16 * c) >> 2) * a.BS * 4 : m * a.dim + 16 * c; };
  auto v_uni = [&](int t) { return a.swz ? 16 * t * 4 : 16 * t * a.BS; };
  const int k_mul = a.swz ? 4 : KD, v_mul = a.swz ? a.vdim : 1;   // slab offset per key of the tile's first key
  const T* kc_base = static_cast<const T*>(a.k_cache);
  const T* vc_base = static_cast<const T*>(a.v_cache);
  const size_t k_slab = static_cast<size_t>(a.BS) * KD, v_slab = static_cast<size_t>(a.BS) * a.vdim;

  // A cursor walks the sequence in 16-key tiles: page index + key offset in the page, stepped
  // without a division (BS is a multiple of 16).  Tiles past the sequence read some valid page:
  // every one of their keys is masked.
  struct Cursor { int p, o; };
  auto step = [&](Cursor& c) {
    c.o += 16;
    if (c.o >= a.BS) { c.o = 0; ++c.p; }
  };
  auto slab_base = [&](const Cursor& c) {
    int page = table[min(c.p, a.max_blocks - 1)];
    page = (page < 0 || page >= a.num_blocks) ? 0 : page;
    return static_cast<size_t>(page) * a.G + g;
  };
  auto load_k = [&](Cursor& c, F (&kf)[KT][NM][KC]) {
#pragma unroll
    for (int u = 0; u < KT; ++u) {
      const T* kp = kc_base + slab_base(c) * k_slab + c.o * k_mul;
      step(c);
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int c2 = 0; c2 < KC; ++c2)
          kf[u][m][c2] = (m < a.maps && c2 < kc) ? load_frag_t<T, FULL>(kp + k_uni(m, c2) + k_lane, a.dim - (16 * c2 + 4 * grp), vec_k)
                                                 : zero_frag<T>();
    }
  };

  Cursor k_cur, v_cur;
  k_cur.p = k_begin / a.BS;
  k_cur.o = k_begin - k_cur.p * a.BS;
  v_cur = k_cur;
  F kf[KT][NM][KC];
  if (PF) load_k(k_cur, kf);
  for (int key0 = k_begin; key0 <= k_last; key0 += 16 * KT) {
    const T* vps[KT];
#pragma unroll
    for (int u = 0; u < KT; ++u) {
      vps[u] = vc_base + slab_base(v_cur) * v_slab + v_cur.o * v_mul;
      step(v_cur);
    }
    F vf[PF ? KT : 1][PF ? VT : 1];
    auto load_v = [&](int u, int t) {
      return (t < vt && 16 * t + col < a.vdim) ? load_frag_t<T, FULL>(vps[u] + v_uni(t) + v_lane, 4, a.vec_v) : zero_frag<T>();
    };
    if constexpr (PF) {
#pragma unroll
      for (int u = 0; u < KT; ++u)
#pragma unroll
        for (int t = 0; t < VT; ++t) vf[u][t] = load_v(u, t);
    } else {
      load_k(k_cur, kf);
    }
    // ---- S^T = K Q^T ----
    f32x4 s[KT][NM];
#pragma unroll
    for (int u = 0; u < KT; ++u)
#pragma unroll
      for (int m = 0; m < NM; ++m) {
        s[u][m] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (m < a.maps) {
#pragma unroll
          for (int c = 0; c < KC; ++c)
            if (c < kc) s[u][m] = mma16(kf[u][m][c], qf[m][c], s[u][m]);
        }
      }
    // the K fragments are spent: the next iteration's go into the same registers, under the
    // softmax and the second product
    if (PF && key0 + 16 * KT <= k_last) load_k(k_cur, kf);
    // ---- online softmax per query column; lane holds keys key0 + 16 u + 4 grp + i ----
    const bool masked = key0 + 16 * KT - 1 > limit_min || key0 < lo_max;   // (wave-uniform) some key of the iteration is hidden
    F pf[KT][NM];
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      if (m >= a.maps) {
#pragma unroll
        for (int u = 0; u < KT; ++u) pf[u][m] = zero_frag<T>();
        continue;
      }
      float v[KT][4], bm = -INFINITY;
#pragma unroll
      for (int u = 0; u < KT; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[u][i] = s[u][m][i] * sc;
          if (masked && (key0 + 16 * u + 4 * grp + i > limit || key0 + 16 * u + 4 * grp + i < lo)) v[u][i] = -INFINITY;
          bm = fmaxf(bm, v[u][i]);
        }
      bm = fmaxf(bm, __shfl_xor(bm, 16, WAVE));
      bm = fmaxf(bm, __shfl_xor(bm, 32, WAVE));
      const float m_new = fmaxf(mx[m], bm);                 // finite: the running maximum starts finite
      float ps = 0.f;
#pragma unroll
      for (int u = 0; u < KT; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[u][i] = __builtin_amdgcn_exp2f(v[u][i] - m_new);
          ps += v[u][i];
        }
      ps += __shfl_xor(ps, 16, WAVE);
      ps += __shfl_xor(ps, 32, WAVE);
      if (__any(m_new > mx[m])) {                           // (wave-uniform) the running maximum moved
        const float alpha = __builtin_amdgcn_exp2f(mx[m] - m_new);
        den[m] *= alpha;
#pragma unroll
        for (int t = 0; t < VT; ++t)
          if (t < vt) acc[m][t] *= alpha;
      }
      den[m] += ps;
      mx[m] = m_new;
#pragma unroll
      for (int u = 0; u < KT; ++u) pf[u][m] = Elem<T>::pack(v[u][0], v[u][1], v[u][2], v[u][3]);
    }
    // ---- O^T += V^T P^T ----
#pragma unroll
    for (int u = 0; u < KT; ++u)
#pragma unroll
      for (int t = 0; t < VT; ++t)
        if (t < vt) {
          F x;
          if constexpr (PF) x = vf[u][t]; else x = load_v(u, t);
          acc[0][t] = mma16(x, pf[u][0], acc[0][t]);
          if constexpr (NM > 1) {
            if (a.maps > 1) acc[1][t] = mma16(x, pf[u][1], acc[1][t]);
          }
        }
  }
}

template <typename T, int KC, int VT, int KT, bool PF, bool FULL, int OCC, int EXACT = 0, int NM = 2>
__global__ __launch_bounds__(256, OCC) void prefill_kernel(AttnArgs a) {
  typedef typename Elem<T>::frag F;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = lane & 15, grp = lane >> 4;
  const int h = blockIdx.y, g = h / (a.H / a.G);
  const int seq = a.work[3 * blockIdx.x], row0 = a.work[3 * blockIdx.x + 1] + 16 * wave, row_end = a.work[3 * blockIdx.x + 2];
  if (row0 >= row_end) return;
  const int ctx = a.seq_lens[seq], q_end = a.q_start[seq + 1];
  const int n_rows = min(16, row_end - row0);
  const int row = row0 + min(col, n_rows - 1);             // columns past the tile repeat its last row (never stored)
  const int pos = ctx - (q_end - row);                     // position of this lane's query column
  const int pos_min = ctx - (q_end - row0), pos_max = pos_min + n_rows - 1;
  const int KD = a.maps * a.dim;
  const int kc = (a.dim + 15) >> 4, vt = (a.vdim + 15) >> 4;
  const bool vec_k = a.vec_k && (a.dim & 3) == 0;
  const T* qrow = static_cast<const T*>(a.q) + (static_cast<size_t>(row) * a.H + h) * KD;

  F qf[NM][KC];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const int f = 16 * c + 4 * grp;
      qf[m][c] = (m < a.maps && c < kc) ? load_frag_t<T, FULL>(qrow + m * a.dim + f, a.dim - f, vec_k) : zero_frag<T>();
    }
  f32x4 acc[NM][VT];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int t = 0; t < VT; ++t) acc[m][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  float mx[NM], den[NM];
#pragma unroll
  for (int m = 0; m < NM; ++m) {
    mx[m] = MAX_FLOOR;
    den[m] = 0.f;
  }
  if (a.sink != nullptr) {   // the sink starts the softmax: weight 1 at its own logit
    mx[0] = a.sink[h] * LOG2E;
    den[0] = 1.0f;
  }
  const int lo = first_key(a, pos), lo_max = first_key(a, pos_max);   // (both masks: the first key grows with the position)
  const int k_begin = first_key(a, pos_min) & ~15;
  attend_range<T, KC, VT, KT, PF, FULL, EXACT, NM>(a, g, qf, pos, pos_min, lo, lo_max, k_begin, pos_max,
                                        a.block_tables + static_cast<size_t>(seq) * a.max_blocks, acc, mx, den);
  // ---- combine the maps, unit norm over the head's value features, store ----
  const float i0 = 1.0f / den[0];
  float i1 = 0.f;
  if constexpr (NM > 1) {
    if (a.maps > 1) i1 = a.lam / den[1];
  }
  float ss = 0.f;
#pragma unroll
  for (int t = 0; t < VT; ++t)
    if (t < vt) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float o = acc[0][t][i] * i0;
        if constexpr (NM > 1) {
          if (a.maps > 1) o -= acc[1][t][i] * i1;
        }
        acc[0][t][i] = o;
        ss += o * o;   // rows >= vdim are zero (their V^T fragments were zero)
      }
    }
  ss += __shfl_xor(ss, 16, WAVE);
  ss += __shfl_xor(ss, 32, WAVE);
  const float r = (a.head_eps >= 0.f ? 1.0f / sqrtf(ss / a.vdim + a.head_eps) : 1.0f) * a.out_scale;
  if (col < n_rows) {
    T* orow = static_cast<T*>(a.out) + (static_cast<size_t>(row) * a.H + h) * a.vdim;
#pragma unroll
    for (int t = 0; t < VT; ++t)
      if (t < vt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int e = 16 * t + 4 * grp + i;
          if (e < a.vdim) orow[e] = Elem<T>::st(acc[0][t][i] * r);
        }
      }
  }
}

// Single-token rows, the query heads of one KV head packed into the 16 MFMA columns: column c is
// head g (H / G) + 16 cg + c of the same token, so K and V^T are read once per KV head.  One wave
// per (item, KV head x column group, SPLIT_KEYS-key split); partials as the merge kernel reads them
// (running maxima in the log2 domain of `attend_range`).
template <typename T, int KC, int VT, int KT, bool PF, bool FULL, int OCC, int EXACT = 0, int NM = 2>
__global__ __launch_bounds__(64, OCC) void decode_mfma_kernel(AttnArgs a) {
  typedef typename Elem<T>::frag F;
  const int lane = threadIdx.x, col = lane & 15, grp = lane >> 4;
  const int per = a.H / a.G;
  const int g = blockIdx.x % a.G, cg = blockIdx.x / a.G;
  const int split = blockIdx.y, item = blockIdx.z;
  const int row = a.work ? a.work[2 * item] : item, seq = a.work ? a.work[2 * item + 1] : item;
  const int ctx = a.seq_lens[seq];
  const int lo = first_key(a, ctx - 1);                             // first visible key
  const int split_abs = lo / SPLIT_KEYS + split;                    // splits count from the window's first
  const int k_end = min(ctx, (split_abs + 1) * SPLIT_KEYS);
  const int k_begin = max(split_abs * SPLIT_KEYS, lo & ~15);
  if (k_begin >= k_end) return;
  const bool col_ok = 16 * cg + col < per;
  const int h = g * per + min(16 * cg + col, per - 1);
  const int KD = a.maps * a.dim;
  const int kc = (a.dim + 15) >> 4, vt = (a.vdim + 15) >> 4;
  const bool vec_k = a.vec_k && (a.dim & 3) == 0;
  const T* qrow = static_cast<const T*>(a.q) + (static_cast<size_t>(row) * a.H + h) * KD;
  F qf[NM][KC];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const int f = 16 * c + 4 * grp;
      qf[m][c] = (m < a.maps && c < kc) ? load_frag_t<T, FULL>(qrow + m * a.dim + f, a.dim - f, vec_k) : zero_frag<T>();
    }
  f32x4 acc[NM][VT];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int t = 0; t < VT; ++t) acc[m][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  float mx[NM], den[NM];
#pragma unroll
  for (int m = 0; m < NM; ++m) {
    mx[m] = MAX_FLOOR;
    den[m] = 0.f;
  }
  attend_range<T, KC, VT, KT, PF, FULL, EXACT, NM>(a, g, qf, k_end - 1, k_end - 1, lo, lo, k_begin, k_end - 1,
                                        a.block_tables + static_cast<size_t>(seq) * a.max_blocks, acc, mx, den);
  if (!col_ok) return;
  float* w = a.ws + ((static_cast<size_t>(item) * a.H + h) * a.n_splits + split) * (2 * a.maps + a.maps * a.vdim);
#pragma unroll
  for (int m = 0; m < NM; ++m)
    if (grp == 0 && m < a.maps) {
      w[m] = mx[m];
      w[a.maps + m] = den[m];
    }
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int t = 0; t < VT; ++t)
      if (m < a.maps && t < vt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int e = 16 * t + 4 * grp + i;
          if (e < a.vdim) w[2 * a.maps + m * a.vdim + e] = acc[m][t][i];
        }
      }
}

// ws layout per (item, head, split): [maps] max, [maps] denominator, [maps][vdim] numerators.
template <typename T, int VPL>
__global__ __launch_bounds__(64) void decode_merge_kernel(AttnArgs a) {
  const int lane = threadIdx.x, h = blockIdx.x, item = blockIdx.y;
  const int row = a.work ? a.work[2 * item] : item, seq = a.work ? a.work[2 * item + 1] : item;
  const int ctx = a.seq_lens[seq];
  const int s_first = first_key(a, ctx - 1) / SPLIT_KEYS;
  const int n = min(a.n_splits, (ctx + SPLIT_KEYS - 1) / SPLIT_KEYS - s_first);
  const float sink = a.sink != nullptr ? a.sink[h] * LOG2E : MAX_FLOOR;
  const int stride = 2 * a.maps + a.maps * a.vdim;
  const float* w = a.ws + (static_cast<size_t>(item) * a.H + h) * a.n_splits * stride;
  float o[VPL];
#pragma unroll
  for (int j = 0; j < VPL; ++j) o[j] = 0.f;
  for (int m = 0; m < a.maps; ++m) {
    float mx = m == 0 ? sink : MAX_FLOOR;
    for (int s = 0; s < n; ++s) mx = fmaxf(mx, w[s * stride + m]);
    float den = (m == 0 && a.sink != nullptr) ? exp2f(sink - mx) : 0.f, num[VPL];
#pragma unroll
    for (int j = 0; j < VPL; ++j) num[j] = 0.f;
    for (int s = 0; s < n; ++s) {
      const float f = exp2f(w[s * stride + m] - mx);   // (maxima are kept in the log2 domain)
      den += w[s * stride + a.maps + m] * f;
#pragma unroll
      for (int j = 0; j < VPL; ++j) {
        const int e = lane + 64 * j;
        if (e < a.vdim) num[j] += w[s * stride + 2 * a.maps + m * a.vdim + e] * f;
      }
    }
    const float c = (m == 0 ? 1.0f : -a.lam) / den;
#pragma unroll
    for (int j = 0; j < VPL; ++j) o[j] += num[j] * c;
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < VPL; ++j) ss += (lane + 64 * j < a.vdim) ? o[j] * o[j] : 0.f;
  ss = wave_sum(ss);
  const float r = (a.head_eps >= 0.f ? 1.0f / sqrtf(ss / a.vdim + a.head_eps) : 1.0f) * a.out_scale;
  T* orow = static_cast<T*>(a.out) + (static_cast<size_t>(row) * a.H + h) * a.vdim;
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int e = lane + 64 * j;
    if (e < a.vdim) orow[e] = Elem<T>::st(o[j] * r);
  }
}

template <typename T>
int launch_prefill(const AttnArgs& a, int n_tiles, int tile_rows, hipStream_t s) {
  dim3 grid(n_tiles, a.H);
  const bool small = a.dim <= 64 && a.vdim <= 128;
  const bool full = a.dim % 16 == 0 && a.vdim % 16 == 0 && a.vec_k && a.vec_v;   // whole, aligned fragments only
  if (tile_rows != 64) return -2;
  if constexpr (sizeof(T) == 2) if (full && a.maps == 1 && a.swz && a.BS == 16) {   // one-map heads, exact shapes
#define BCG_EXACT1(KC_, VT_)                                                                     \
  if (a.dim == 16 * KC_ && a.vdim == 16 * VT_) {                                                 \
    prefill_kernel<T, KC_, VT_, 2, true, true, 2, 1, 1><<<grid, 256, 0, s>>>(a);                 \
    return BCG_CHECK_LAUNCH();                                                                   \
  }
    BCG_EXACT1(8, 8) BCG_EXACT1(4, 4) BCG_EXACT1(4, 8) BCG_EXACT1(2, 2) BCG_EXACT1(6, 6) BCG_EXACT1(6, 4) BCG_EXACT1(12, 8)
#undef BCG_EXACT1
  }
  if constexpr (sizeof(T) == 2) if (small) {
    const bool exact = full && a.maps == 2 && a.swz && a.BS == 16;
#define BCG_EXACT(KC_, VT_)                                                                      \
  if (exact && a.dim == 16 * KC_ && a.vdim == 16 * VT_) {                                        \
    prefill_kernel<T, KC_, VT_, 2, true, true, 2, 2><<<grid, 256, 0, s>>>(a);                    \
    return BCG_CHECK_LAUNCH();                                                                   \
  }
    BCG_EXACT(4, 8) BCG_EXACT(3, 6) BCG_EXACT(2, 4) BCG_EXACT(4, 4) BCG_EXACT(2, 2)
#undef BCG_EXACT
    if (full) prefill_kernel<T, 4, 8, 2, true, true, 2><<<grid, 256, 0, s>>>(a);
    else prefill_kernel<T, 4, 8, 2, true, false, 2><<<grid, 256, 0, s>>>(a);
    return BCG_CHECK_LAUNCH();
  }
  if (small) {
    if (full) prefill_kernel<T, 4, 8, 1, false, true, 2><<<grid, 256, 0, s>>>(a);
    else prefill_kernel<T, 4, 8, 1, false, false, 2><<<grid, 256, 0, s>>>(a);
  } else if (a.dim <= 128) {   // (the branch-free form of the wide instance runs out of registers)
    prefill_kernel<T, 8, 16, 1, false, false, 1><<<grid, 256, 0, s>>>(a);
  } else if (a.dim <= 256) {   // one map of up to 256 key features (a latent plus a rotated part)
    prefill_kernel<T, 16, 16, 1, false, false, 1, 0, 1><<<grid, 256, 0, s>>>(a);
  } else {   // ... up to 512 (slow: the fragments of a row fill the register file)
    prefill_kernel<T, 32, 16, 1, false, false, 1, 0, 1><<<grid, 256, 0, s>>>(a);
  }
  return BCG_CHECK_LAUNCH();
}

template <typename T>
int launch_decode(const AttnArgs& a, int n_items, hipStream_t s) {
  const int per = a.H / a.G;
  dim3 grid(a.G * ((per + 15) / 16), a.n_splits, n_items);
  const bool full = a.dim % 16 == 0 && a.vdim % 16 == 0 && a.vec_k && a.vec_v;
  bool done = false;
  if constexpr (sizeof(T) == 2) if (full && a.maps == 1 && a.swz && a.BS == 16) {   // one-map heads, exact shapes
#define BCG_EXACT1(KC_, VT_)                                                                     \
  if (!done && a.dim == 16 * KC_ && a.vdim == 16 * VT_) {                                        \
    done = true;                                                                                 \
    decode_mfma_kernel<T, KC_, VT_, 2, true, true, 2, 1, 1><<<grid, 64, 0, s>>>(a);              \
  }
    BCG_EXACT1(8, 8) BCG_EXACT1(4, 4) BCG_EXACT1(4, 8) BCG_EXACT1(2, 2) BCG_EXACT1(6, 6) BCG_EXACT1(6, 4) BCG_EXACT1(12, 8)
#undef BCG_EXACT1
  }
  if constexpr (sizeof(T) == 2) if (!done && a.dim <= 64 && a.vdim <= 128) {
    done = true;
    const bool exact = full && a.maps == 2 && a.swz && a.BS == 16;
    bool hit = false;
#define BCG_EXACT(KC_, VT_)                                                                      \
  if (!hit && exact && a.dim == 16 * KC_ && a.vdim == 16 * VT_) {                                \
    hit = true;                                                                                  \
    decode_mfma_kernel<T, KC_, VT_, 2, true, true, 2, 2><<<grid, 64, 0, s>>>(a);                 \
  }
    BCG_EXACT(4, 8) BCG_EXACT(3, 6) BCG_EXACT(2, 4) BCG_EXACT(4, 4) BCG_EXACT(2, 2)
#undef BCG_EXACT
    if (hit) {
    } else
    if (full) decode_mfma_kernel<T, 4, 8, 2, true, true, 2><<<grid, 64, 0, s>>>(a);
    else decode_mfma_kernel<T, 4, 8, 2, true, false, 2><<<grid, 64, 0, s>>>(a);
  }
  if (done) {
  } else if (a.dim <= 64 && a.vdim <= 128) {
    if (full) decode_mfma_kernel<T, 4, 8, 1, false, true, 2><<<grid, 64, 0, s>>>(a);
    else decode_mfma_kernel<T, 4, 8, 1, false, false, 2><<<grid, 64, 0, s>>>(a);
  } else if (a.dim <= 128) {
    decode_mfma_kernel<T, 8, 16, 1, false, false, 1><<<grid, 64, 0, s>>>(a);
  } else if (a.dim <= 256) {
    decode_mfma_kernel<T, 16, 16, 1, false, false, 1, 0, 1><<<grid, 64, 0, s>>>(a);
  } else {
    decode_mfma_kernel<T, 32, 16, 1, false, false, 1, 0, 1><<<grid, 64, 0, s>>>(a);
  }
  if (a.vdim <= 128) decode_merge_kernel<T, 2><<<dim3(a.H, n_items), 64, 0, s>>>(a);
  else decode_merge_kernel<T, 4><<<dim3(a.H, n_items), 64, 0, s>>>(a);
  return BCG_CHECK_LAUNCH();
}

}  // namespace

BCG_API int bcg_multimap_split_keys() { return SPLIT_KEYS; }

// mode 0: prefill tiles (work = tiles [n_work, 3]); mode 1: single-token items (work = [n_work, 2]
// {row, sequence}, or null: item i is row i of sequence i).
BCG_API int bcg_multimap_attention(int mode, const void* q, const void* k_cache, const void* v_cache,
                                   const void* block_tables, int max_blocks, const void* q_start, const void* seq_lens,
                                   const void* work, int n_work, void* out, void* ws, int n_splits, int H, int G, int maps,
                                   int dim, int vdim, int BS, int num_blocks, float scale, float lam, float head_eps,
                                   float out_scale, int tile_rows, int is_f32, int window, int chunk, const void* sink,
                                   void* stream) {
  if (n_work <= 0) return 0;
  if ((window > 0 || chunk > 0 || sink != nullptr) && maps != 1) return -2;
  if (window > 0 && chunk > 0) return -2;
  if (maps < 1 || maps > 2 || dim > (maps == 1 ? 512 : 128) || vdim > 256 || BS % 16 || H % G || n_work > 65535 * 16) return -2;
  AttnArgs a;
  a.q = q; a.k_cache = k_cache; a.v_cache = v_cache;
  a.block_tables = static_cast<const int*>(block_tables); a.q_start = static_cast<const int*>(q_start);
  a.seq_lens = static_cast<const int*>(seq_lens); a.work = static_cast<const int*>(work);
  a.out = out; a.ws = static_cast<float*>(ws);
  a.max_blocks = max_blocks; a.H = H; a.G = G; a.maps = maps; a.dim = dim; a.vdim = vdim; a.BS = BS;
  a.num_blocks = num_blocks; a.n_splits = n_splits;
  a.scale = scale; a.lam = lam; a.head_eps = head_eps; a.out_scale = out_scale;
  a.vec_k = ((maps * dim) % 4 == 0) ? 1 : 0;
  a.vec_v = 1;  // BS % 16 == 0: every 4-key group of a V^T row is aligned
  a.swz = a.vec_k;
  a.window = window; a.chunk = chunk; a.sink = static_cast<const float*>(sink);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (mode == 0) return is_f32 ? launch_prefill<float>(a, n_work, tile_rows, s) : launch_prefill<bf16_t>(a, n_work, tile_rows, s);
  if (n_splits < 1 || H > 65535 || n_splits > 65535 || n_work > 65535) return -2;
  return is_f32 ? launch_decode<float>(a, n_work, s) : launch_decode<bf16_t>(a, n_work, s);
}
