// Hyper-connection residual streams with layer norms, the rotary / unit-norm / value-mix cache
// write of a softmax mixer, the gates of a matrix memory with exponential gating, and a logit cap.
//
//   streams        X [T, S, W] fp32 instead of one residual row.  A sublayer reads u = sum_s r[s] X[s],
//                  and its output y is written back as X'[t] = sum_s M[s, t] X[s] + o[t] y (all
//                  streams from the old ones).  S = 1 with r = M = o = 1 is the plain residual sum.
//   layer norm     (u - mean) / sqrt(var + eps) * w, biased variance, two passes over the row
//   cache write    rotate-half rotary on the first 2 half features of every q / k head, then the
//                  head divided by its root mean square (no weight); values blended with the values
//                  that an earlier layer computed for the same token, v' = (1 - lam) v + lam v0
//   matrix memory  log gates i = c tanh((z_i + b_i) / c), f = logsigmoid(c tanh((z_f + b_f) / c)), the
//                  running maximum m_t = max(f_t + m_(t-1), i_t) carried per (sequence, head), and from
//                  it the decay exp(f_t + m_(t-1) - m_t), the write scale exp(i_t - m_t) and the
//                  floor exp(-m_t) of the output's denominator
//
// T is the activation type (bf16 bits or float); streams, norms, angles, gates are fp32.
#include <algorithm>

#include "seqmix_common.h"

namespace {

constexpr int NT = 256;
constexpr int MAX_STREAMS = 16;

__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[w] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NT / 64; ++i) t += red[i];
  return t;
}

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float log_sigmoidf_(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// V consecutive elements (V = 4: one 16-byte or 8-byte access, the caller checked the alignment).
template <typename T, int V> struct Pack;
template <typename T> struct Pack<T, 1> {
  typedef float vec;
  static __device__ __forceinline__ float ld(const T* p) { return Elem<T>::ld(*p); }
  static __device__ __forceinline__ void st(T* p, float v) { *p = Elem<T>::st(v); }
  static __device__ __forceinline__ float get(float v, int) { return v; }
  static __device__ __forceinline__ void set(float& v, int, float x) { v = x; }
};
template <> struct Pack<float, 4> {
  typedef f32x4 vec;
  static __device__ __forceinline__ f32x4 ld(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
  static __device__ __forceinline__ void st(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
  static __device__ __forceinline__ float get(const f32x4& v, int j) { return v[j]; }
  static __device__ __forceinline__ void set(f32x4& v, int j, float x) { v[j] = x; }
};
template <> struct Pack<bf16_t, 4> {
  typedef f32x4 vec;
  static __device__ __forceinline__ f32x4 ld(const bf16_t* p) {
    const u16x4 r = *reinterpret_cast<const u16x4*>(p);
    return f32x4{bf2f(r[0]), bf2f(r[1]), bf2f(r[2]), bf2f(r[3])};
  }
  static __device__ __forceinline__ void st(bf16_t* p, f32x4 v) {
    *reinterpret_cast<u16x4*>(p) = u16x4{f2bf(v[0]), f2bf(v[1]), f2bf(v[2]), f2bf(v[3])};
  }
  static __device__ __forceinline__ float get(const f32x4& v, int j) { return v[j]; }
  static __device__ __forceinline__ void set(f32x4& v, int j, float x) { v[j] = x; }
};

// Layer norm of the row staged in `u` (LDS, W floats, element i written by the thread that reads it).
template <typename T, int V>
__device__ __forceinline__ void layer_norm_row(const float* u, float part_sum, const float* __restrict__ w, float eps,
                                               T* __restrict__ out, int W, float* red) {
  typedef Pack<float, V> PF;
  const float mean = block_sum(part_sum, red) / W;
  float sq = 0.f;
  for (int i = V * threadIdx.x; i < W; i += V * NT) {
    const typename PF::vec x = PF::ld(u + i);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float d = PF::get(x, j) - mean;
      sq += d * d;
    }
  }
  const float r = 1.0f / sqrtf(block_sum(sq, red) / W + eps);
  for (int i = V * threadIdx.x; i < W; i += V * NT) {
    const typename PF::vec x = PF::ld(u + i), g = PF::ld(w + i);
    typename PF::vec o;
#pragma unroll
    for (int j = 0; j < V; ++j) PF::set(o, j, (PF::get(x, j) - mean) * r * PF::get(g, j));
    Pack<T, V>::st(out + i, o);
  }
}

// X[t, s, :] = table[token] for every stream; h = layer_norm(sum_s r[s] X[s]).
template <typename T>
__global__ __launch_bounds__(NT) void hyper_embed_norm_kernel(const int* __restrict__ tokens, const T* __restrict__ table,
                                                              const float* __restrict__ read_w,
                                                              const float* __restrict__ norm_w, float eps,
                                                              float* __restrict__ X, T* __restrict__ h, int S, int W,
                                                              int vocab) {
  extern __shared__ float u[];
  __shared__ float red[NT / 64];
  const int t = blockIdx.x;
  int tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  const T* row = table + static_cast<size_t>(tok) * W;
  float* x = X + static_cast<size_t>(t) * S * W;
  float sum = 0.f;
  for (int i = threadIdx.x; i < W; i += NT) {
    const float v = Elem<T>::ld(row[i]);
    float acc = 0.f;
    for (int s = 0; s < S; ++s) {
      x[static_cast<size_t>(s) * W + i] = v;
      acc += read_w[s] * v;
    }
    u[i] = acc;
    sum += acc;
  }
  layer_norm_row<T, 1>(u, sum, norm_w, eps, h + static_cast<size_t>(t) * W, W, red);
}

// X'[t] = sum_s mix[s, t] X[s] + out_w[t] (y0 + y1) in place (mix null: X stays), then
// h = layer_norm(sum_s read_w[s] X'[s]) (read_w null: no read).  SM >= S is the unrolled stream count,
// V the columns per thread and access (4 when the width is a multiple of 4).
template <typename T, int SM, int V>
__global__ __launch_bounds__(NT) void hyper_update_norm_kernel(float* __restrict__ X, const T* __restrict__ y0,
                                                               const float* __restrict__ y1,
                                                               const float* __restrict__ mix,
                                                               const float* __restrict__ out_w,
                                                               const float* __restrict__ read_w,
                                                               const float* __restrict__ norm_w, float eps,
                                                               T* __restrict__ h, int S, int W) {
  extern __shared__ __attribute__((aligned(16))) float u[];
  __shared__ float red[NT / 64];
  __shared__ float cm[MAX_STREAMS * MAX_STREAMS], co[MAX_STREAMS], cr[MAX_STREAMS];
  typedef Pack<float, V> PF;
  typedef typename PF::vec vec;
  if (threadIdx.x < S * S) cm[threadIdx.x] = mix != nullptr ? mix[threadIdx.x] : 0.f;
  if (threadIdx.x < S) {
    co[threadIdx.x] = out_w != nullptr ? out_w[threadIdx.x] : 0.f;
    cr[threadIdx.x] = read_w != nullptr ? read_w[threadIdx.x] : 0.f;
  }
  __syncthreads();
  const size_t t = blockIdx.x;
  float* x = X + t * S * W;
  float sum = 0.f;
  for (int i = V * threadIdx.x; i < W; i += V * NT) {
    vec xs[SM], ya, yb, acc;
#pragma unroll
    for (int s = 0; s < SM; ++s)
      if (s < S) xs[s] = PF::ld(x + static_cast<size_t>(s) * W + i);
    if (y0 != nullptr) ya = Pack<T, V>::ld(y0 + t * W + i);
    if (y1 != nullptr) yb = PF::ld(y1 + t * W + i);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      float y = 0.f;
      if (y0 != nullptr) y += PF::get(ya, j);
      if (y1 != nullptr) y += PF::get(yb, j);
      PF::set(ya, j, y);
      PF::set(acc, j, 0.f);
    }
#pragma unroll
    for (int d = 0; d < SM; ++d)
      if (d < S) {
        vec v = xs[d];
        if (mix != nullptr) {
#pragma unroll
          for (int j = 0; j < V; ++j) {
            float e = co[d] * PF::get(ya, j);
#pragma unroll
            for (int s = 0; s < SM; ++s)
              if (s < S) e += cm[s * S + d] * PF::get(xs[s], j);
            PF::set(v, j, e);
          }
          PF::st(x + static_cast<size_t>(d) * W + i, v);
        }
#pragma unroll
        for (int j = 0; j < V; ++j) PF::set(acc, j, PF::get(acc, j) + cr[d] * PF::get(v, j));
      }
    PF::st(u + i, acc);
#pragma unroll
    for (int j = 0; j < V; ++j) sum += PF::get(acc, j);
  }
  if (read_w != nullptr) layer_norm_row<T, V>(u, sum, norm_w, eps, h + t * W, W, red);
}

// One workgroup per token, a wave per q / k head: rotary on the first 2 half features (feature i
// pairs with i + half), the head over its root mean square (qk_eps < 0: none), q to q_out and k
// into the paged K slab; then the values, blended with v_first when given, into the V^T slab
// (slab layouts: seqmix_attention.hip).  EPL = ceil(dim / 64) elements per lane.
template <typename T, int EPL>
__global__ __launch_bounds__(NT) void rope_norm_kv_kernel(const T* __restrict__ qkv, int64_t row_stride,
                                                          const int* __restrict__ positions, const int* __restrict__ slots,
                                                          const float* __restrict__ inv_freq, int half, float qk_eps,
                                                          const T* __restrict__ v_first, int64_t vf_stride, float lam,
                                                          T* __restrict__ q_out, T* __restrict__ k_cache,
                                                          T* __restrict__ v_cache, int n_q, int n_kv, int dim, int vdim,
                                                          int BS, int num_blocks) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* row = qkv + static_cast<size_t>(t) * row_stride;
  const float pos = static_cast<float>(positions[t]);
  const int slot = slots[t];
  const int blk = slot / BS, off = slot - blk * BS;
  const bool kv_ok = slot >= 0 && blk < num_blocks;
  const bool swz = (dim & 3) == 0;
  for (int hh = wave; hh < n_q + n_kv; hh += NT / 64) {
    const T* head = row + static_cast<size_t>(hh) * dim;
    float val[EPL], ss = 0.f;
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
      const int i = lane + 64 * j;
      val[j] = 0.f;
      if (i < dim) {
        float v = Elem<T>::ld(head[i]);
        if (i < 2 * half) {
          const bool lo = i < half;
          const float other = Elem<T>::ld(head[lo ? i + half : i - half]);
          float s, c;
          sincosf(pos * inv_freq[lo ? i : i - half], &s, &c);
          v = lo ? v * c - other * s : v * c + other * s;
        }
        val[j] = v;
        ss += v * v;
      }
    }
    const float r = qk_eps >= 0.f ? 1.0f / sqrtf(wave_sum(ss) / dim + qk_eps) : 1.0f;
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
      const int i = lane + 64 * j;
      if (i >= dim) continue;
      const T o = Elem<T>::st(val[j] * r);
      if (hh < n_q) {
        q_out[(static_cast<size_t>(t) * n_q + hh) * dim + i] = o;
      } else if (kv_ok) {
        T* slab = k_cache + (static_cast<size_t>(blk) * n_kv + (hh - n_q)) * BS * dim;
        if (swz) slab[(static_cast<size_t>(i >> 2) * BS + off) * 4 + (i & 3)] = o;
        else slab[static_cast<size_t>(off) * dim + i] = o;
      }
    }
  }
  if (!kv_ok) return;
  const int vw = n_kv * vdim;
  const T* vrow = row + static_cast<size_t>(n_q + n_kv) * dim;
  for (int idx = threadIdx.x; idx < vw; idx += NT) {
    const int g = idx / vdim, e = idx - g * vdim;
    T o = vrow[idx];
    if (v_first != nullptr)
      o = Elem<T>::st((1.0f - lam) * Elem<T>::ld(o) + lam * Elem<T>::ld(v_first[static_cast<size_t>(t) * vf_stride + idx]));
    T* slab = v_cache + (static_cast<size_t>(blk) * n_kv + g) * vdim * BS;
    if (swz) slab[(static_cast<size_t>(off >> 2) * vdim + e) * 4 + (off & 3)] = o;
    else slab[static_cast<size_t>(e) * BS + off] = o;
  }
}

// One workgroup per token: fp32 copies q32 = q_scale * y[off_q + .] and k32 = y[off_k + .] of two
// column blocks of n features, and per head the log gates i = cap tanh((y_i + b_i) / cap) (into
// `write`) and f = logsigmoid(cap tanh((y_f + b_f) / cap)) (into `decay`).
template <typename T>
__global__ __launch_bounds__(NT) void gate_rows_kernel(const T* __restrict__ y, int64_t stride, int off_q, int off_k, int off_i,
                                                       int off_f, int n, float q_scale, const float* __restrict__ i_bias,
                                                       const float* __restrict__ f_bias, float cap,
                                                       float* __restrict__ q32, float* __restrict__ k32,
                                                       float* __restrict__ decay, float* __restrict__ write, int H) {
  const size_t t = blockIdx.x;
  const T* row = y + t * stride;
  for (int c = threadIdx.x; c < n; c += NT) {
    q32[t * n + c] = Elem<T>::ld(row[off_q + c]) * q_scale;
    k32[t * n + c] = Elem<T>::ld(row[off_k + c]);
  }
  const float inv = 1.0f / cap;
  for (int h = threadIdx.x; h < H; h += NT) {
    write[t * H + h] = cap * tanhf((Elem<T>::ld(row[off_i + h]) + i_bias[h]) * inv);
    decay[t * H + h] = log_sigmoidf_(cap * tanhf((Elem<T>::ld(row[off_f + h]) + f_bias[h]) * inv));
  }
}

constexpr int GATE_TILE = 4096;   // (token, head) pairs of a segment staged in LDS at a time

// One workgroup per segment.  A tile of GATE_TILE / H tokens at a time: the workgroup stages the log
// gates that `gate_rows_kernel` left in `write` (i) and `decay` (f) in LDS (coalesced loads); thread
// h then walks the tile's tokens for head h, the running maximum m_t = max(f_t + m_(t-1), i_t) being
// a chain of one add and one max per token, and leaves the logarithms f_t + m_(t-1) - m_t, i_t - m_t
// and -m_t in LDS; every thread exponentiates them on the way out (decay, write scale, floor of the
// denominator).  The chain is the same token by token
// whatever the segment's length, so a sequence's gates do not depend on how it was cut.
// m_state [n_rows, H] is read unless the segment starts at position 0.
__global__ __launch_bounds__(NT) void gate_chain_kernel(const int* __restrict__ positions,
                                                        const int* __restrict__ q_start, const int* __restrict__ state_rows,
                                                        float* __restrict__ m_state, int n_rows, float* __restrict__ decay,
                                                        float* __restrict__ write, float* __restrict__ floor_, int H) {
  __shared__ float li[GATE_TILE], lf[GATE_TILE], lm[GATE_TILE];
  const int b = blockIdx.x, tid = threadIdx.x;
  const int t0 = q_start[b], t1 = q_start[b + 1];
  const int sr = state_rows[b];
  if (t1 <= t0 || sr < 0 || sr >= n_rows) return;   // (the same for the whole workgroup)
  const int tile = GATE_TILE / H;                  // tokens per tile
  float m = 0.f;
  if (tid < H && positions[t0] != 0) m = m_state[static_cast<size_t>(sr) * H + tid];
  for (int first = t0; first < t1; first += tile) {
    const int nt = min(tile, t1 - first), ne = nt * H;
    const size_t base = static_cast<size_t>(first) * H;
    for (int e = tid; e < ne; e += NT) {
      li[e] = write[base + e];
      lf[e] = decay[base + e];
    }
    __syncthreads();
    if (tid < H) {
      constexpr int CH = 16;   // tokens read from LDS before their chain runs: the reads' latency is paid once per CH
      for (int tt0 = 0; tt0 < nt; tt0 += CH) {
        float gi[CH], gf[CH], mm[CH + 1];
#pragma unroll
        for (int j = 0; j < CH; ++j) {
          const int e = min(tt0 + j, nt - 1) * H + tid;
          gi[j] = li[e];
          gf[j] = lf[e];
        }
        mm[0] = m;
#pragma unroll
        for (int j = 0; j < CH; ++j) mm[j + 1] = fmaxf(gf[j] + mm[j], gi[j]);
#pragma unroll
        for (int j = 0; j < CH; ++j)
          if (tt0 + j < nt) {
            const int e = (tt0 + j) * H + tid;
            lf[e] = gf[j] + mm[j] - mm[j + 1];
            li[e] = gi[j] - mm[j + 1];
            lm[e] = -mm[j + 1];
            m = mm[j + 1];
          }
      }
    }
    __syncthreads();
    for (int e = tid; e < ne; e += NT) {
      decay[base + e] = expf(lf[e]);
      write[base + e] = expf(li[e]);
      floor_[base + e] = expf(lm[e]);
    }
    __syncthreads();
  }
  if (tid < H) m_state[static_cast<size_t>(sr) * H + tid] = m;
}

// x <- cap tanh(x / cap) over fp32 logits.
__global__ __launch_bounds__(NT) void softcap_kernel(float* __restrict__ x, int64_t total, float cap) {
  const float inv = 1.0f / cap;
  for (int64_t e = static_cast<int64_t>(blockIdx.x) * NT + threadIdx.x; e < total; e += static_cast<int64_t>(gridDim.x) * NT)
    x[e] = cap * tanhf(x[e] * inv);
}

inline int ew_grid(int64_t total) { return static_cast<int>(std::min<int64_t>((total + NT - 1) / NT, 65536)); }

template <typename T>
int launch_update(float* X, const T* y0, const float* y1, const float* mix, const float* ow, const float* rw, const float* nw,
                  float eps, T* h, int T_, int S, int W, hipStream_t s) {
  const size_t lds = static_cast<size_t>(W) * sizeof(float);
#define BCG_UPDATE(SM_)                                                                                        \
  do {                                                                                                         \
    if (W % 4 == 0) hyper_update_norm_kernel<T, SM_, 4><<<T_, NT, lds, s>>>(X, y0, y1, mix, ow, rw, nw, eps, h, S, W); \
    else hyper_update_norm_kernel<T, SM_, 1><<<T_, NT, lds, s>>>(X, y0, y1, mix, ow, rw, nw, eps, h, S, W);     \
  } while (0)
  if (S == 1) BCG_UPDATE(1);
  else if (S == 2) BCG_UPDATE(2);
  else if (S <= 4) BCG_UPDATE(4);
  else if (S <= 8) BCG_UPDATE(8);
  else BCG_UPDATE(16);
#undef BCG_UPDATE
  return BCG_CHECK_LAUNCH();
}

template <typename T>
int launch_rope_norm(const T* qkv, int64_t stride, const int* pos, const int* slots, const float* inv_freq, int half,
                     float qk_eps, const T* v_first, int64_t vf_stride, float lam, T* q_out, T* kc, T* vc, int T_, int n_q,
                     int n_kv, int dim, int vdim, int BS, int NB, hipStream_t s) {
#define BCG_ROPE_NORM(E_)                                                                                             \
  rope_norm_kv_kernel<T, E_><<<T_, NT, 0, s>>>(qkv, stride, pos, slots, inv_freq, half, qk_eps, v_first, vf_stride, lam, \
                                               q_out, kc, vc, n_q, n_kv, dim, vdim, BS, NB)
  if (dim <= 64) BCG_ROPE_NORM(1);
  else if (dim <= 128) BCG_ROPE_NORM(2);
  else if (dim <= 256) BCG_ROPE_NORM(4);
  else BCG_ROPE_NORM(8);
#undef BCG_ROPE_NORM
  return BCG_CHECK_LAUNCH();
}

}  // namespace

#define BCG_BY_TYPE(CALL_F32, CALL_BF16) do { if (is_f32) { CALL_F32; } else { CALL_BF16; } } while (0)

constexpr int MAX_NORM_WIDTH = 12288;   // the normed row is staged in LDS (48 KB)

BCG_API int bcg_hyper_embed_norm(const void* tokens, const void* table, const void* read_w, const void* norm_w, float eps,
                                 void* X, void* h, int T_, int S, int W, int vocab, int is_f32, void* stream) {
  if (T_ <= 0) return 0;
  if (S < 1 || S > MAX_STREAMS || W < 1 || W > MAX_NORM_WIDTH) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t lds = static_cast<size_t>(W) * sizeof(float);
  const int* tk = static_cast<const int*>(tokens);
  const float *rw = static_cast<const float*>(read_w), *nw = static_cast<const float*>(norm_w);
  BCG_BY_TYPE((hyper_embed_norm_kernel<float><<<T_, NT, lds, s>>>(tk, static_cast<const float*>(table), rw, nw, eps,
                                                                 static_cast<float*>(X), static_cast<float*>(h), S, W, vocab)),
              (hyper_embed_norm_kernel<bf16_t><<<T_, NT, lds, s>>>(tk, static_cast<const bf16_t*>(table), rw, nw, eps,
                                                                  static_cast<float*>(X), static_cast<bf16_t*>(h), S, W, vocab)));
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_hyper_update_norm(void* X, const void* y0, const void* y1, const void* mix, const void* out_w,
                                  const void* read_w, const void* norm_w, float eps, void* h, int T_, int S, int W, int is_f32,
                                  void* stream) {
  if (T_ <= 0) return 0;
  if (S < 1 || S > MAX_STREAMS || W < 1 || W > MAX_NORM_WIDTH) return -2;
  if ((mix == nullptr) != (out_w == nullptr) || (read_w != nullptr && (norm_w == nullptr || h == nullptr))) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* x = static_cast<float*>(X);
  const float *f1 = static_cast<const float*>(y1), *mx = static_cast<const float*>(mix), *ow = static_cast<const float*>(out_w),
              *rw = static_cast<const float*>(read_w), *nw = static_cast<const float*>(norm_w);
  if (is_f32) return launch_update<float>(x, static_cast<const float*>(y0), f1, mx, ow, rw, nw, eps, static_cast<float*>(h), T_, S, W, s);
  return launch_update<bf16_t>(x, static_cast<const bf16_t*>(y0), f1, mx, ow, rw, nw, eps, static_cast<bf16_t*>(h), T_, S, W, s);
}

BCG_API int bcg_rope_norm_kv_write(const void* qkv, int64_t row_stride, const void* positions, const void* slots,
                                   const void* inv_freq, int half, float qk_eps, const void* v_first, int64_t vf_stride,
                                   float lam, void* q_out, void* k_cache, void* v_cache, int T_, int n_q, int n_kv, int dim,
                                   int vdim, int BS, int num_blocks, int is_f32, void* stream) {
  if (T_ <= 0) return 0;
  if (dim < 1 || dim > 512 || 2 * half > dim || BS < 1) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int *ps = static_cast<const int*>(positions), *sl = static_cast<const int*>(slots);
  const float* fr = static_cast<const float*>(inv_freq);
  if (is_f32)
    return launch_rope_norm<float>(static_cast<const float*>(qkv), row_stride, ps, sl, fr, half, qk_eps,
                                   static_cast<const float*>(v_first), vf_stride, lam, static_cast<float*>(q_out),
                                   static_cast<float*>(k_cache), static_cast<float*>(v_cache), T_, n_q, n_kv, dim, vdim, BS,
                                   num_blocks, s);
  return launch_rope_norm<bf16_t>(static_cast<const bf16_t*>(qkv), row_stride, ps, sl, fr, half, qk_eps,
                                  static_cast<const bf16_t*>(v_first), vf_stride, lam, static_cast<bf16_t*>(q_out),
                                  static_cast<bf16_t*>(k_cache), static_cast<bf16_t*>(v_cache), T_, n_q, n_kv, dim, vdim, BS,
                                  num_blocks, s);
}

// fp32 q (scaled) and k copies and the log gates per token; then per segment the running maximum of
// every head and the exponentials.
BCG_API int bcg_exp_gate_prepare(const void* y, int64_t stride, int off_q, int off_k, int off_i, int off_f, const void* i_bias,
                                 const void* f_bias, float cap, float q_scale, const void* positions, const void* q_start,
                                 const void* state_rows, void* m_state, int n_rows, void* q32, void* k32, void* decay,
                                 void* write, void* floor_, int T_, int B, int H, int dim, int is_f32, void* stream) {
  if (T_ <= 0 || B <= 0) return 0;
  if (H < 1 || H > NT || !(cap > 0.f)) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int n = H * dim;
  const float *bi = static_cast<const float*>(i_bias), *bf = static_cast<const float*>(f_bias);
  const int *ps = static_cast<const int*>(positions), *qs = static_cast<const int*>(q_start), *sr = static_cast<const int*>(state_rows);
  float *q = static_cast<float*>(q32), *k = static_cast<float*>(k32), *m = static_cast<float*>(m_state),
        *dc = static_cast<float*>(decay), *wr = static_cast<float*>(write), *fl = static_cast<float*>(floor_);
  BCG_BY_TYPE((gate_rows_kernel<float><<<T_, NT, 0, s>>>(static_cast<const float*>(y), stride, off_q, off_k, off_i, off_f, n, q_scale, bi, bf,
                                                        cap, q, k, dc, wr, H)),
              (gate_rows_kernel<bf16_t><<<T_, NT, 0, s>>>(static_cast<const bf16_t*>(y), stride, off_q, off_k, off_i, off_f, n, q_scale, bi,
                                                         bf, cap, q, k, dc, wr, H)));
  gate_chain_kernel<<<B, NT, 0, s>>>(ps, qs, sr, m, n_rows, dc, wr, fl, H);
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_softcap(void* x, int64_t total, float cap, void* stream) {
  if (total <= 0) return 0;
  if (!(cap > 0.f)) return -2;
  softcap_kernel<<<ew_grid(total), NT, 0, static_cast<hipStream_t>(stream)>>>(static_cast<float*>(x), total, cap);
  return BCG_CHECK_LAUNCH();
}
