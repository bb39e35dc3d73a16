// Mixers with per-sequence state on the fp32 residual stream: hashed-bigram embedding, scalar-gain
// norms fused with the residual update, short causal convolutions that continue from a state
// row, pair rotary with whole-projection norms and rotated values, and the gated-state
// recurrence (HGRN2 / gated delta rule) with its preparation and head-norm kernels.
//
// A packed step holds B segments: segment b is rows q_start[b] .. q_start[b + 1] - 1 (consecutive
// positions of one sequence), token_seq[t] is the segment of row t, state_rows[b] the row of the
// state tables that the segment continues.  A segment that starts at position 0 starts from
// empty state whatever the row holds.  State that rows of a segment read is written by a
// second launch, after every reader has finished.
//
// T is the activation type (bf16 bits or float); everything that the recurrences and norms
// compute is fp32.
#include <algorithm>

#include "seqmix_common.h"

namespace {

constexpr int NT = 256;
constexpr int MAX_TAPS = 16;
constexpr int SCAN_CHUNK_ELEMS = 512;   // rows x tokens of a recurrence staged through LDS at a time
constexpr int SCAN_WAVES = 4;   // waves of a recurrence workgroup (8 value columns each)   // tokens of a recurrence staged through LDS at a time

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

// ---------------------------------------------------------------- embedding + hashed bigram + scalar norms
template <typename T>
__global__ __launch_bounds__(NT) void embed_bigram_kernel(const int* __restrict__ tokens, const int* __restrict__ positions,
                                                          const int* __restrict__ token_seq, const int* __restrict__ q_start,
                                                          const int* __restrict__ state_rows, const int* __restrict__ prev,
                                                          int n_rows, const T* __restrict__ table, float scale,
                                                          const T* __restrict__ bigram, int buckets, int mul_prev, int mul_cur,
                                                          float eps, float g1, float g2, float* __restrict__ resid,
                                                          T* __restrict__ out1, T* __restrict__ out2, int W, int vocab) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x;
  int tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  const T* row = table + static_cast<size_t>(tok) * W;
  const T* brow = nullptr;
  if (bigram != nullptr) {
    int64_t r = buckets;                                   // position 0: the table's last row
    if (positions[t] != 0) {
      const int seg = token_seq[t];
      int before;
      if (t > q_start[seg]) {
        before = tokens[t - 1];
      } else {
        const int sr = state_rows[seg];
        before = (sr >= 0 && sr < n_rows) ? prev[sr] : 0;
      }
      r = (static_cast<int64_t>(before) * mul_prev + static_cast<int64_t>(tok) * mul_cur) % buckets;
      if (r < 0) r += buckets;
    }
    brow = bigram + static_cast<size_t>(r) * W;
  }
  float* x = resid + static_cast<size_t>(t) * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += NT) {
    float v = Elem<T>::ld(row[i]) * scale;
    if (brow != nullptr) v += Elem<T>::ld(brow[i]);
    x[i] = v;
    ss += v * v;
  }
  const float r = 1.0f / sqrtf(block_sum(ss, red) / W + eps);
  T* o1 = out1 + static_cast<size_t>(t) * W;
  T* o2 = out2 != nullptr ? out2 + static_cast<size_t>(t) * W : nullptr;
  for (int i = threadIdx.x; i < W; i += NT) {
    const float u = x[i] * r;
    o1[i] = Elem<T>::st(u * g1);
    if (o2 != nullptr) o2[i] = Elem<T>::st(u * g2);
  }
}

__global__ void last_token_kernel(const int* __restrict__ tokens, const int* __restrict__ q_start,
                                  const int* __restrict__ state_rows, int* __restrict__ prev, int n_rows, int B) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  const int sr = state_rows[b], e = q_start[b + 1];
  if (e > q_start[b] && sr >= 0 && sr < n_rows) prev[sr] = tokens[e - 1];
}

// x += mult (nscale (rms(a) wa + rms(b) wb) + p0 + p1);  out1 = x / rms(x) g1, out2 = ... g2.
template <typename T>
__global__ __launch_bounds__(NT) void residual_mix_norm_kernel(float* __restrict__ resid, const T* __restrict__ a,
                                                               const float* __restrict__ wa, const T* __restrict__ b,
                                                               const float* __restrict__ wb, const T* __restrict__ p0,
                                                               const T* __restrict__ p1, float nscale, float mult, float eps,
                                                               float g1, float g2, T* __restrict__ out1,
                                                               T* __restrict__ out2, int W) {
  __shared__ float red[NT / 64];
  const size_t base = static_cast<size_t>(blockIdx.x) * W;
  float* x = resid + base;
  float ra = 0.f, rb = 0.f;
  if (a != nullptr) {
    float s = 0.f;
    for (int i = threadIdx.x; i < W; i += NT) {
      const float v = Elem<T>::ld(a[base + i]);
      s += v * v;
    }
    ra = nscale / sqrtf(block_sum(s, red) / W + eps);
  }
  if (b != nullptr) {
    float s = 0.f;
    for (int i = threadIdx.x; i < W; i += NT) {
      const float v = Elem<T>::ld(b[base + i]);
      s += v * v;
    }
    rb = nscale / sqrtf(block_sum(s, red) / W + eps);
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += NT) {
    float s = 0.f;
    if (a != nullptr) s = Elem<T>::ld(a[base + i]) * ra * wa[i];
    if (b != nullptr) s += Elem<T>::ld(b[base + i]) * rb * wb[i];
    if (p0 != nullptr) s += Elem<T>::ld(p0[base + i]);
    if (p1 != nullptr) s += Elem<T>::ld(p1[base + i]);
    const float v = x[i] + mult * s;
    x[i] = v;
    ss += v * v;
  }
  if (out1 == nullptr) return;
  const float r = 1.0f / sqrtf(block_sum(ss, red) / W + eps);
  for (int i = threadIdx.x; i < W; i += NT) {
    const float u = x[i] * r;
    out1[base + i] = Elem<T>::st(u * g1);
    if (out2 != nullptr) out2[base + i] = Elem<T>::st(u * g2);
  }
}

// ---------------------------------------------------------------- short causal convolution over time
// out[t, c] = act(bias[c] + sum_j w[c, j] u(pos_t - taps + 1 + j)[c]) (bias null: none); u before the segment comes from the
// state row (its last taps - 1 inputs, oldest first), u before position 0 is zero.
template <typename T>
__global__ __launch_bounds__(NT) void short_conv_kernel(const T* __restrict__ y, int64_t y_stride, int C,
                                                        const float* __restrict__ w, int taps,
                                                        const int* __restrict__ positions, const int* __restrict__ token_seq,
                                                        const int* __restrict__ q_start, const int* __restrict__ state_rows,
                                                        const T* __restrict__ state, int n_rows, T* __restrict__ out, int act,
                                                        const float* __restrict__ bias) {
  const int t = blockIdx.x, c = blockIdx.y * NT + threadIdx.x;
  if (c >= C) return;
  const int seg = token_seq[t], off = t - q_start[seg], pos = positions[t];
  const int sr = state_rows[seg];
  const bool row_ok = sr >= 0 && sr < n_rows;
  float acc = bias != nullptr ? bias[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int back = taps - 1 - j;
    float u = 0.f;
    if (off >= back) u = Elem<T>::ld(y[static_cast<size_t>(t - back) * y_stride + c]);
    else if (pos - back >= 0 && row_ok) u = Elem<T>::ld(state[(static_cast<size_t>(sr) * (taps - 1) + (j + off)) * C + c]);
    acc += w[static_cast<size_t>(c) * taps + j] * u;
  }
  if (act == 1) acc = acc * sigmoidf_(acc);
  out[static_cast<size_t>(t) * C + c] = Elem<T>::st(acc);
}

// The same for VEC consecutive channels per thread (one 16-byte load per tap) and `rows`
// consecutive rows per block (CONV_ROWS in large steps, where a thread's weights are worth keeping;
// one in small steps, which need the blocks), the thread's TAPS x VEC weights in registers.  Needs C, the row
// strides and the base addresses to be multiples of VEC elements.
constexpr int CONV_ROWS = 8;

template <typename T, int VEC, int TAPS>
__global__ __launch_bounds__(NT) void short_conv_vec_kernel(const T* __restrict__ y, int64_t y_stride, int C,
                                                            const float* __restrict__ w, const int* __restrict__ positions,
                                                            const int* __restrict__ token_seq, const int* __restrict__ q_start,
                                                            const int* __restrict__ state_rows, const T* __restrict__ state,
                                                            int n_rows, T* __restrict__ out, int act, int T_,
                                                            const float* __restrict__ bias, int rows) {
  struct alignas(sizeof(T) * VEC) Vec { T e[VEC]; };
  const int c = (blockIdx.y * NT + threadIdx.x) * VEC;
  if (c >= C) return;
  float wr[VEC][TAPS], br[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    br[e] = bias != nullptr ? bias[c + e] : 0.f;
#pragma unroll
    for (int j = 0; j < TAPS; ++j) wr[e][j] = w[static_cast<size_t>(c + e) * TAPS + j];
  }
  const int t_end = min(T_, (static_cast<int>(blockIdx.x) + 1) * rows);
  for (int t = blockIdx.x * rows; t < t_end; ++t) {
    const int seg = token_seq[t], off = t - q_start[seg], pos = positions[t];
    const int sr = state_rows[seg];
    const bool row_ok = sr >= 0 && sr < n_rows;
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = br[e];
#pragma unroll
    for (int j = 0; j < TAPS; ++j) {
      const int back = TAPS - 1 - j;
      const T* src = nullptr;
      if (off >= back) src = y + static_cast<size_t>(t - back) * y_stride + c;
      else if (pos - back >= 0 && row_ok) src = state + (static_cast<size_t>(sr) * (TAPS - 1) + (j + off)) * C + c;
      if (src != nullptr) {
        const Vec u = *reinterpret_cast<const Vec*>(src);
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] += wr[e][j] * Elem<T>::ld(u.e[e]);
      }
    }
    Vec o;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float v = act == 1 ? acc[e] * sigmoidf_(acc[e]) : acc[e];
      o.e[e] = Elem<T>::st(v);
    }
    *reinterpret_cast<Vec*>(out + static_cast<size_t>(t) * C + c) = o;
  }
}

template <typename T>
bool launch_conv_vec(const T* y, int64_t y_stride, int C, const float* w, int taps, const int* ps, const int* ts, const int* qs,
                     const int* sr, const T* state, int n_rows, T* out, int act, int T_, const float* bias, hipStream_t s) {
  constexpr int VEC = 16 / sizeof(T);
  const uintptr_t bits = reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(state) | reinterpret_cast<uintptr_t>(out);
  if (C % VEC || y_stride % VEC || bits % 16 || taps < 2 || taps > 4) return false;
  const int rows = T_ >= 2048 ? CONV_ROWS : 1;
  dim3 grid((T_ + rows - 1) / rows, (C / VEC + NT - 1) / NT);
  if (taps == 2) short_conv_vec_kernel<T, VEC, 2><<<grid, NT, 0, s>>>(y, y_stride, C, w, ps, ts, qs, sr, state, n_rows, out, act, T_, bias, rows);
  else if (taps == 3) short_conv_vec_kernel<T, VEC, 3><<<grid, NT, 0, s>>>(y, y_stride, C, w, ps, ts, qs, sr, state, n_rows, out, act, T_, bias, rows);
  else short_conv_vec_kernel<T, VEC, 4><<<grid, NT, 0, s>>>(y, y_stride, C, w, ps, ts, qs, sr, state, n_rows, out, act, T_, bias, rows);
  return true;
}

// The state row after the segment: its last taps - 1 inputs (older ones move up from the old state).
template <typename T>
__global__ __launch_bounds__(NT) void short_conv_state_kernel(const T* __restrict__ y, int64_t y_stride, int C, int taps,
                                                              const int* __restrict__ positions,
                                                              const int* __restrict__ q_start,
                                                              const int* __restrict__ state_rows, T* __restrict__ state,
                                                              int n_rows) {
  const int b = blockIdx.x, c = blockIdx.y * NT + threadIdx.x;
  if (c >= C) return;
  const int t0 = q_start[b], t1 = q_start[b + 1], n = t1 - t0;
  const int sr = state_rows[b];
  if (n <= 0 || sr < 0 || sr >= n_rows) return;
  const bool fresh = positions[t0] == 0;
  T* row = state + static_cast<size_t>(sr) * (taps - 1) * C + c;
  T nw[MAX_TAPS - 1];
#pragma unroll
  for (int i = 0; i < MAX_TAPS - 1; ++i) {
    if (i < taps - 1) {
      const int back = taps - 1 - i;
      if (n >= back) nw[i] = y[static_cast<size_t>(t1 - back) * y_stride + c];
      else nw[i] = fresh ? T(0) : row[static_cast<size_t>(i + n) * C];
    }
  }
#pragma unroll
  for (int i = 0; i < MAX_TAPS - 1; ++i)
    if (i < taps - 1) row[static_cast<size_t>(i) * C] = nw[i];
}

// ---------------------------------------------------------------- whole-projection norms, pair rotary, rotated values
// One block per token.  Row [q (n_q dim) | k (n_kv dim) | v (n_kv vdim) | ...].  q and k are each
// RMS-normed over their whole width (weights q_norm / k_norm; null = as they are); features
// (2i, 2i + 1), i < half, of every q / k head turn by position * inv_freq[i]; every pair of every v
// head by position * v_inv_freq[i] (null = as they are).  K / V^T go to the paged cache in the
// slab layout of seqmix_attention.hip (one map).
template <typename T>
__global__ __launch_bounds__(NT) void rope_pairs_kv_kernel(const T* __restrict__ qkv, int64_t row_stride,
                                                           const int* __restrict__ positions, const int* __restrict__ slots,
                                                           const float* __restrict__ q_norm, const float* __restrict__ k_norm,
                                                           float eps, const float* __restrict__ inv_freq, int half,
                                                           const float* __restrict__ v_inv_freq, T* __restrict__ q_out,
                                                           T* __restrict__ k_cache, T* __restrict__ v_cache, int n_q, int n_kv,
                                                           int dim, int vdim, int BS, int num_blocks) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x;
  const T* row = qkv + static_cast<size_t>(t) * row_stride;
  const float pos = static_cast<float>(positions[t]);
  const int slot = slots[t];
  const int blk = slot / BS, off = slot - blk * BS;
  const bool kv_ok = slot >= 0 && blk < num_blocks;
  const int qw = n_q * dim, kw = n_kv * dim, vw = n_kv * vdim;
  float rq = 1.0f, rk = 1.0f;
  if (q_norm != nullptr) {
    float s = 0.f;
    for (int i = threadIdx.x; i < qw; i += NT) {
      const float v = Elem<T>::ld(row[i]);
      s += v * v;
    }
    rq = 1.0f / sqrtf(block_sum(s, red) / qw + eps);
  }
  if (k_norm != nullptr) {
    float s = 0.f;
    for (int i = threadIdx.x; i < kw; i += NT) {
      const float v = Elem<T>::ld(row[qw + i]);
      s += v * v;
    }
    rk = 1.0f / sqrtf(block_sum(s, red) / kw + eps);
  }
  const bool swz = (dim & 3) == 0;
  for (int idx = threadIdx.x; idx < qw + kw; idx += NT) {
    const bool is_q = idx < qw;
    const float* wn = is_q ? q_norm : k_norm;
    const int wi = is_q ? idx : idx - qw;
    const float rn = is_q ? rq : rk;
    const int i = wi % dim;
    float val = Elem<T>::ld(row[idx]) * rn * (wn != nullptr ? wn[wi] : 1.0f);
    if (i < 2 * half) {
      const float other = Elem<T>::ld(row[idx ^ 1]) * rn * (wn != nullptr ? wn[wi ^ 1] : 1.0f);
      float s, c;
      sincosf(pos * inv_freq[i >> 1], &s, &c);
      val = (i & 1) ? val * c + other * s : val * c - other * s;
    }
    if (is_q) {
      q_out[static_cast<size_t>(t) * qw + idx] = Elem<T>::st(val);
    } else if (kv_ok) {
      const int g = wi / dim;
      T* slab = k_cache + (static_cast<size_t>(blk) * n_kv + g) * BS * dim;
      if (swz) slab[(static_cast<size_t>(i >> 2) * BS + off) * 4 + (i & 3)] = Elem<T>::st(val);
      else slab[static_cast<size_t>(off) * dim + i] = Elem<T>::st(val);
    }
  }
  if (kv_ok) {
    const T* vrow = row + qw + kw;
    for (int idx = threadIdx.x; idx < vw; idx += NT) {
      const int g = idx / vdim, e = idx - g * vdim;
      float val = Elem<T>::ld(vrow[idx]);
      if (v_inv_freq != nullptr) {
        const float other = Elem<T>::ld(vrow[idx ^ 1]);
        float s, c;
        sincosf(pos * v_inv_freq[e >> 1], &s, &c);
        val = (e & 1) ? val * c + other * s : val * c - other * s;
      }
      T* slab = v_cache + (static_cast<size_t>(blk) * n_kv + g) * vdim * BS;
      if (swz) slab[(static_cast<size_t>(off >> 2) * vdim + e) * 4 + (off & 3)] = Elem<T>::st(val);
      else slab[static_cast<size_t>(e) * BS + off] = Elem<T>::st(val);
    }
  }
}

// x [T, heads, width]: pair (2i, 2i + 1) of every head turned by sign * position * inv_freq[i].
template <typename T>
__global__ __launch_bounds__(NT) void rotate_pairs_kernel(const T* __restrict__ x, const int* __restrict__ positions,
                                                          const float* __restrict__ inv_freq, float sign, T* __restrict__ out,
                                                          int64_t total_pairs, int heads, int width) {
  const int hp = width >> 1;
  for (int64_t p = static_cast<int64_t>(blockIdx.x) * NT + threadIdx.x; p < total_pairs;
       p += static_cast<int64_t>(gridDim.x) * NT) {
    const int64_t th = p / hp;
    const int i = static_cast<int>(p - th * hp);
    const int64_t t = th / heads;
    const float a = Elem<T>::ld(x[2 * p]), b = Elem<T>::ld(x[2 * p + 1]);
    float s, c;
    sincosf(sign * static_cast<float>(positions[t]) * inv_freq[i], &s, &c);
    out[2 * p] = Elem<T>::st(a * c - b * s);
    out[2 * p + 1] = Elem<T>::st(b * c + a * s);
  }
}

// ---------------------------------------------------------------- read / write / decay vectors of the recurrence
// HGRN2: q = silu(y_q), f = l + (1 - l) sigmoid(y_f + bias); emits q, 1 - f (the write), f (the decay).
template <typename T>
__global__ __launch_bounds__(NT) void hgrn2_prepare_kernel(const T* __restrict__ y, int64_t stride, int off_q, int off_f,
                                                           const float* __restrict__ f_bias, const float* __restrict__ lower,
                                                           float* __restrict__ q32, float* __restrict__ k32,
                                                           float* __restrict__ g32, int64_t total, int n) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * NT + threadIdx.x; i < total; i += static_cast<int64_t>(gridDim.x) * NT) {
    const int64_t t = i / n;
    const int c = static_cast<int>(i - t * n);
    const T* row = y + t * stride;
    const float q = Elem<T>::ld(row[off_q + c]);
    const float l = lower[c];
    const float f = l + (1.0f - l) * sigmoidf_(Elem<T>::ld(row[off_f + c]) + f_bias[c]);
    q32[i] = q * sigmoidf_(q);
    k32[i] = 1.0f - f;
    g32[i] = f;
  }
}

// Gated delta rule.  One block per token: q / k heads (G of them, from the convolved row c) become
// unit vectors x / sqrt(sum x^2 + 1e-6), q also times dim^-1/2; beta = sigmoid(y[off_beta + h]);
// decay g[h, i] = exp(-exp(a_log[h]) softplus(a[h, i] + dt_bias[h, i])), i < gd: gd = dim (a decay per
// key channel) or 1 (one per head); a rows have their own stride.
template <typename T>
__global__ __launch_bounds__(NT) void delta_prepare_kernel(const T* __restrict__ c, int64_t c_stride, const T* __restrict__ y,
                                                           int64_t y_stride, int off_beta, const T* __restrict__ a,
                                                           int64_t a_stride, int gd,
                                                           const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                                                           float* __restrict__ q32, float* __restrict__ k32,
                                                           float* __restrict__ g32, float* __restrict__ beta, int H, int G,
                                                           int dim) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* crow = c + static_cast<size_t>(t) * c_stride;
  const float qs = 1.0f / sqrtf(static_cast<float>(dim));
  for (int v = wave; v < 2 * G; v += NT / 64) {           // vector v: q heads, then k heads
    const T* x = crow + static_cast<size_t>(v) * dim;
    float s = 0.f;
    for (int i = lane; i < dim; i += 64) {
      const float e = Elem<T>::ld(x[i]);
      s += e * e;
    }
    const float r = (v < G ? qs : 1.0f) / sqrtf(wave_sum(s) + 1e-6f);
    float* o = (v < G ? q32 : k32) + (static_cast<size_t>(t) * G + (v < G ? v : v - G)) * dim;
    for (int i = lane; i < dim; i += 64) o[i] = Elem<T>::ld(x[i]) * r;
  }
  const int n = H * gd;
  for (int i = threadIdx.x; i < n; i += NT) {
    const float z = Elem<T>::ld(a[static_cast<size_t>(t) * a_stride + i]) + dt_bias[i];
    const float sp = z > 20.f ? z : log1pf(expf(z));
    g32[static_cast<size_t>(t) * n + i] = expf(-expf(a_log[i / gd]) * sp);
  }
  if (threadIdx.x < H) beta[static_cast<size_t>(t) * H + threadIdx.x] = sigmoidf_(Elem<T>::ld(y[static_cast<size_t>(t) * y_stride + off_beta + threadIdx.x]));
}

// ---------------------------------------------------------------- the recurrence
// Per head a dim x vdim fp32 state S; token after token
//     S <- diag(g_t) S;  u = DELTA ? beta_t (v_t - S^T k_t) : beta_t v_t;  S <- S + k_t u^T;  o_t = S^T q_t
// (beta null without DELTA: u = v_t; gd = 1: g_t is one number per head, else one per key channel).
// One workgroup of SCAN_WAVES waves per (segment, head, 8 SCAN_WAVES value columns); a wave owns 8
// columns: lane = 8 column + row group, so a lane keeps
// dim / 8 rows of one column of S in registers and the two sums over rows (S^T k and S^T q) are
// finished inside a group of 8 neighbouring lanes with three DPP adds (no LDS round trip).  The
// tokens' q / k / g vectors are staged through LDS a few tokens at a time (every lane reads
// its row group's 16-byte pieces; the groups' pieces are padded apart so that they fall into
// different banks) by the whole workgroup, so a head's vectors are fetched once per 8 SCAN_WAVES
// columns; the next chunk's loads fly under this chunk's arithmetic.
struct ScanArgs {
  const float* q; const float* k; const float* g;   // [T, Gq, dim], [T, Gq, dim], [T, H, gd]
  const void* v; int64_t v_stride;                  // [T, >= H v_head]; head h's values start at h v_head
  int v_head;                                       // = vdim, or vdim - 1 with unit_last
  int unit_last;                                    // the state's last column reads a value of 1 for every token (it
                                                    // accumulates the written keys alone: a normaliser beside the memory)
  const float* beta;                                // [T, H]
  const int* positions; const int* q_start; const int* state_rows;
  float* state;                                     // [n_rows, H, dim, vdim]
  float* out;                                       // [T, H, vdim]
  int n_rows, H, Gq, dim, vdim, gd;
};

template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  return x + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false));
}
// sum over the 8 lanes of a group (lanes 8n .. 8n + 7), the result in every lane of the group:
// neighbours in a quad, the quad's other pair, then the mirror lane of the other quad
__device__ __forceinline__ float group8_sum(float x) {
  x = dpp_add<0xB1>(x);    // quad_perm [1, 0, 3, 2]
  x = dpp_add<0x4E>(x);    // quad_perm [2, 3, 0, 1]
  return dpp_add<0x141>(x);  // row_half_mirror
}

template <typename T, int DMAX, bool DELTA>
__global__ __launch_bounds__(64 * SCAN_WAVES) void state_scan_kernel(ScanArgs a) {
  constexpr int RPL = DMAX / 8;                      // rows per lane
  constexpr int GP = RPL + 4;                        // a row group's piece of a staged vector, padded
  constexpr int VP = 8 * GP;                         // one staged vector
  constexpr int NTH = 64 * SCAN_WAVES;
  constexpr int NL = (3 * DMAX + NTH - 1) / NTH;     // staged elements per thread and token: q | k | g
  constexpr int CT = SCAN_CHUNK_ELEMS / DMAX;        // tokens staged at a time: fewer, longer waits for narrow states
  __shared__ __attribute__((aligned(16))) float vec[2][CT][3 * VP];
  const int tid = threadIdx.x, lane = tid & 63, col = lane >> 3, rg = lane & 7;
  const int b = blockIdx.x, h = blockIdx.y, j = (blockIdx.z * SCAN_WAVES + (tid >> 6)) * 8 + col;
  const int t0 = a.q_start[b], t1 = a.q_start[b + 1];
  const int sr = a.state_rows[b];
  if (t1 <= t0 || sr < 0 || sr >= a.n_rows) return;
  const bool col_ok = j < a.vdim;
  const int gq = h / (a.H / a.Gq);
  const int dim = a.dim, vdim = a.vdim;
  float* Sp = a.state + ((static_cast<size_t>(sr) * a.H + h) * dim + rg * RPL) * vdim + (col_ok ? j : 0);
  const bool load_state = a.positions[t0] != 0 && col_ok;
  float S[RPL];
#pragma unroll
  for (int i = 0; i < RPL; ++i) S[i] = (load_state && rg * RPL + i < dim) ? Sp[static_cast<size_t>(i) * vdim] : 0.f;
  const bool unit_col = a.unit_last && j == vdim - 1;
  const T* vbase = static_cast<const T*>(a.v) + h * a.v_head + ((col_ok && !unit_col) ? j : 0);

  // element e of a token is (which of q, k, g; row); rows past dim are zero.  A thread's sources
  // are walked token by token (chunks are loaded in order): one pointer step per element and
  // token instead of the full address arithmetic
  struct Chunk { float r[CT][NL], v[CT], be[CT]; };
  const float* src[NL];
  int64_t step[NL];
  bool src_ok[NL];
#pragma unroll
  for (int n = 0; n < NL; ++n) {
    const int e = tid + NTH * n, which = e / DMAX, i = e - which * DMAX;
    src_ok[n] = which < 3 && i < dim;
    const float* p = which == 0 ? a.q + (static_cast<size_t>(t0) * a.Gq + gq) * dim
                   : which == 1 ? a.k + (static_cast<size_t>(t0) * a.Gq + gq) * dim
                                : a.g + (static_cast<size_t>(t0) * a.H + h) * a.gd;
    src[n] = p + ((src_ok[n] && (which < 2 || a.gd > 1)) ? i : 0);
    step[n] = which < 2 ? static_cast<int64_t>(a.Gq) * dim : static_cast<int64_t>(a.H) * a.gd;
  }
  const T* vsrc = vbase + static_cast<size_t>(t0) * a.v_stride;
  const bool scaled = a.beta != nullptr;   // (always with DELTA)
  const float* bsrc = scaled ? a.beta + static_cast<size_t>(t0) * a.H + h : nullptr;
  auto load = [&](int first, Chunk& c) {
#pragma unroll
    for (int tt = 0; tt < CT; ++tt) {
      const bool live = first + tt < t1;
#pragma unroll
      for (int n = 0; n < NL; ++n) {
        c.r[tt][n] = (live && src_ok[n]) ? *src[n] : 0.f;
        src[n] += step[n];
      }
      c.v[tt] = (live && col_ok) ? (unit_col ? 1.0f : Elem<T>::ld(*vsrc)) : 0.f;
      vsrc += a.v_stride;
      c.be[tt] = 1.0f;
      if (scaled) {
        if (live) c.be[tt] = *bsrc;
        bsrc += a.H;
      }
    }
  };
  auto stage = [&](int buf, const Chunk& c) {
#pragma unroll
    for (int tt = 0; tt < CT; ++tt)
#pragma unroll
      for (int n = 0; n < NL; ++n) {
        const int e = tid + NTH * n, which = e / DMAX, i = e - which * DMAX;
        if (e < 3 * DMAX) vec[buf][tt][which * VP + (i / RPL) * GP + (i % RPL)] = c.r[tt][n];
      }
  };
  Chunk cur, nxt;
  load(t0, cur);
  stage(0, cur);
  __syncthreads();
  int buf = 0;
  for (int first = t0; first < t1; first += CT, buf ^= 1) {
    const bool more = first + CT < t1;
    if (more) load(first + CT, nxt);
    float keep[(CT + 7) / 8];   // outputs of the chunk: the lane of row group r keeps tokens r, r + 8, ...
#pragma unroll
    for (int tt = 0; tt < CT; ++tt) {
      const int t = first + tt;
      if (t < t1) {
        const f32x4* qv = reinterpret_cast<const f32x4*>(&vec[buf][tt][rg * GP]);
        const f32x4* kv = reinterpret_cast<const f32x4*>(&vec[buf][tt][VP + rg * GP]);
        const f32x4* gv = reinterpret_cast<const f32x4*>(&vec[buf][tt][2 * VP + rg * GP]);
        float u = cur.v[tt];
        if (!DELTA) u *= cur.be[tt];
        if (DELTA) {
          float d[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int m = 0; m < RPL / 4; ++m) {
            const f32x4 g4 = gv[m], k4 = kv[m];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              S[4 * m + i] *= g4[i];
              d[i] += S[4 * m + i] * k4[i];
            }
          }
          u = cur.be[tt] * (u - group8_sum((d[0] + d[1]) + (d[2] + d[3])));
        }
        float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int m = 0; m < RPL / 4; ++m) {
          const f32x4 k4 = kv[m], q4 = qv[m];
          f32x4 g4 = {1.f, 1.f, 1.f, 1.f};
          if (!DELTA) g4 = gv[m];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if (DELTA) S[4 * m + i] += k4[i] * u;
            else S[4 * m + i] = S[4 * m + i] * g4[i] + k4[i] * u;
            o[i] += S[4 * m + i] * q4[i];
          }
        }
        const float os = group8_sum((o[0] + o[1]) + (o[2] + o[3]));   // (in every lane of the group)
        if (rg == (tt & 7)) keep[tt >> 3] = os;
      }
    }
    if (more) {
      stage(buf ^ 1, nxt);   // (the other buffer: its readers finished before the last barrier)
      cur = nxt;
    }
    // one store per 8 tokens, after the wait for the next chunk's loads: a store in flight never
    // stands between a load and its use
#pragma unroll
    for (int r = 0; r < (CT + 7) / 8; ++r) {
      const int t = first + 8 * r + rg;
      if (col_ok && 8 * r + rg < CT && t < t1) a.out[(static_cast<size_t>(t) * a.H + h) * vdim + j] = keep[r];
    }
    __syncthreads();
  }
  if (col_ok) {
#pragma unroll
    for (int i = 0; i < RPL; ++i)
      if (rg * RPL + i < dim) Sp[static_cast<size_t>(i) * vdim] = S[i];
  }
}

// o fp32 [T, H, vdim] -> out [T, H vdim]: every head over its root mean square, times w [vdim]
// (w_head = 0) or w [H vdim] (w_head = vdim), times sigmoid(gate[t, h vdim + e]) (gate_kind 0) or silu
// of it (1) (gate null: none).  With `floor_` [T, H] a head of o has vdim + 1 columns and is first
// divided by max(|last column|, floor) + 1e-6 (a memory read beside its normaliser).  One wave per
// (token, head).
template <typename T>
__global__ __launch_bounds__(NT) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w, float eps,
                                                            const T* __restrict__ gate, int64_t gate_stride,
                                                            T* __restrict__ out, int64_t n_heads_total, int H, int vdim,
                                                            int gate_kind, const float* __restrict__ floor_, int w_head) {
  const int lane = threadIdx.x & 63;
  const int64_t th = static_cast<int64_t>(blockIdx.x) * (NT / 64) + (threadIdx.x >> 6);
  if (th >= n_heads_total) return;
  const float* x = o + th * (vdim + (floor_ != nullptr ? 1 : 0));
  const float pre = floor_ != nullptr ? 1.0f / (fmaxf(fabsf(x[vdim]), floor_[th]) + 1e-6f) : 1.0f;
  float s = 0.f;
  for (int e = lane; e < vdim; e += 64) s += (x[e] * pre) * (x[e] * pre);
  const float r = pre / sqrtf(wave_sum(s) / vdim + eps);
  const int64_t t = th / H;
  const int h = static_cast<int>(th - t * H);
  for (int e = lane; e < vdim; e += 64) {
    float v = x[e] * r * w[h * w_head + e];
    if (gate != nullptr) {
      const float z = Elem<T>::ld(gate[t * gate_stride + static_cast<int64_t>(h) * vdim + e]);
      v *= gate_kind == 0 ? sigmoidf_(z) : z * sigmoidf_(z);
    }
    out[th * vdim + e] = Elem<T>::st(v);
  }
}

template <typename T, bool DELTA>
int launch_scan(const ScanArgs& a, int B, hipStream_t s) {
  dim3 grid(B, a.H, (a.vdim + 8 * SCAN_WAVES - 1) / (8 * SCAN_WAVES));
  if (a.dim <= 32) state_scan_kernel<T, 32, DELTA><<<grid, 64 * SCAN_WAVES, 0, s>>>(a);
  else if (a.dim <= 64) state_scan_kernel<T, 64, DELTA><<<grid, 64 * SCAN_WAVES, 0, s>>>(a);
  else if (a.dim <= 128) state_scan_kernel<T, 128, DELTA><<<grid, 64 * SCAN_WAVES, 0, s>>>(a);
  else state_scan_kernel<T, 256, DELTA><<<grid, 64 * SCAN_WAVES, 0, s>>>(a);
  return BCG_CHECK_LAUNCH();
}

inline int ew_grid(int64_t total) { return static_cast<int>(std::min<int64_t>((total + NT - 1) / NT, 65536)); }

}  // namespace

#define BCG_BY_TYPE(CALL_F32, CALL_BF16) do { if (is_f32) { CALL_F32; } else { CALL_BF16; } } while (0)

BCG_API int bcg_embed_hashed_bigram(const void* tokens, const void* positions, const void* token_seq, const void* q_start,
                                    const void* state_rows, void* prev, int n_rows, const void* table, float scale,
                                    const void* bigram, int buckets, int mul_prev, int mul_cur, float eps, float g1, float g2,
                                    void* resid, void* out1, void* out2, int T_, int B, int W, int vocab, int is_f32,
                                    void* stream) {
  if (T_ <= 0) return 0;
  if (bigram != nullptr && buckets <= 0) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int *tk = static_cast<const int*>(tokens), *ps = static_cast<const int*>(positions),
            *ts = static_cast<const int*>(token_seq), *qs = static_cast<const int*>(q_start),
            *sr = static_cast<const int*>(state_rows);
  BCG_BY_TYPE((embed_bigram_kernel<float><<<T_, NT, 0, s>>>(tk, ps, ts, qs, sr, static_cast<const int*>(prev), n_rows,
                                                           static_cast<const float*>(table), scale, static_cast<const float*>(bigram),
                                                           buckets, mul_prev, mul_cur, eps, g1, g2, static_cast<float*>(resid),
                                                           static_cast<float*>(out1), static_cast<float*>(out2), W, vocab)),
              (embed_bigram_kernel<bf16_t><<<T_, NT, 0, s>>>(tk, ps, ts, qs, sr, static_cast<const int*>(prev), n_rows,
                                                            static_cast<const bf16_t*>(table), scale, static_cast<const bf16_t*>(bigram),
                                                            buckets, mul_prev, mul_cur, eps, g1, g2, static_cast<float*>(resid),
                                                            static_cast<bf16_t*>(out1), static_cast<bf16_t*>(out2), W, vocab)));
  if (bigram != nullptr && B > 0)   // after every reader of the old value
    last_token_kernel<<<(B + 63) / 64, 64, 0, s>>>(tk, qs, sr, static_cast<int*>(prev), n_rows, B);
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_residual_mix_norm(void* resid, const void* a, const void* wa, const void* b, const void* wb, const void* p0,
                                  const void* p1, float nscale, float mult, float eps, float g1, float g2, void* out1,
                                  void* out2, int T_, int W, int is_f32, void* stream) {
  if (T_ <= 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float *fa = static_cast<const float*>(wa), *fb = static_cast<const float*>(wb);
  BCG_BY_TYPE((residual_mix_norm_kernel<float><<<T_, NT, 0, s>>>(static_cast<float*>(resid), static_cast<const float*>(a), fa,
                                                                static_cast<const float*>(b), fb, static_cast<const float*>(p0),
                                                                static_cast<const float*>(p1), nscale, mult, eps, g1, g2,
                                                                static_cast<float*>(out1), static_cast<float*>(out2), W)),
              (residual_mix_norm_kernel<bf16_t><<<T_, NT, 0, s>>>(static_cast<float*>(resid), static_cast<const bf16_t*>(a), fa,
                                                                 static_cast<const bf16_t*>(b), fb, static_cast<const bf16_t*>(p0),
                                                                 static_cast<const bf16_t*>(p1), nscale, mult, eps, g1, g2,
                                                                 static_cast<bf16_t*>(out1), static_cast<bf16_t*>(out2), W)));
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_short_conv(const void* y, int64_t y_stride, int C, const void* w, int taps, const void* positions,
                           const void* token_seq, const void* q_start, const void* state_rows, void* state, int n_rows,
                           void* out, int act, const void* bias, int T_, int B, int is_f32, void* stream) {
  if (T_ <= 0 || C <= 0) return 0;
  if (taps < 1 || taps > MAX_TAPS || (taps > 1 && state == nullptr)) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int *ps = static_cast<const int*>(positions), *ts = static_cast<const int*>(token_seq),
            *qs = static_cast<const int*>(q_start), *sr = static_cast<const int*>(state_rows);
  const float *wf = static_cast<const float*>(w), *bf = static_cast<const float*>(bias);
  dim3 grid(T_, (C + NT - 1) / NT), sgrid(B, (C + NT - 1) / NT);
  if (T_ > 2147483647 / 2 || grid.y > 65535) return -2;
  const bool vec = is_f32 ? launch_conv_vec<float>(static_cast<const float*>(y), y_stride, C, wf, taps, ps, ts, qs, sr,
                                                   static_cast<const float*>(state), n_rows, static_cast<float*>(out), act, T_, bf, s)
                          : launch_conv_vec<bf16_t>(static_cast<const bf16_t*>(y), y_stride, C, wf, taps, ps, ts, qs, sr,
                                                    static_cast<const bf16_t*>(state), n_rows, static_cast<bf16_t*>(out), act, T_, bf, s);
  if (!vec)
  BCG_BY_TYPE((short_conv_kernel<float><<<grid, NT, 0, s>>>(static_cast<const float*>(y), y_stride, C, wf, taps, ps, ts, qs, sr,
                                                           static_cast<const float*>(state), n_rows, static_cast<float*>(out), act, bf)),
              (short_conv_kernel<bf16_t><<<grid, NT, 0, s>>>(static_cast<const bf16_t*>(y), y_stride, C, wf, taps, ps, ts, qs, sr,
                                                            static_cast<const bf16_t*>(state), n_rows, static_cast<bf16_t*>(out), act, bf)));
  if (taps > 1 && B > 0)
    BCG_BY_TYPE((short_conv_state_kernel<float><<<sgrid, NT, 0, s>>>(static_cast<const float*>(y), y_stride, C, taps, ps, qs, sr,
                                                                    static_cast<float*>(state), n_rows)),
                (short_conv_state_kernel<bf16_t><<<sgrid, NT, 0, s>>>(static_cast<const bf16_t*>(y), y_stride, C, taps, ps, qs, sr,
                                                                     static_cast<bf16_t*>(state), n_rows)));
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_rope_pairs_kv_write(const void* qkv, int64_t row_stride, const void* positions, const void* slots,
                                    const void* q_norm, const void* k_norm, float eps, const void* inv_freq, int half,
                                    const void* v_inv_freq, void* q_out, void* k_cache, void* v_cache, int T_, int n_q,
                                    int n_kv, int dim, int vdim, int BS, int num_blocks, int is_f32, void* stream) {
  if (T_ <= 0) return 0;
  if (2 * half > dim || (half > 0 && (dim & 1)) || (v_inv_freq != nullptr && (vdim & 1))) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int *ps = static_cast<const int*>(positions), *sl = static_cast<const int*>(slots);
  const float *qn = static_cast<const float*>(q_norm), *kn = static_cast<const float*>(k_norm),
              *fr = static_cast<const float*>(inv_freq), *vf = static_cast<const float*>(v_inv_freq);
  BCG_BY_TYPE((rope_pairs_kv_kernel<float><<<T_, NT, 0, s>>>(static_cast<const float*>(qkv), row_stride, ps, sl, qn, kn, eps, fr, half,
                                                            vf, static_cast<float*>(q_out), static_cast<float*>(k_cache),
                                                            static_cast<float*>(v_cache), n_q, n_kv, dim, vdim, BS, num_blocks)),
              (rope_pairs_kv_kernel<bf16_t><<<T_, NT, 0, s>>>(static_cast<const bf16_t*>(qkv), row_stride, ps, sl, qn, kn, eps, fr, half,
                                                             vf, static_cast<bf16_t*>(q_out), static_cast<bf16_t*>(k_cache),
                                                             static_cast<bf16_t*>(v_cache), n_q, n_kv, dim, vdim, BS, num_blocks)));
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_rotate_pairs(const void* x, const void* positions, const void* inv_freq, float sign, void* out, int T_,
                             int heads, int width, int is_f32, void* stream) {
  if (T_ <= 0 || heads <= 0 || width <= 0) return 0;
  if (width & 1) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t total = static_cast<int64_t>(T_) * heads * (width / 2);
  const int* ps = static_cast<const int*>(positions);
  const float* fr = static_cast<const float*>(inv_freq);
  BCG_BY_TYPE((rotate_pairs_kernel<float><<<ew_grid(total), NT, 0, s>>>(static_cast<const float*>(x), ps, fr, sign,
                                                                       static_cast<float*>(out), total, heads, width)),
              (rotate_pairs_kernel<bf16_t><<<ew_grid(total), NT, 0, s>>>(static_cast<const bf16_t*>(x), ps, fr, sign,
                                                                        static_cast<bf16_t*>(out), total, heads, width)));
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_hgrn2_prepare(const void* y, int64_t stride, int off_q, int off_f, const void* f_bias, const void* lower,
                              void* q32, void* k32, void* g32, int T_, int n, int is_f32, void* stream) {
  if (T_ <= 0 || n <= 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t total = static_cast<int64_t>(T_) * n;
  const float *fb = static_cast<const float*>(f_bias), *lo = static_cast<const float*>(lower);
  BCG_BY_TYPE((hgrn2_prepare_kernel<float><<<ew_grid(total), NT, 0, s>>>(static_cast<const float*>(y), stride, off_q, off_f, fb, lo,
                                                                        static_cast<float*>(q32), static_cast<float*>(k32),
                                                                        static_cast<float*>(g32), total, n)),
              (hgrn2_prepare_kernel<bf16_t><<<ew_grid(total), NT, 0, s>>>(static_cast<const bf16_t*>(y), stride, off_q, off_f, fb, lo,
                                                                         static_cast<float*>(q32), static_cast<float*>(k32),
                                                                         static_cast<float*>(g32), total, n)));
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_delta_prepare(const void* c, int64_t c_stride, const void* y, int64_t y_stride, int off_beta, const void* a,
                              int64_t a_stride, int gd, const void* a_log, const void* dt_bias, void* q32, void* k32, void* g32,
                              void* beta, int T_, int H, int G, int dim, int is_f32, void* stream) {
  if (T_ <= 0) return 0;
  if (H > NT || H <= 0 || G <= 0 || H % G || (gd != 1 && gd != dim)) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float *al = static_cast<const float*>(a_log), *db = static_cast<const float*>(dt_bias);
  float *q = static_cast<float*>(q32), *k = static_cast<float*>(k32), *g = static_cast<float*>(g32), *be = static_cast<float*>(beta);
  BCG_BY_TYPE((delta_prepare_kernel<float><<<T_, NT, 0, s>>>(static_cast<const float*>(c), c_stride, static_cast<const float*>(y),
                                                            y_stride, off_beta, static_cast<const float*>(a), a_stride, gd, al, db, q, k, g, be, H, G, dim)),
              (delta_prepare_kernel<bf16_t><<<T_, NT, 0, s>>>(static_cast<const bf16_t*>(c), c_stride, static_cast<const bf16_t*>(y),
                                                             y_stride, off_beta, static_cast<const bf16_t*>(a), a_stride, gd, al, db, q, k, g, be, H, G, dim)));
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_gated_state_scan(const void* q32, const void* k32, const void* g32, const void* v, int64_t v_stride,
                                 const void* beta, const void* positions, const void* q_start, const void* state_rows,
                                 void* state, int n_rows, void* out, int B, int H, int Gq, int dim, int vdim, int gd, int delta,
                                 int unit_last, int is_f32, void* stream) {
  if (B <= 0) return 0;
  if (dim < 1 || dim > 256 || H <= 0 || Gq <= 0 || H % Gq || H > 65535 || (delta && beta == nullptr) || (gd != 1 && gd != dim)) return -2;
  if (unit_last && (delta || vdim < 2)) return -2;
  ScanArgs a;
  a.q = static_cast<const float*>(q32); a.k = static_cast<const float*>(k32); a.g = static_cast<const float*>(g32);
  a.v = v; a.v_stride = v_stride; a.v_head = unit_last ? vdim - 1 : vdim; a.unit_last = unit_last; a.beta = static_cast<const float*>(beta);
  a.positions = static_cast<const int*>(positions); a.q_start = static_cast<const int*>(q_start);
  a.state_rows = static_cast<const int*>(state_rows);
  a.state = static_cast<float*>(state); a.out = static_cast<float*>(out);
  a.n_rows = n_rows; a.H = H; a.Gq = Gq; a.dim = dim; a.vdim = vdim; a.gd = gd;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (delta) return is_f32 ? launch_scan<float, true>(a, B, s) : launch_scan<bf16_t, true>(a, B, s);
  return is_f32 ? launch_scan<float, false>(a, B, s) : launch_scan<bf16_t, false>(a, B, s);
}

BCG_API int bcg_head_norm_gate(const void* o32, const void* w, float eps, const void* gate, int64_t gate_stride, void* out,
                               int T_, int H, int vdim, int gate_kind, const void* floor_, int w_head, int is_f32,
                               void* stream) {
  if (T_ <= 0 || H <= 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t n = static_cast<int64_t>(T_) * H;
  const int grid = static_cast<int>((n + NT / 64 - 1) / (NT / 64));
  const float *o = static_cast<const float*>(o32), *wf = static_cast<const float*>(w);
  BCG_BY_TYPE((head_norm_gate_kernel<float><<<grid, NT, 0, s>>>(o, wf, eps, static_cast<const float*>(gate), gate_stride,
                                                               static_cast<float*>(out), n, H, vdim, gate_kind,
                                                               static_cast<const float*>(floor_), w_head)),
              (head_norm_gate_kernel<bf16_t><<<grid, NT, 0, s>>>(o, wf, eps, static_cast<const bf16_t*>(gate), gate_stride,
                                                                static_cast<bf16_t*>(out), n, H, vdim, gate_kind,
                                                                static_cast<const float*>(floor_), w_head)));
  return BCG_CHECK_LAUNCH();
}
