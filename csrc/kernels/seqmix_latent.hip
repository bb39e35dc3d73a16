// Dynamic-tanh norms around the fp32 residual stream, the latent-attention cache write and query
// assembly, output gates, the preparation and the gated grouped norm of the selective state-space
// mixer, and the per-layer token input.
//
//   dynamic-tanh norm (alpha, w, b):  tanh(alpha x) w + b   -- elementwise, no row statistic
//   latent cache of a token:          K row = [rms(c) w | turned shared key part],  V^T column = rms(c) w
//                                     in the slab layout of seqmix_attention.hip with ONE KV head
//   rotary:                           feature i of the turned part pairs with i + half; cos and sin
//                                     both carry an amplitude (frequency-scaled rotary)
//
// T is the activation type (bf16 bits or float); the stream, the norms, angles, decays and step
// sizes are fp32.
#include <algorithm>

#include "seqmix_common.h"

namespace {

constexpr int NT = 256;

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
__device__ __forceinline__ float siluf_(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float gelu_tanhf_(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

struct Dyt { float alpha; const float* w; const float* b; };
__device__ __forceinline__ float dyt(const Dyt& n, float x, int i) { return tanhf(n.alpha * x) * n.w[i] + n.b[i]; }

// ---------------------------------------------------------------- embedding * scale -> stream, first norm
template <typename T>
__global__ __launch_bounds__(NT) void embed_scale_dyt_kernel(const int* __restrict__ tokens, const T* __restrict__ table,
                                                             float scale, Dyt norm, float* __restrict__ resid,
                                                             T* __restrict__ out, int W, int vocab) {
  const int t = blockIdx.x;
  int tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  const T* row = table + static_cast<size_t>(tok) * W;
  const size_t base = static_cast<size_t>(t) * W;
  for (int i = threadIdx.x; i < W; i += NT) {
    const float v = Elem<T>::ld(row[i]) * scale;
    resid[base + i] = v;
    out[base + i] = Elem<T>::st(dyt(norm, v, i));
  }
}

// ---------------------------------------------------------------- x += post(y); out = pre(x)
// POST 0: dynamic tanh of y; 1: y / sqrt(mean(y^2) + eps) * w.  PRE 0: nothing; 1: x rounded to T;
// 2: dynamic tanh of the new x.  Y is the type of the sublayer output (T, or float for the fp32
// sum of the experts).
template <typename T> struct Vec4 { typedef f32x4 type; };
template <> struct Vec4<bf16_t> { typedef u16x4 type; };

// The same with four consecutive columns per thread (W a multiple of 4, every pointer 16-byte
// aligned): 8- / 16-byte loads and stores.
template <typename T, typename Y, int POST>
__global__ __launch_bounds__(NT) void residual_post_norm_vec_kernel(float* __restrict__ resid, const Y* __restrict__ y, Dyt post,
                                                                    float eps, int pre_kind, Dyt pre, T* __restrict__ out, int W) {
  typedef typename Vec4<T>::type VT;
  typedef typename Vec4<Y>::type VY;
  __shared__ float red[NT / 64];
  const size_t base = static_cast<size_t>(blockIdx.x) * W;
  float r = 1.0f;
  if (POST == 1) {
    float ss = 0.f;
    for (int i = 4 * threadIdx.x; i < W; i += 4 * NT) {
      const VY v = *reinterpret_cast<const VY*>(y + base + i);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float f = Elem<Y>::ld(v[j]);
        ss += f * f;
      }
    }
    r = 1.0f / sqrtf(block_sum(ss, red) / W + eps);
  }
  for (int i = 4 * threadIdx.x; i < W; i += 4 * NT) {
    const VY v = *reinterpret_cast<const VY*>(y + base + i);
    f32x4 x = *reinterpret_cast<const f32x4*>(resid + base + i);
    const f32x4 pw = *reinterpret_cast<const f32x4*>(post.w + i);
    f32x4 pb = {0.f, 0.f, 0.f, 0.f}, qw = pb, qb = pb;
    if (POST == 0) pb = *reinterpret_cast<const f32x4*>(post.b + i);
    if (pre_kind == 2) {
      qw = *reinterpret_cast<const f32x4*>(pre.w + i);
      qb = *reinterpret_cast<const f32x4*>(pre.b + i);
    }
    VT o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float f = Elem<Y>::ld(v[j]);
      x[j] += POST == 0 ? tanhf(post.alpha * f) * pw[j] + pb[j] : f * r * pw[j];
      o[j] = Elem<T>::st(pre_kind == 2 ? tanhf(pre.alpha * x[j]) * qw[j] + qb[j] : x[j]);
    }
    *reinterpret_cast<f32x4*>(resid + base + i) = x;
    if (pre_kind != 0) *reinterpret_cast<VT*>(out + base + i) = o;
  }
}

template <typename T, typename Y, int POST>
__global__ __launch_bounds__(NT) void residual_post_norm_kernel(float* __restrict__ resid, const Y* __restrict__ y, Dyt post,
                                                                float eps, int pre_kind, Dyt pre, T* __restrict__ out, int W) {
  __shared__ float red[NT / 64];
  const size_t base = static_cast<size_t>(blockIdx.x) * W;
  float r = 1.0f;
  if (POST == 1) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < W; i += NT) {
      const float v = Elem<Y>::ld(y[base + i]);
      ss += v * v;
    }
    r = 1.0f / sqrtf(block_sum(ss, red) / W + eps);
  }
  for (int i = threadIdx.x; i < W; i += NT) {
    const float v = Elem<Y>::ld(y[base + i]);
    const float x = resid[base + i] + (POST == 0 ? dyt(post, v, i) : v * r * post.w[i]);
    resid[base + i] = x;
    if (pre_kind == 1) out[base + i] = Elem<T>::st(x);
    else if (pre_kind == 2) out[base + i] = Elem<T>::st(dyt(pre, x, i));
  }
}

// ---------------------------------------------------------------- RMS norm over a column block of a strided row
template <typename T>
__global__ __launch_bounds__(NT) void rmsnorm_cols_kernel(const T* __restrict__ y, int64_t stride, int off, int n,
                                                          const float* __restrict__ w, float eps, T* __restrict__ out) {
  __shared__ float red[NT / 64];
  const T* row = y + static_cast<size_t>(blockIdx.x) * stride + off;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += NT) {
    const float v = Elem<T>::ld(row[i]);
    ss += v * v;
  }
  const float r = 1.0f / sqrtf(block_sum(ss, red) / n + eps);
  T* o = out + static_cast<size_t>(blockIdx.x) * n;
  for (int i = threadIdx.x; i < n; i += NT) o[i] = Elem<T>::st(Elem<T>::ld(row[i]) * r * w[i]);
}

// ---------------------------------------------------------------- latent + shared rotated key part -> pages
// One wave per token (a row is a few hundred features: no block-wide reduction, four tokens per
// workgroup).  Columns off .. off + R - 1 of the row are the latent (RMS norm, weight w),
// the next RD the shared key part (the first 2 half of them turned by position * inv_freq, times
// amp).  K slab of the token's page: features [latent | key part]; V^T slab: the latent.
template <typename T>
__global__ __launch_bounds__(NT) void latent_kv_write_kernel(const T* __restrict__ y, int64_t stride, int off, int R, int RD,
                                                             const float* __restrict__ w, float eps,
                                                             const int* __restrict__ positions, const int* __restrict__ slots,
                                                             const float* __restrict__ inv_freq, int half, float amp,
                                                             T* __restrict__ k_cache, T* __restrict__ v_cache, int BS,
                                                             int num_blocks, int T_) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * (NT / 64) + (threadIdx.x >> 6);
  if (t >= T_) return;
  const T* row = y + static_cast<size_t>(t) * stride + off;
  float ss = 0.f;
  for (int i = lane; i < R; i += 64) {
    const float v = Elem<T>::ld(row[i]);
    ss += v * v;
  }
  const float r = 1.0f / sqrtf(wave_sum(ss) / R + eps);
  const int slot = slots[t];
  const int blk = slot / BS, o = slot - blk * BS;
  if (slot < 0 || blk >= num_blocks) return;
  const int KD = R + RD;
  const bool swz = (KD & 3) == 0;
  T* ks = k_cache + static_cast<size_t>(blk) * BS * KD;
  T* vs = v_cache + static_cast<size_t>(blk) * R * BS;
  const float pos = static_cast<float>(positions[t]);
  for (int i = lane; i < KD; i += 64) {
    float val;
    if (i < R) {
      val = Elem<T>::ld(row[i]) * r * w[i];
      const T c = Elem<T>::st(val);
      if (swz) vs[(static_cast<size_t>(o >> 2) * R + i) * 4 + (o & 3)] = c;
      else vs[static_cast<size_t>(i) * BS + o] = c;
    } else {
      const int j = i - R;
      val = Elem<T>::ld(row[i]);
      if (j < 2 * half) {
        const int f = j < half ? j : j - half;
        float s, c;
        sincosf(pos * inv_freq[f], &s, &c);
        s *= amp;
        c *= amp;
        const float other = Elem<T>::ld(row[j < half ? i + half : i - half]);
        val = j < half ? val * c - other * s : val * c + other * s;
      }
    }
    if (swz) ks[(static_cast<size_t>(i >> 2) * BS + o) * 4 + (i & 3)] = Elem<T>::st(val);
    else ks[static_cast<size_t>(o) * KD + i] = Elem<T>::st(val);
  }
}

// dst[t, h, dst_off + j] = turn(src[t, h, src_off + j]), j < n: the first 2 half features of the
// tail turn by position * inv_freq (j pairs with j + half), the others are copied.  A thread owns
// one pair (or one copied feature) of a token for `hpt` heads: with hpt = H one sincos serves all
// heads of a token (large steps), with hpt = 1 every head has a thread of its own (small steps).
template <typename T>
__global__ __launch_bounds__(NT) void rope_half_tail_kernel(const T* __restrict__ src, int Ds, int src_off, T* __restrict__ dst,
                                                            int Dd, int dst_off, int n, const int* __restrict__ positions,
                                                            const float* __restrict__ inv_freq, int half, float amp,
                                                            int64_t total, int H, int hpt) {
  const int per = n - half;   // work items of a (token, head chunk): `half` pairs, then the copied features
  const int chunks = H / hpt;
  for (int64_t e = static_cast<int64_t>(blockIdx.x) * NT + threadIdx.x; e < total; e += static_cast<int64_t>(gridDim.x) * NT) {
    const int64_t tc = e / per;
    const int j = static_cast<int>(e - tc * per);
    const int64_t t = tc / chunks;
    const int h0 = static_cast<int>(tc - t * chunks) * hpt;
    const T* s = src + (t * H + h0) * Ds + src_off;
    T* d = dst + (t * H + h0) * Dd + dst_off;
    if (j < half) {
      float sn, cs;
      sincosf(static_cast<float>(positions[t]) * inv_freq[j], &sn, &cs);
      sn *= amp;
      cs *= amp;
      for (int h = 0; h < hpt; ++h) {
        const float a = Elem<T>::ld(s[h * Ds + j]), b = Elem<T>::ld(s[h * Ds + j + half]);
        d[h * Dd + j] = Elem<T>::st(a * cs - b * sn);
        d[h * Dd + j + half] = Elem<T>::st(b * cs + a * sn);
      }
    } else {
      for (int h = 0; h < hpt; ++h) d[h * Dd + j + half] = s[h * Ds + j + half];
    }
  }
}

// out = x * sigmoid(gate) (kind 0) or x * silu(gate) (kind 1); gate rows have their own stride and
// one gate column serves `group` neighbouring columns of x (group = a head's width: one gate per head).
template <typename T>
__global__ __launch_bounds__(NT) void gate_mul_kernel(const T* __restrict__ x, const T* __restrict__ gate, int64_t gate_stride,
                                                      T* __restrict__ out, int64_t rows, int n, int kind, int group) {
  const int64_t total = rows * n;
  for (int64_t e = static_cast<int64_t>(blockIdx.x) * NT + threadIdx.x; e < total; e += static_cast<int64_t>(gridDim.x) * NT) {
    const int64_t r = e / n;
    const int c = static_cast<int>(e - r * n);
    const float g = Elem<T>::ld(gate[r * gate_stride + c / group]);
    out[e] = Elem<T>::st(Elem<T>::ld(x[e]) * (kind == 0 ? sigmoidf_(g) : siluf_(g)));
  }
}

// out[r, c] = silu(in[r, c]) * in[r, n + c]: the hidden activation of a gated expert from its
// stacked [gate | up] projection.
template <typename T>
__global__ __launch_bounds__(NT) void gated_act_kernel(const T* __restrict__ in, T* __restrict__ out, int64_t rows, int n) {
  const int64_t total = rows * n;
  for (int64_t e = static_cast<int64_t>(blockIdx.x) * NT + threadIdx.x; e < total; e += static_cast<int64_t>(gridDim.x) * NT) {
    const int64_t r = e / n;
    const int c = static_cast<int>(e - r * n);
    // rounded as a projection's output before the product, like every other activation
    const float g = Elem<T>::ld(Elem<T>::st(siluf_(Elem<T>::ld(in[r * 2 * n + c]))));
    out[e] = Elem<T>::st(g * Elem<T>::ld(in[r * 2 * n + n + c]));
  }
}

// ---------------------------------------------------------------- selective state space: read / write / decay / step
// c row: B (G N) | C (G N) at off_b after convolution and activation; y row: dt logits at off_dt.
// q32 = C, k32 = B (fp32 copies), dt = softplus(y + dt_bias), g = exp(-exp(a_log) dt).
template <typename T>
__global__ __launch_bounds__(NT) void ssm_prepare_kernel(const T* __restrict__ c, int64_t c_stride, int off_b,
                                                         const T* __restrict__ y, int64_t y_stride, int off_dt,
                                                         const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                                                         float* __restrict__ q32, float* __restrict__ k32,
                                                         float* __restrict__ g32, float* __restrict__ dt32, int H, int GN) {
  const int t = blockIdx.x;
  const T* crow = c + static_cast<size_t>(t) * c_stride + off_b;
  for (int i = threadIdx.x; i < GN; i += NT) {
    k32[static_cast<size_t>(t) * GN + i] = Elem<T>::ld(crow[i]);
    q32[static_cast<size_t>(t) * GN + i] = Elem<T>::ld(crow[GN + i]);
  }
  for (int h = threadIdx.x; h < H; h += NT) {
    const float dt = softplusf_(Elem<T>::ld(y[static_cast<size_t>(t) * y_stride + off_dt + h]) + dt_bias[h]);
    dt32[static_cast<size_t>(t) * H + h] = dt;
    g32[static_cast<size_t>(t) * H + h] = expf(-expf(a_log[h]) * dt);
  }
}

// u = (o + skip_w[h] skip) silu(z); the row in `parts` equal pieces, each over its own root mean
// square, times w.  One block per (token, piece).
template <typename T>
__global__ __launch_bounds__(NT) void gated_group_norm_kernel(const float* __restrict__ o, const T* __restrict__ skip,
                                                              int64_t skip_stride, const float* __restrict__ skip_w,
                                                              const T* __restrict__ z, int64_t z_stride,
                                                              const float* __restrict__ w, float eps, T* __restrict__ out,
                                                              int inner, int vdim, int parts) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x, n = inner / parts, c0 = blockIdx.y * n;
  const float* orow = o + static_cast<size_t>(t) * inner;
  const T* srow = skip + static_cast<size_t>(t) * skip_stride;
  const T* zrow = z + static_cast<size_t>(t) * z_stride;
  auto value = [&](int cidx) {
    return (orow[cidx] + skip_w[cidx / vdim] * Elem<T>::ld(srow[cidx])) * siluf_(Elem<T>::ld(zrow[cidx]));
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += NT) {
    const float u = value(c0 + i);
    ss += u * u;
  }
  const float r = 1.0f / sqrtf(block_sum(ss, red) / n + eps);
  for (int i = threadIdx.x; i < n; i += NT) out[static_cast<size_t>(t) * inner + c0 + i] = Elem<T>::st(value(c0 + i) * r * w[c0 + i]);
}

// out[t, c] = gelu_tanh(z[t, c]) * table[token_t, off + c]
template <typename T>
__global__ __launch_bounds__(NT) void gelu_gather_mul_kernel(const T* __restrict__ z, const int* __restrict__ tokens,
                                                             const T* __restrict__ table, int64_t table_stride, int off,
                                                             T* __restrict__ out, int64_t rows, int n, int vocab) {
  const int64_t total = rows * n;
  for (int64_t e = static_cast<int64_t>(blockIdx.x) * NT + threadIdx.x; e < total; e += static_cast<int64_t>(gridDim.x) * NT) {
    const int64_t r = e / n;
    const int c = static_cast<int>(e - r * n);
    int tok = tokens[r];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    out[e] = Elem<T>::st(gelu_tanhf_(Elem<T>::ld(z[e])) * Elem<T>::ld(table[static_cast<size_t>(tok) * table_stride + off + c]));
  }
}

inline int ew_grid(int64_t total) { return static_cast<int>(std::min<int64_t>((total + NT - 1) / NT, 65536)); }

}  // namespace

#define BCG_BY_TYPE(CALL_F32, CALL_BF16) do { if (is_f32) { CALL_F32; } else { CALL_BF16; } } while (0)

BCG_API int bcg_embed_scale_dyt(const void* tokens, const void* table, float scale, float alpha, const void* w, const void* b,
                                void* resid, void* out, int T_, int W, int vocab, int is_f32, void* stream) {
  if (T_ <= 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const Dyt n{alpha, static_cast<const float*>(w), static_cast<const float*>(b)};
  const int* tk = static_cast<const int*>(tokens);
  float* x = static_cast<float*>(resid);
  BCG_BY_TYPE((embed_scale_dyt_kernel<float><<<T_, NT, 0, s>>>(tk, static_cast<const float*>(table), scale, n, x, static_cast<float*>(out), W, vocab)),
              (embed_scale_dyt_kernel<bf16_t><<<T_, NT, 0, s>>>(tk, static_cast<const bf16_t*>(table), scale, n, x, static_cast<bf16_t*>(out), W, vocab)));
  return BCG_CHECK_LAUNCH();
}

// post_kind 0: dynamic tanh (post_alpha, post_w, post_b); 1: RMS norm (post_w, eps).  pre_kind 0 / 1 / 2:
// nothing / rounded copy / dynamic tanh (pre_alpha, pre_w, pre_b).  y_f32: y is float whatever the activation type.
BCG_API int bcg_residual_post_norm(void* resid, const void* y, int y_f32, int post_kind, float post_alpha, const void* post_w,
                                   const void* post_b, float eps, int pre_kind, float pre_alpha, const void* pre_w,
                                   const void* pre_b, void* out, int T_, int W, int is_f32, void* stream) {
  if (T_ <= 0) return 0;
  if (post_kind < 0 || post_kind > 1 || pre_kind < 0 || pre_kind > 2) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const Dyt post{post_alpha, static_cast<const float*>(post_w), static_cast<const float*>(post_b)};
  const Dyt pre{pre_alpha, static_cast<const float*>(pre_w), static_cast<const float*>(pre_b)};
  float* x = static_cast<float*>(resid);
  auto al16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const bool vec = W % 4 == 0 && al16(resid) && al16(y) && al16(out) && al16(post_w) && al16(post_b) && al16(pre_w) && al16(pre_b);
#define BCG_RPN(TYPE, YTYPE)                                                                                                  \
  do {                                                                                                                        \
    if (vec && post_kind == 0)                                                                                                \
      residual_post_norm_vec_kernel<TYPE, YTYPE, 0><<<T_, NT, 0, s>>>(x, static_cast<const YTYPE*>(y), post, eps, pre_kind,  \
                                                                      pre, static_cast<TYPE*>(out), W);                       \
    else if (vec)                                                                                                             \
      residual_post_norm_vec_kernel<TYPE, YTYPE, 1><<<T_, NT, 0, s>>>(x, static_cast<const YTYPE*>(y), post, eps, pre_kind,  \
                                                                      pre, static_cast<TYPE*>(out), W);                       \
    else if (post_kind == 0)                                                                                                  \
      residual_post_norm_kernel<TYPE, YTYPE, 0><<<T_, NT, 0, s>>>(x, static_cast<const YTYPE*>(y), post, eps, pre_kind, pre, \
                                                                  static_cast<TYPE*>(out), W);                                \
    else                                                                                                                      \
      residual_post_norm_kernel<TYPE, YTYPE, 1><<<T_, NT, 0, s>>>(x, static_cast<const YTYPE*>(y), post, eps, pre_kind, pre, \
                                                                  static_cast<TYPE*>(out), W);                                \
  } while (0)
  if (is_f32) BCG_RPN(float, float);
  else if (y_f32) BCG_RPN(bf16_t, float);
  else BCG_RPN(bf16_t, bf16_t);
#undef BCG_RPN
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_rmsnorm_cols(const void* y, int64_t stride, int off, int n, const void* w, float eps, void* out, int T_,
                             int is_f32, void* stream) {
  if (T_ <= 0 || n <= 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float* wf = static_cast<const float*>(w);
  BCG_BY_TYPE((rmsnorm_cols_kernel<float><<<T_, NT, 0, s>>>(static_cast<const float*>(y), stride, off, n, wf, eps, static_cast<float*>(out))),
              (rmsnorm_cols_kernel<bf16_t><<<T_, NT, 0, s>>>(static_cast<const bf16_t*>(y), stride, off, n, wf, eps, static_cast<bf16_t*>(out))));
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_latent_kv_write(const void* y, int64_t stride, int off, int R, int RD, const void* w, float eps,
                                const void* positions, const void* slots, const void* inv_freq, int half, float amp,
                                void* k_cache, void* v_cache, int T_, int BS, int num_blocks, int is_f32, void* stream) {
  if (T_ <= 0) return 0;
  if (R < 1 || RD < 0 || 2 * half > RD || BS % 16) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float *wf = static_cast<const float*>(w), *fr = static_cast<const float*>(inv_freq);
  const int *ps = static_cast<const int*>(positions), *sl = static_cast<const int*>(slots);
  const int grid = (T_ + NT / 64 - 1) / (NT / 64);
  BCG_BY_TYPE((latent_kv_write_kernel<float><<<grid, NT, 0, s>>>(static_cast<const float*>(y), stride, off, R, RD, wf, eps, ps, sl, fr, half, amp,
                                                                static_cast<float*>(k_cache), static_cast<float*>(v_cache), BS, num_blocks, T_)),
              (latent_kv_write_kernel<bf16_t><<<grid, NT, 0, s>>>(static_cast<const bf16_t*>(y), stride, off, R, RD, wf, eps, ps, sl, fr, half, amp,
                                                                 static_cast<bf16_t*>(k_cache), static_cast<bf16_t*>(v_cache), BS, num_blocks, T_)));
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_rope_half_tail(const void* src, int Ds, int src_off, void* dst, int Dd, int dst_off, const void* positions,
                               const void* inv_freq, int half, float amp, int T_, int H, int is_f32, void* stream) {
  const int n = Ds - src_off;
  if (T_ <= 0 || H <= 0 || n <= 0) return 0;
  if (n != Dd - dst_off || 2 * half > n) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int hpt = static_cast<int64_t>(T_) * (n - half) >= (1 << 16) ? H : 1;
  const int64_t total = static_cast<int64_t>(T_) * (H / hpt) * (n - half);
  const int* ps = static_cast<const int*>(positions);
  const float* fr = static_cast<const float*>(inv_freq);
  BCG_BY_TYPE((rope_half_tail_kernel<float><<<ew_grid(total), NT, 0, s>>>(static_cast<const float*>(src), Ds, src_off, static_cast<float*>(dst), Dd,
                                                                         dst_off, n, ps, fr, half, amp, total, H, hpt)),
              (rope_half_tail_kernel<bf16_t><<<ew_grid(total), NT, 0, s>>>(static_cast<const bf16_t*>(src), Ds, src_off, static_cast<bf16_t*>(dst), Dd,
                                                                          dst_off, n, ps, fr, half, amp, total, H, hpt)));
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_gate_mul(const void* x, const void* gate, int64_t gate_stride, void* out, int64_t rows, int n, int kind,
                         int group, int is_f32, void* stream) {
  if (rows <= 0 || n <= 0) return 0;
  if (group < 1 || n % group) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  BCG_BY_TYPE((gate_mul_kernel<float><<<ew_grid(rows * n), NT, 0, s>>>(static_cast<const float*>(x), static_cast<const float*>(gate), gate_stride,
                                                                      static_cast<float*>(out), rows, n, kind, group)),
              (gate_mul_kernel<bf16_t><<<ew_grid(rows * n), NT, 0, s>>>(static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(gate), gate_stride,
                                                                       static_cast<bf16_t*>(out), rows, n, kind, group)));
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_gated_act(const void* in, void* out, int64_t rows, int n, int is_f32, void* stream) {
  if (rows <= 0 || n <= 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  BCG_BY_TYPE((gated_act_kernel<float><<<ew_grid(rows * n), NT, 0, s>>>(static_cast<const float*>(in), static_cast<float*>(out), rows, n)),
              (gated_act_kernel<bf16_t><<<ew_grid(rows * n), NT, 0, s>>>(static_cast<const bf16_t*>(in), static_cast<bf16_t*>(out), rows, n)));
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_ssm_prepare(const void* c, int64_t c_stride, int off_b, const void* y, int64_t y_stride, int off_dt,
                            const void* dt_bias, const void* a_log, void* q32, void* k32, void* g32, void* dt32, int T_, int H,
                            int GN, int is_f32, void* stream) {
  if (T_ <= 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float *db = static_cast<const float*>(dt_bias), *al = static_cast<const float*>(a_log);
  float *q = static_cast<float*>(q32), *k = static_cast<float*>(k32), *g = static_cast<float*>(g32), *d = static_cast<float*>(dt32);
  BCG_BY_TYPE((ssm_prepare_kernel<float><<<T_, NT, 0, s>>>(static_cast<const float*>(c), c_stride, off_b, static_cast<const float*>(y), y_stride,
                                                          off_dt, db, al, q, k, g, d, H, GN)),
              (ssm_prepare_kernel<bf16_t><<<T_, NT, 0, s>>>(static_cast<const bf16_t*>(c), c_stride, off_b, static_cast<const bf16_t*>(y), y_stride,
                                                           off_dt, db, al, q, k, g, d, H, GN)));
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_gated_group_norm(const void* o32, const void* skip, int64_t skip_stride, const void* skip_w, const void* z,
                                 int64_t z_stride, const void* w, float eps, void* out, int T_, int H, int vdim, int parts,
                                 int is_f32, void* stream) {
  if (T_ <= 0) return 0;
  const int inner = H * vdim;
  if (parts < 1 || inner % parts || parts > 65535) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(T_, parts);
  const float *o = static_cast<const float*>(o32), *sw = static_cast<const float*>(skip_w), *wf = static_cast<const float*>(w);
  BCG_BY_TYPE((gated_group_norm_kernel<float><<<grid, NT, 0, s>>>(o, static_cast<const float*>(skip), skip_stride, sw, static_cast<const float*>(z),
                                                                 z_stride, wf, eps, static_cast<float*>(out), inner, vdim, parts)),
              (gated_group_norm_kernel<bf16_t><<<grid, NT, 0, s>>>(o, static_cast<const bf16_t*>(skip), skip_stride, sw, static_cast<const bf16_t*>(z),
                                                                  z_stride, wf, eps, static_cast<bf16_t*>(out), inner, vdim, parts)));
  return BCG_CHECK_LAUNCH();
}

BCG_API int bcg_gelu_gather_mul(const void* z, const void* tokens, const void* table, int64_t table_stride, int off, void* out,
                                int64_t rows, int n, int vocab, int is_f32, void* stream) {
  if (rows <= 0 || n <= 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int* tk = static_cast<const int*>(tokens);
  BCG_BY_TYPE((gelu_gather_mul_kernel<float><<<ew_grid(rows * n), NT, 0, s>>>(static_cast<const float*>(z), tk, static_cast<const float*>(table),
                                                                             table_stride, off, static_cast<float*>(out), rows, n, vocab)),
              (gelu_gather_mul_kernel<bf16_t><<<ew_grid(rows * n), NT, 0, s>>>(static_cast<const bf16_t*>(z), tk, static_cast<const bf16_t*>(table),
                                                                              table_stride, off, static_cast<bf16_t*>(out), rows, n, vocab)));
  return BCG_CHECK_LAUNCH();
}
