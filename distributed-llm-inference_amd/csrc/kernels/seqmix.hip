// Kernels of the heterogeneous decoder stacks (models/mixers.py, ops/seqmix.py): layer norm with token shift,
// post-norm residual update, unit-RMS q/k + cache write, latent-attention cache write with pair rotation,
// attention over token-major pages (sliding window, distance penalty, two-part scores), the decayed
// linear-attention scan over per-sequence state, and the element-wise pieces around them.
//
// Arithmetic: the residual stream, norm statistics, scores, softmax weights, rotation angles and the recurrent
// state are fp32 (angles: double until reduced); activations are the template type A = float or bf16 (uint16_t
// bit pattern).  Small parameters (norm weights / biases, per-head constants) are fp32 tensors.
//
// Step metadata (all int32, static device buffers → capturable): positions[T], slot_mapping[T] (cache row, < 0:
// padding), token_seq[T] (batch row of a token, < 0: padding), query_start_loc[B+1], state_slots[B] (< 0: none),
// counts[3] = number of valid batch rows (grids over batch rows are launched at an upper bound).
#include <algorithm>

#include "common.h"
#include "kernels.h"

namespace dli {

namespace {

constexpr int NT = 256;

template <typename A> __device__ __forceinline__ float ldf(const A* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf2f(*p); }
template <typename A> __device__ __forceinline__ void stf(A* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f2bf(v); }

__device__ __forceinline__ float silu_f(float x) { return x / (1.f + expf(-x)); }
// activation of a projection output: for bf16 inputs the hardware exp2 / rcp (relative error ≈ 1e-6, far inside bf16)
template <typename A> __device__ __forceinline__ float silu_act(float x);
template <> __device__ __forceinline__ float silu_act<float>(float x) { return silu_f(x); }
template <> __device__ __forceinline__ float silu_act<uint16_t>(float x) {
  return x * fast_rcp(1.f + fast_exp2(-1.4426950408889634f * x));
}

// 4 consecutive row elements ↔ fp32 (16-byte / 8-byte accesses; the callers check divisibility and alignment)
template <typename A> __device__ __forceinline__ f32x4 ld4(const A* p);
template <> __device__ __forceinline__ f32x4 ld4<float>(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
template <> __device__ __forceinline__ f32x4 ld4<uint16_t>(const uint16_t* p) {
  const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
  return f32x4{bf2f((uint16_t)v[0]), bf2f((uint16_t)v[1]), bf2f((uint16_t)v[2]), bf2f((uint16_t)v[3])};
}
template <typename A> __device__ __forceinline__ void st4(A* p, f32x4 v);
template <> __device__ __forceinline__ void st4<float>(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
template <> __device__ __forceinline__ void st4<uint16_t>(uint16_t* p, f32x4 v) {
  bf16x4 o;
#pragma unroll
  for (int j = 0; j < 4; ++j) o[j] = (short)f2bf(v[j]);
  *reinterpret_cast<bf16x4*>(p) = o;
}
__device__ __forceinline__ bool aligned_to(const void* p, int bytes) { return (reinterpret_cast<uintptr_t>(p) & (bytes - 1)) == 0; }

// q (fp32, LDS) · one cache row: 16-byte loads where the row allows them
template <typename A> __device__ __forceinline__ float dot_row(const float* __restrict__ qs, const A* __restrict__ kr, int n);
template <> __device__ __forceinline__ float dot_row<float>(const float* __restrict__ qs, const float* __restrict__ kr, int n) {
  float d = 0.f;
  int i = 0;
  if ((n & 3) == 0 && (reinterpret_cast<uintptr_t>(kr) & 15) == 0) {
    for (; i < n; i += 4) {
      const f32x4 k = *reinterpret_cast<const f32x4*>(kr + i);
      d += qs[i] * k[0] + qs[i + 1] * k[1] + qs[i + 2] * k[2] + qs[i + 3] * k[3];
    }
  }
  for (; i < n; ++i) d += qs[i] * kr[i];
  return d;
}
template <> __device__ __forceinline__ float dot_row<uint16_t>(const float* __restrict__ qs, const uint16_t* __restrict__ kr, int n) {
  float d = 0.f;
  int i = 0;
  if ((n & 7) == 0 && (reinterpret_cast<uintptr_t>(kr) & 15) == 0) {
    for (; i < n; i += 8) {
      const bf16x8 k = *reinterpret_cast<const bf16x8*>(kr + i);
#pragma unroll
      for (int j = 0; j < 8; ++j) d += qs[i + j] * bf2f((uint16_t)k[j]);
    }
  }
  for (; i < n; ++i) d += qs[i] * bf2f(kr[i]);
  return d;
}

// mean and 1/sqrt(var + eps) of a row held in LDS (two passes: the variance is the mean squared deviation)
__device__ __forceinline__ void row_stats(const float* row, int W, float eps, float* red, float& mean, float& inv) {
  const bool v4 = (W & 3) == 0;
  float s = 0.f;
  if (v4) {
    for (int i = threadIdx.x * 4; i < W; i += NT * 4) {
      const f32x4 a = *reinterpret_cast<const f32x4*>(row + i);
      s += (a[0] + a[1]) + (a[2] + a[3]);
    }
  } else {
    for (int i = threadIdx.x; i < W; i += NT) s += row[i];
  }
  mean = block_sum<NT>(s, red) / (float)W;
  float v = 0.f;
  if (v4) {
    for (int i = threadIdx.x * 4; i < W; i += NT * 4) {
      const f32x4 a = *reinterpret_cast<const f32x4*>(row + i);
#pragma unroll
      for (int j = 0; j < 4; ++j) v += (a[j] - mean) * (a[j] - mean);
    }
  } else {
    for (int i = threadIdx.x; i < W; i += NT) {
      const float d = row[i] - mean;
      v += d * d;
    }
  }
  inv = 1.f / sqrtf(block_sum<NT>(v, red) / (float)W + eps);
}

// ------------------------------------------------------------------------------------------------ norms
template <typename O>
__global__ __launch_bounds__(NT) void layer_norm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                        const float* __restrict__ b, float eps, int W, O* __restrict__ out) {
  extern __shared__ float sh[];
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const bool v4 = (W & 3) == 0;
  if (v4) {
    for (int i = threadIdx.x * 4; i < W; i += NT * 4) *reinterpret_cast<f32x4*>(sh + i) = ld4<float>(x + t * W + i);
  } else {
    for (int i = threadIdx.x; i < W; i += NT) sh[i] = x[t * W + i];
  }
  __syncthreads();
  float mean, inv;
  row_stats(sh, W, eps, red, mean, inv);
  if (v4) {
    for (int i = threadIdx.x * 4; i < W; i += NT * 4) {
      const f32x4 a = *reinterpret_cast<const f32x4*>(sh + i), ww = ld4<float>(w + i), bb = ld4<float>(b + i);
      f32x4 o;
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = (a[j] - mean) * inv * ww[j] + bb[j];
      st4<O>(out + t * W + i, o);
    }
  } else {
    for (int i = threadIdx.x; i < W; i += NT) stf<O>(out + t * W + i, (sh[i] - mean) * inv * w[i] + b[i]);
  }
}

// h[t] = g[t] + (g[t-1] - g[t]) * mix with g = layer_norm(x (+ add)); g[t-1] is recomputed from the row above inside a
// chunk, read from the sequence's state row at a chunk start, zero at position 0.  xout (with add): the new stream.
template <typename O>
__global__ __launch_bounds__(NT) void ln_shift_kernel(const float* __restrict__ x, const float* __restrict__ add,
                                                      float* __restrict__ xout, const float* __restrict__ w,
                                                      const float* __restrict__ b, const float* __restrict__ mix,
                                                      const float* __restrict__ state, const int* __restrict__ positions,
                                                      const int* __restrict__ token_seq, const int* __restrict__ qsl,
                                                      const int* __restrict__ state_slots, float eps, int W,
                                                      O* __restrict__ out) {
  extern __shared__ float sh[];
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const int seq = token_seq[t];
  if (seq < 0) return;
  const int slot = state_slots[seq];
  const int pos = positions[t];
  const bool first = (int)t == qsl[seq];
  const int mode = pos == 0 ? 0 : (first ? (slot >= 0 ? 1 : 0) : 2);
  float* cur = sh;
  float* prv = sh + W;
  const bool v4 = (W & 3) == 0;
  if (v4) {
    for (int i = threadIdx.x * 4; i < W; i += NT * 4) {
      f32x4 v = ld4<float>(x + t * W + i);
      if (add != nullptr) {
        const f32x4 a = ld4<float>(add + t * W + i);
        v = f32x4{v[0] + a[0], v[1] + a[1], v[2] + a[2], v[3] + a[3]};
        st4<float>(xout + t * W + i, v);
      }
      *reinterpret_cast<f32x4*>(cur + i) = v;
      if (mode == 2) {
        f32x4 u = ld4<float>(x + (t - 1) * W + i);
        if (add != nullptr) {
          const f32x4 a = ld4<float>(add + (t - 1) * W + i);
          u = f32x4{u[0] + a[0], u[1] + a[1], u[2] + a[2], u[3] + a[3]};
        }
        *reinterpret_cast<f32x4*>(prv + i) = u;
      }
    }
  } else {
    for (int i = threadIdx.x; i < W; i += NT) {
      float v = x[t * W + i];
      if (add != nullptr) {
        v += add[t * W + i];
        xout[t * W + i] = v;
      }
      cur[i] = v;
      if (mode == 2) prv[i] = x[(t - 1) * W + i] + (add != nullptr ? add[(t - 1) * W + i] : 0.f);
    }
  }
  __syncthreads();
  float mean, inv, pmean = 0.f, pinv = 0.f;
  row_stats(cur, W, eps, red, mean, inv);
  if (mode == 2) row_stats(prv, W, eps, red, pmean, pinv);
  if (v4) {
    for (int i = threadIdx.x * 4; i < W; i += NT * 4) {
      const f32x4 c4 = *reinterpret_cast<const f32x4*>(cur + i), ww = ld4<float>(w + i), bb = ld4<float>(b + i), mm = ld4<float>(mix + i);
      f32x4 p4 = {0.f, 0.f, 0.f, 0.f};
      if (mode == 1) p4 = ld4<float>(state + (int64_t)slot * W + i);
      else if (mode == 2) {
        const f32x4 u = *reinterpret_cast<const f32x4*>(prv + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) p4[j] = (u[j] - pmean) * pinv * ww[j] + bb[j];
      }
      f32x4 o;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float g = (c4[j] - mean) * inv * ww[j] + bb[j];
        o[j] = g + (p4[j] - g) * mm[j];
      }
      st4<O>(out + t * W + i, o);
    }
  } else {
    for (int i = threadIdx.x; i < W; i += NT) {
      const float g = (cur[i] - mean) * inv * w[i] + b[i];
      float p = 0.f;
      if (mode == 1) p = state[(int64_t)slot * W + i];
      else if (mode == 2) p = (prv[i] - pmean) * pinv * w[i] + b[i];
      stf<O>(out + t * W + i, g + (p - g) * mix[i]);
    }
  }
}

// state[slot] = layer_norm(x (+ add)) of every sequence's last token of the step (runs behind ln_shift_kernel)
__global__ __launch_bounds__(NT) void ln_state_kernel(const float* __restrict__ x, const float* __restrict__ add,
                                                      const float* __restrict__ w, const float* __restrict__ b,
                                                      float* __restrict__ state, const int* __restrict__ qsl,
                                                      const int* __restrict__ state_slots, const int* __restrict__ counts,
                                                      float eps, int W) {
  extern __shared__ float sh[];
  __shared__ float red[NT / 64];
  const int seq = blockIdx.x;
  if (seq >= counts[3]) return;
  const int slot = state_slots[seq];
  const int t0 = qsl[seq], t1 = qsl[seq + 1];
  if (slot < 0 || t1 <= t0) return;
  const int64_t t = t1 - 1;
  for (int i = threadIdx.x; i < W; i += NT) sh[i] = x[t * W + i] + (add != nullptr ? add[t * W + i] : 0.f);
  __syncthreads();
  float mean, inv;
  row_stats(sh, W, eps, red, mean, inv);
  for (int i = threadIdx.x; i < W; i += NT) state[(int64_t)slot * W + i] = (sh[i] - mean) * inv * w[i] + b[i];
}

// x += mult * layer_norm(y; w1, b1); optionally out = layer_norm(x; w2, b2)
template <typename Y, typename O>
__global__ __launch_bounds__(NT) void add_ln_kernel(float* __restrict__ x, const Y* __restrict__ y, int64_t y_stride,
                                                    const float* __restrict__ w1, const float* __restrict__ b1, float mult,
                                                    const float* __restrict__ w2, const float* __restrict__ b2, float eps,
                                                    int W, O* __restrict__ out) {
  extern __shared__ float sh[];
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const bool v4 = (W & 3) == 0 && (y_stride & 3) == 0 && aligned_to(y, 4 * sizeof(Y));
  if (v4) {
    for (int i = threadIdx.x * 4; i < W; i += NT * 4) *reinterpret_cast<f32x4*>(sh + i) = ld4<Y>(y + t * y_stride + i);
  } else {
    for (int i = threadIdx.x; i < W; i += NT) sh[i] = ldf<Y>(y + t * y_stride + i);
  }
  __syncthreads();
  float mean, inv;
  row_stats(sh, W, eps, red, mean, inv);
  if (v4) {
    for (int i = threadIdx.x * 4; i < W; i += NT * 4) {
      const f32x4 a = *reinterpret_cast<const f32x4*>(sh + i), ww = ld4<float>(w1 + i), bb = ld4<float>(b1 + i);
      f32x4 v = ld4<float>(x + t * W + i);
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] += mult * ((a[j] - mean) * inv * ww[j] + bb[j]);
      st4<float>(x + t * W + i, v);
      *reinterpret_cast<f32x4*>(sh + i) = v;
    }
  } else {
    for (int i = threadIdx.x; i < W; i += NT) {
      const float v = x[t * W + i] + mult * ((sh[i] - mean) * inv * w1[i] + b1[i]);
      x[t * W + i] = v;
      sh[i] = v;
    }
  }
  if (w2 == nullptr) return;
  __syncthreads();
  row_stats(sh, W, eps, red, mean, inv);
  if (v4) {
    for (int i = threadIdx.x * 4; i < W; i += NT * 4) {
      const f32x4 a = *reinterpret_cast<const f32x4*>(sh + i), ww = ld4<float>(w2 + i), bb = ld4<float>(b2 + i);
      f32x4 o;
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = (a[j] - mean) * inv * ww[j] + bb[j];
      st4<O>(out + t * W + i, o);
    }
  } else {
    for (int i = threadIdx.x; i < W; i += NT) stf<O>(out + t * W + i, (sh[i] - mean) * inv * w2[i] + b2[i]);
  }
}

// o: `parts` planes of partial sums [parts][T][N] (the scan cuts the state rows into parts); the row is their sum
template <typename G, typename O>
__global__ __launch_bounds__(NT) void rms_gate_kernel(const float* __restrict__ o, int parts, int64_t part_stride,
                                                      const float* __restrict__ w, float eps, const G* __restrict__ gate,
                                                      int64_t gate_stride, int N, O* __restrict__ out, int groups, int silu) {
  extern __shared__ float sh[];
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  float s = 0.f;
  for (int i = threadIdx.x; i < N; i += NT) {
    float v = o[t * N + i];
    for (int p = 1; p < parts; ++p) v += o[p * part_stride + t * N + i];
    sh[i] = v;
    s += v * v;
  }
  if (groups <= 1) {
    const float inv = 1.f / sqrtf(block_sum<NT>(s, red) / (float)N + eps);
    for (int i = threadIdx.x; i < N; i += NT) {
      const float g = ldf<G>(gate + t * gate_stride + i);
      const float a = 1.f / (1.f + expf(-g));
      stf<O>(out + t * N + i, sh[i] * inv * (w != nullptr ? w[i] : 1.f) * (silu ? g * a : a));
    }
    return;
  }
  // every slice of N / groups entries has its own statistic: a wave per slice
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int Dg = N / groups;
  for (int gi = wave; gi < groups; gi += NT / 64) {
    const float* row = sh + gi * Dg;
    float q = 0.f;
    for (int i = lane; i < Dg; i += 64) q += row[i] * row[i];
    const float inv = 1.f / sqrtf(wave_sum(q) / (float)Dg + eps);
    for (int i = lane; i < Dg; i += 64) {
      const int c = gi * Dg + i;
      const float g = ldf<G>(gate + t * gate_stride + c);
      const float a = 1.f / (1.f + expf(-g));
      stf<O>(out + t * N + c, row[i] * inv * (w != nullptr ? w[c] : 1.f) * (silu ? g * a : a));
    }
  }
}

template <typename A>
__global__ __launch_bounds__(NT) void relu2_kernel(const A* __restrict__ x, A* __restrict__ out, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x; i < n; i += (int64_t)gridDim.x * NT) {
    const float v = fmaxf(ldf<A>(x + i), 0.f);
    stf<A>(out + i, v * v);
  }
}

template <typename A>
__global__ __launch_bounds__(NT) void softcap_kernel(const A* __restrict__ x, float* __restrict__ out, float cap, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x; i < n; i += (int64_t)gridDim.x * NT)
    out[i] = cap * tanhf(ldf<A>(x + i) / cap);
}

// ------------------------------------------------------------------------------------------------ cache writers
// one workgroup per token; a wave per head vector: unit RMS times weight; q in place, k and v to the token's cache rows
template <typename A>
__global__ __launch_bounds__(NT) void qk_norm_cache_kernel(A* __restrict__ qkv, int64_t row_stride,
                                                           const float* __restrict__ qw, const float* __restrict__ kw,
                                                           float eps, const int* __restrict__ slot_mapping,
                                                           A* __restrict__ k_cache, A* __restrict__ v_cache, int H, int G,
                                                           int D, int Dv) {
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int slot = slot_mapping[t];
  A* row = qkv + t * row_stride;
  for (int u = wave; u < H + G; u += NT / 64) {
    A* p = row + (int64_t)u * D;
    float ss = 0.f;
    for (int i = lane; i < D; i += 64) {
      const float v = ldf<A>(p + i);
      ss += v * v;
    }
    const float inv = 1.f / sqrtf(wave_sum(ss) / (float)D + eps);
    if (u < H) {
      for (int i = lane; i < D; i += 64) stf<A>(p + i, ldf<A>(p + i) * inv * qw[i]);
    } else if (slot >= 0) {
      A* dst = k_cache + ((int64_t)slot * G + (u - H)) * D;
      for (int i = lane; i < D; i += 64) stf<A>(dst + i, ldf<A>(p + i) * inv * kw[i]);
    }
  }
  if (slot >= 0) {
    const A* v = row + (int64_t)(H + G) * D;
    A* dst = v_cache + (int64_t)slot * G * Dv;
    for (int i = threadIdx.x; i < G * Dv; i += NT) dst[i] = v[i];
  }
}

// latent attention: cache row = [unit-RMS latent * cw | rotated shared key]; the rotated part of every q head in place
template <typename A>
__global__ __launch_bounds__(NT) void latent_prep_kernel(A* __restrict__ q, int64_t q_stride, const A* __restrict__ dkv,
                                                         int64_t dkv_stride, const float* __restrict__ cw, float eps,
                                                         const int* __restrict__ positions, const double* __restrict__ inv_freq,
                                                         int rot_dims, const int* __restrict__ slot_mapping,
                                                         A* __restrict__ cache, int H, int D, int R, int C) {
  extern __shared__ float sh[];          // cos[rot_dims/2], sin[rot_dims/2]
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const int slot = slot_mapping[t];
  const int half = rot_dims >> 1;
  const double pos = (double)positions[t];
  for (int i = threadIdx.x; i < half; i += NT) {
    double a = pos * inv_freq[i];
    a -= 6.283185307179586476925 * floor(a * 0.15915494309189533577);    // reduced in double, then exact enough in fp32
    double sn, cs;
    sincos(a, &sn, &cs);
    sh[i] = (float)cs;
    sh[half + i] = (float)sn;
  }
  const A* crow = dkv + t * dkv_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < C; i += NT) {
    const float v = ldf<A>(crow + i);
    ss += v * v;
  }
  const float inv = 1.f / sqrtf(block_sum<NT>(ss, red) / (float)C + eps);      // (block_sum's barriers also publish sh)
  A* dst = cache + (int64_t)slot * (C + R);
  if (slot >= 0) {
    for (int i = threadIdx.x; i < C; i += NT) stf<A>(dst + i, ldf<A>(crow + i) * inv * cw[i]);
    for (int i = threadIdx.x; i < R; i += NT) {
      float v = ldf<A>(crow + C + i);
      if (i < rot_dims) {
        const int pr = i >> 1;
        const float o = ldf<A>(crow + C + (i ^ 1));
        v = (i & 1) ? v * sh[pr] + o * sh[half + pr] : v * sh[pr] - o * sh[half + pr];
      }
      stf<A>(dst + C + i, v);
    }
  }
  // q heads: one pair per thread and trip (both entries read before either is written)
  A* qrow = q + t * q_stride;
  for (int idx = threadIdx.x; idx < H * half; idx += NT) {
    const int h = idx / half, pr = idx - h * half;
    A* p = qrow + (int64_t)h * (D + R) + D + 2 * pr;
    const float u = ldf<A>(p), v = ldf<A>(p + 1);
    stf<A>(p, u * sh[pr] - v * sh[half + pr]);
    stf<A>(p + 1, v * sh[pr] + u * sh[half + pr]);
  }
}

// ------------------------------------------------------------------------------------------------ attention
// VPL contiguous elements of a cache row → fp32 (one wide load when the row allows it)
template <typename A, int VPL>
__device__ __forceinline__ void load_vals(const A* __restrict__ p, bool wide, float* __restrict__ dst);
template <int VPL>
__device__ __forceinline__ void load_vals_f32(const float* __restrict__ p, bool wide, float* __restrict__ dst) {
  if (wide && VPL >= 4) {
#pragma unroll
    for (int i = 0; i < VPL; i += 4) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(p + i);
      dst[i] = v[0]; dst[i + 1] = v[1]; dst[i + 2] = v[2]; dst[i + 3] = v[3];
    }
  } else if (wide && VPL == 2) {
    const f32x2 v = *reinterpret_cast<const f32x2*>(p);
    dst[0] = v[0]; dst[1] = v[1];
  } else {
#pragma unroll
    for (int i = 0; i < VPL; ++i) dst[i] = p[i];
  }
}
template <int VPL>
__device__ __forceinline__ void load_vals_bf16(const uint16_t* __restrict__ p, bool wide, float* __restrict__ dst) {
  if (wide && VPL == 8) {
    const bf16x8 v = *reinterpret_cast<const bf16x8*>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) dst[i] = bf2f((uint16_t)v[i]);
  } else if (wide && VPL == 4) {
    const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) dst[i] = bf2f((uint16_t)v[i]);
  } else if (wide && VPL == 2) {
    const uint32_t v = *reinterpret_cast<const uint32_t*>(p);
    dst[0] = __uint_as_float(v << 16);
    dst[1] = __uint_as_float(v & 0xffff0000u);
  } else {
#pragma unroll
    for (int i = 0; i < VPL; ++i) dst[i] = bf2f(p[i]);
  }
}
template <> __device__ __forceinline__ void load_vals<float, 1>(const float* p, bool w, float* d) { load_vals_f32<1>(p, w, d); }
template <> __device__ __forceinline__ void load_vals<float, 2>(const float* p, bool w, float* d) { load_vals_f32<2>(p, w, d); }
template <> __device__ __forceinline__ void load_vals<float, 4>(const float* p, bool w, float* d) { load_vals_f32<4>(p, w, d); }
template <> __device__ __forceinline__ void load_vals<float, 8>(const float* p, bool w, float* d) { load_vals_f32<8>(p, w, d); }
template <> __device__ __forceinline__ void load_vals<uint16_t, 1>(const uint16_t* p, bool w, float* d) { load_vals_bf16<1>(p, w, d); }
template <> __device__ __forceinline__ void load_vals<uint16_t, 2>(const uint16_t* p, bool w, float* d) { load_vals_bf16<2>(p, w, d); }
template <> __device__ __forceinline__ void load_vals<uint16_t, 4>(const uint16_t* p, bool w, float* d) { load_vals_bf16<4>(p, w, d); }
template <> __device__ __forceinline__ void load_vals<uint16_t, 8>(const uint16_t* p, bool w, float* d) { load_vals_bf16<8>(p, w, d); }

// One workgroup per (token, group of HG query heads that read the same key / value head): a key row and a value row are
// loaded once for the HG heads.  Every wave takes chunks of 64 consecutive keys: a lane per key for the scores (the HG
// queries broadcast from LDS, the key row in 16-byte pieces), then lanes over the value columns for P·V — lane owns the
// VPL contiguous columns lane·VPL …, one wide load per key, the key's weight and cache row broadcast as scalars
// (v_readlane).  Online softmax per wave and head, the four waves merged through LDS.  Serves decode rows and
// prefill-chunk tokens alike: a token's position and batch row come from the step metadata, keys from the sequence's
// block-table row.  Value sizes up to 64·VPL.
template <typename A, int VPL, int HG>
__global__ __launch_bounds__(NT) void token_attention_kernel(
    A* __restrict__ out, int64_t o_ts, int64_t o_hs, const A* __restrict__ q1, int64_t q1_ts, int64_t q1_hs, int D1,
    const A* __restrict__ q2, int64_t q2_ts, int64_t q2_hs, int D2, const A* __restrict__ kc, int rowk,
    const A* __restrict__ vc, int rowv, int vhead, int Dv, const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ positions, const int* __restrict__ token_seq, int H, int G, float scale, int window,
    const float* __restrict__ temp, const float* __restrict__ r1, const float* __restrict__ r2, int nsplit,
    float* __restrict__ part, const A* __restrict__ gate, int64_t g_ts, const float* __restrict__ sink) {
  extern __shared__ float sh[];          // q [HG][Dk] | acc [4 waves][HG][Dv] | m [4][HG] | l [4][HG]
  constexpr int NW = NT / 64;
  const int64_t t = blockIdx.x;
  const int h0 = blockIdx.y * HG;        // first head of the group (all HG heads share one key / value head)
  const int seq = token_seq[t];
  if (seq < 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int Dk = D1 + D2;
  const int p = positions[t];
  const int lo = window > 0 ? max(p - window + 1, 0) : 0;
  const int g = h0 / (H / G);
  float* qs = sh;
  float* accs = sh + HG * Dk;
  float* ms = accs + NW * HG * Dv;
  float* ls = ms + NW * HG;
  for (int i = threadIdx.x; i < HG * Dk; i += NT) {
    const int hh = i / Dk, d = i - hh * Dk, h = h0 + hh;
    const float qmul = scale * (temp != nullptr ? temp[h] : 1.f);
    qs[i] = qmul * (d < D1 ? ldf<A>(q1 + t * q1_ts + h * q1_hs + d) : ldf<A>(q2 + t * q2_ts + h * q2_hs + (d - D1)));
  }
  __syncthreads();
  const bool pen = r1 != nullptr;
  float r1h[HG], r2h[HG];
#pragma unroll
  for (int hh = 0; hh < HG; ++hh) {
    r1h[hh] = pen ? r1[h0 + hh] : 0.f;
    r2h[hh] = pen ? r2[h0 + hh] : 0.f;
  }
  const int* bt = block_tables + (int64_t)seq * max_blocks;
  constexpr int esz = sizeof(A);
  const bool kwide = (Dk * esz) % 16 == 0 && (rowk * esz) % 16 == 0 && (reinterpret_cast<uintptr_t>(kc) & 15) == 0;
  const bool vwide = ((int64_t)rowv * esz) % (VPL * esz) == 0 && ((int64_t)vhead * esz) % (VPL * esz) == 0 &&
                     (reinterpret_cast<uintptr_t>(vc) % (VPL * esz)) == 0 && Dv % VPL == 0;
  const int e0 = lane * VPL;             // this lane's value columns

  float m[HG], l[HG], acc[HG][VPL];
#pragma unroll
  for (int hh = 0; hh < HG; ++hh) {
    m[hh] = -INFINITY;
    l[hh] = 0.f;
#pragma unroll
    for (int v = 0; v < VPL; ++v) acc[hh][v] = 0.f;
  }

  // gridDim.z = nsplit workgroups share a long key range: each takes a contiguous run of 64-key chunks and leaves
  // (max, sum, unnormalised output) in `part`; token_attention_merge_kernel combines them
  const int nchunks = (p - lo + 64) >> 6;
  const int per_split = (nchunks + nsplit - 1) / nsplit;
  const int c_begin = blockIdx.z * per_split, c_end = min(c_begin + per_split, nchunks);
  for (int ci = c_begin + wave; ci < c_end; ci += NW) {
    const int base = lo + ci * 64;
    const int j = base + lane;
    const bool valid = j <= p;
    int slot = 0;
    float s[HG];
#pragma unroll
    for (int hh = 0; hh < HG; ++hh) s[hh] = 0.f;
    if (valid) {
      slot = bt[j / kBlockTokens] * kBlockTokens + (j % kBlockTokens);
      const A* kr = kc + (int64_t)slot * rowk + g * Dk;
      constexpr int KV = 16 / esz;       // elements per 16-byte piece
      int i = 0;
      if (kwide) {
        for (; i + 2 * KV <= Dk; i += 2 * KV) {          // two 16-byte pieces in flight
          float kv[2][KV];
#pragma unroll
          for (int c4 = 0; c4 < 2; ++c4) load_vals<A, KV == 8 ? 8 : 4>(kr + i + c4 * KV, true, kv[c4]);
#pragma unroll
          for (int hh = 0; hh < HG; ++hh) {
            float d = 0.f;
#pragma unroll
            for (int c4 = 0; c4 < 2; ++c4)
#pragma unroll
              for (int u = 0; u < KV; ++u) d += qs[hh * Dk + i + c4 * KV + u] * kv[c4][u];
            s[hh] += d;
          }
        }
        for (; i + KV <= Dk; i += KV) {
          float kv[KV];
          load_vals<A, KV == 8 ? 8 : 4>(kr + i, true, kv);
#pragma unroll
          for (int hh = 0; hh < HG; ++hh) {
            float d = 0.f;
#pragma unroll
            for (int u = 0; u < KV; ++u) d += qs[hh * Dk + i + u] * kv[u];
            s[hh] += d;
          }
        }
      }
      for (; i < Dk; ++i) {
        const float kv = ldf<A>(kr + i);
#pragma unroll
        for (int hh = 0; hh < HG; ++hh) s[hh] += qs[hh * Dk + i] * kv;
      }
    }
    float pl[HG];
#pragma unroll
    for (int hh = 0; hh < HG; ++hh) {
      float sv = -INFINITY;
      if (valid) sv = pen ? s[hh] - r1h[hh] * log1pf(r2h[hh] * (float)(p - j)) : s[hh];
      const float mn = fmaxf(m[hh], wave_max(sv));
      const float corr = expf(m[hh] - mn);             // first chunk: exp(-inf) = 0
      pl[hh] = valid ? expf(sv - mn) : 0.f;
      l[hh] = l[hh] * corr + wave_sum(pl[hh]);
      m[hh] = mn;
#pragma unroll
      for (int v = 0; v < VPL; ++v) acc[hh][v] *= corr;
    }
    const int nvalid = min(p - base + 1, 64);
    if (e0 < Dv) {
      int jj = 0;
      if (vwide) {
        constexpr int UB = VPL >= 8 ? 2 : (VPL >= 4 ? 4 : 8);   // value rows fetched together
        for (; jj + UB <= nvalid; jj += UB) {
          float vv[UB][VPL];
#pragma unroll
          for (int u = 0; u < UB; ++u) {
            const int sj = __builtin_amdgcn_readlane(slot, jj + u);
            load_vals<A, VPL>(vc + (int64_t)sj * rowv + g * vhead + e0, true, vv[u]);
          }
#pragma unroll
          for (int u = 0; u < UB; ++u)
#pragma unroll
            for (int hh = 0; hh < HG; ++hh) {
              const float pj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(pl[hh]), jj + u));
#pragma unroll
              for (int v = 0; v < VPL; ++v) acc[hh][v] += pj * vv[u][v];
            }
        }
      }
      for (; jj < nvalid; ++jj) {
        const int sj = __builtin_amdgcn_readlane(slot, jj);
        float vv[VPL];
        const A* vr = vc + (int64_t)sj * rowv + g * vhead + e0;
        if (vwide) {
          load_vals<A, VPL>(vr, true, vv);
        } else {
#pragma unroll
          for (int v = 0; v < VPL; ++v) vv[v] = e0 + v < Dv ? ldf<A>(vr + v) : 0.f;
        }
#pragma unroll
        for (int hh = 0; hh < HG; ++hh) {
          const float pj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(pl[hh]), jj));
#pragma unroll
          for (int v = 0; v < VPL; ++v) acc[hh][v] += pj * vv[v];
        }
      }
    }
  }
#pragma unroll
  for (int hh = 0; hh < HG; ++hh) {
#pragma unroll
    for (int v = 0; v < VPL; ++v)
      if (e0 + v < Dv) accs[(wave * HG + hh) * Dv + e0 + v] = acc[hh][v];
    if (lane == 0) {
      ms[wave * HG + hh] = m[hh];
      ls[wave * HG + hh] = l[hh];
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < HG * Dv; i += NT) {
    const int hh = i / Dv, e = i - hh * Dv;
    float M = ms[hh];
#pragma unroll
    for (int w = 1; w < NW; ++w) M = fmaxf(M, ms[w * HG + hh]);
    float L = 0.f, o = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float f = M == -INFINITY ? 0.f : expf(ms[w * HG + hh] - M);     // a split without keys: all waves empty
      L += f * ls[w * HG + hh];
      o += f * accs[(w * HG + hh) * Dv + e];
    }
    if (nsplit == 1) {
      const float gm = gate != nullptr ? 1.f / (1.f + expf(-ldf<A>(gate + t * g_ts + h0 + hh))) : 1.f;
      if (sink != nullptr) L += expf(sink[h0 + hh] - M);            // a logit without key or value in the denominator
      stf<A>(out + t * o_ts + (h0 + hh) * o_hs + e, o / L * gm);
    } else {
      float* pr = part + ((t * H + (h0 + hh)) * nsplit + blockIdx.z) * (int64_t)(Dv + 2);
      pr[2 + e] = o;
      if (e == 0) {
        pr[0] = M;
        pr[1] = L;
      }
    }
  }
}

// combine the nsplit (≤ 16) partial results of a (token, head): part [T][H][nsplit][2 + Dv] = (max, sum, unnormalised output)
template <typename A>
__global__ __launch_bounds__(128) void token_attention_merge_kernel(A* __restrict__ out, int64_t o_ts, int64_t o_hs,
                                                                    const float* __restrict__ part,
                                                                    const int* __restrict__ token_seq, int H, int Dv,
                                                                    int nsplit, const A* __restrict__ gate, int64_t g_ts, const float* __restrict__ sink) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  if (token_seq[t] < 0) return;
  const float* pr = part + (t * H + h) * nsplit * (int64_t)(Dv + 2);
  float M = -INFINITY;
  for (int z = 0; z < nsplit; ++z) M = fmaxf(M, pr[z * (Dv + 2)]);
  float f[16];
  float L = 0.f;
#pragma unroll
  for (int z = 0; z < 16; ++z) {
    const float mz = z < nsplit ? pr[z * (Dv + 2)] : -INFINITY;
    f[z] = mz == -INFINITY ? 0.f : expf(mz - M);
    if (z < nsplit) L += f[z] * pr[z * (Dv + 2) + 1];
  }
  if (sink != nullptr) L += expf(sink[h] - M);
  const float rl = (gate != nullptr ? 1.f / (1.f + expf(-ldf<A>(gate + t * g_ts + h))) : 1.f) / L;
  for (int e = threadIdx.x; e < Dv; e += 128) {
    float o = 0.f;
#pragma unroll
    for (int z = 0; z < 16; ++z)
      if (z < nsplit) o += f[z] * pr[z * (Dv + 2) + 2 + e];
    stf<A>(out + t * o_ts + h * o_hs + e, o * rl);
  }
}

// ------------------------------------------------------------------------------------------------ attention, prefill tiles
// bf16 only.  One workgroup per (64-query tile of one sequence's chunk, query head); a wave owns 16 queries.  Per 32-key
// page: the page's key rows (this head's slice) and its value rows, transposed, are staged in LDS once for the four
// waves; Sᵀ = K·Qᵀ on v_mfma_f32_16x16x32_bf16 (K rows and the register-resident Q rows are both contiguous 16-byte
// fragments of token-major rows), scale / temperature / distance penalty / window and causal masks and the online
// softmax in fp32 on the accumulators, then Oᵀ += Vᵀ·Pᵀ with the fp32 weights split into a bf16 head and a bf16
// remainder (two MFMAs: P enters the product with 16 mantissa bits, not 8).  The lane's eight Sᵀ values (two 16-key
// tiles) are, in register order, the B fragment of the P·V k-step when the staged V columns sit in the slot order
// slot(t) = ((t & 15) >> 2)·8 + (t >> 4)·4 + (t & 3).  KSMAX / MTMAX: compile-time bounds of ceil(Dk / 32) and Dv / 16.
template <int KSMAX, int MTMAX, int HW>
__global__ __launch_bounds__(NT * HW) void tile_attention_kernel(
    uint16_t* __restrict__ out, int64_t o_ts, int64_t o_hs, const uint16_t* __restrict__ q1, int64_t q1_ts, int64_t q1_hs, int D1,
    const uint16_t* __restrict__ q2, int64_t q2_ts, int64_t q2_hs, int D2, const uint16_t* __restrict__ kc, int rowk,
    const uint16_t* __restrict__ vc, int rowv, int vhead, int Dv, const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ seq_lens, const int* __restrict__ qsl, const int* __restrict__ tile_seq,
    const int* __restrict__ tile_q0, int num_tiles, const int* __restrict__ counts, int H, int G, float scale, int window,
    const float* __restrict__ temp, const float* __restrict__ r1, const float* __restrict__ r2,
    const uint16_t* __restrict__ gate, int64_t g_ts, const float* __restrict__ sink) {
  extern __shared__ __align__(16) uint16_t tl[];
  const int ntiles = counts != nullptr ? min(counts[2], num_tiles) : num_tiles;
  // the host walks causal tiles longest-first from the END of the list
  const int tile = num_tiles - 1 - (int)blockIdx.x;
  if (tile >= ntiles) return;
  // HW heads of one key / value group per workgroup (4 waves each): the staged page serves all of them
  constexpr int TNT = NT * HW;
  const int wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int h = blockIdx.y * HW + (wave_all >> 2);
  const int seq = tile_seq[tile], q0 = tile_q0[tile];
  const int t_begin = qsl[seq];
  const int n_chunk = qsl[seq + 1] - t_begin;
  const int p0 = seq_lens[seq] - n_chunk;                 // position of the chunk's first token
  const int nq = min(64, n_chunk - q0);
  if (nq <= 0) return;
  const int wave = wave_all & 3;
  const int lane = threadIdx.x & 63, g4 = lane >> 4, c = lane & 15;
  const int Dk = D1 + D2;
  const int KS = (Dk + 31) >> 5, MT = Dv >> 4;
  const int KST = KS * 32 + 8;                            // LDS row strides (elements): +16 bytes against bank conflicts
  constexpr int VST = 40;
  uint16_t* Ks = tl;
  uint16_t* Vt = tl + 32 * KST;
  const int g = h / (H / G);

  // zero the K padding columns once (Dk not a multiple of 32): they are never staged over
  for (int i = threadIdx.x; i < 32 * (KS * 32 - Dk); i += TNT) {
    const int row = i / (KS * 32 - Dk), col = Dk + i % (KS * 32 - Dk);
    Ks[row * KST + col] = 0;
  }

  // this lane's query row as B fragments (zero past Dk and for rows past the tile)
  const int qi = 16 * wave + c;
  const bool qvalid = qi < nq;
  const int64_t tq = t_begin + q0 + qi;
  bf16x8 qf[KSMAX];
#pragma unroll
  for (int s = 0; s < KSMAX; ++s) {
    const int d = 32 * s + 8 * g4;
    bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (s < KS && qvalid && d < Dk)
      v = d < D1 ? *reinterpret_cast<const bf16x8*>(q1 + tq * q1_ts + h * q1_hs + d)
                 : *reinterpret_cast<const bf16x8*>(q2 + tq * q2_ts + h * q2_hs + (d - D1));
    qf[s] = v;
  }
  // scores are kept in the log2 domain: s·log2(e) − r1·log2(1 + r2·distance), weights 2^(s − max) — one v_exp_f32 and one
  // v_log_f32 per score (this kernel is bound by the per-score vector arithmetic, not by the matrix cores; its results are
  // rounded to bf16 anyway: the fp32 model never takes this path)
  const float qmul = scale * (temp != nullptr ? temp[h] : 1.f) * 1.4426950408889634f;
  const float r1h = r1 != nullptr ? r1[h] : 0.f, r2h = r1 != nullptr ? r2[h] : 0.f;
  const bool pen = r1h != 0.f;
  const int pq = p0 + q0 + qi;                            // this lane's query position
  const int p_first = p0 + q0, p_last = p0 + q0 + nq - 1;
  const int kb_lo = (window > 0 ? max(p_first - window + 1, 0) : 0) >> 5, kb_hi = p_last >> 5;
  const int* bt = block_tables + (int64_t)seq * max_blocks;

  float m = -INFINITY, l = 0.f;
  f32x4 acc[MTMAX];
#pragma unroll
  for (int i = 0; i < MTMAX; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int kchunks = Dk >> 3, vchunks = Dv >> 3;
  const bool vfromk = vc == kc && rowv == rowk && vhead == Dk;     // latent attention: one row is key and value
  for (int kb = kb_lo; kb <= kb_hi; ++kb) {
    __syncthreads();                                      // everyone is done with the previous page
    const int64_t page_row = (int64_t)bt[kb] * kBlockTokens;
    for (int i = threadIdx.x; i < 32 * kchunks; i += TNT) {
      const int row = i / kchunks, ch = i - row * kchunks;
      *reinterpret_cast<bf16x8*>(Ks + row * KST + 8 * ch) =
          *reinterpret_cast<const bf16x8*>(kc + (page_row + row) * rowk + g * Dk + 8 * ch);
    }
    if (vfromk) __syncthreads();                          // values = leading columns of the key rows just staged
    for (int i = threadIdx.x; i < 32 * vchunks; i += TNT) {
      const int row = i & 31, ch = i >> 5;
      const bf16x8 v = vfromk ? *reinterpret_cast<const bf16x8*>(Ks + row * KST + 8 * ch)
                              : *reinterpret_cast<const bf16x8*>(vc + (page_row + row) * rowv + g * vhead + 8 * ch);
      const int slot = ((row & 15) >> 2) * 8 + (row >> 4) * 4 + (row & 3);
#pragma unroll
      for (int j = 0; j < 8; ++j) Vt[(8 * ch + j) * VST + slot] = (uint16_t)v[j];
    }
    __syncthreads();

    f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KSMAX; ++s) {
      if (s < KS) {
        const bf16x8 ka = *reinterpret_cast<const bf16x8*>(Ks + c * KST + 32 * s + 8 * g4);
        const bf16x8 kb2 = *reinterpret_cast<const bf16x8*>(Ks + (16 + c) * KST + 32 * s + 8 * g4);
        sa = mfma16(ka, qf[s], sa);
        sb = mfma16(kb2, qf[s], sb);
      }
    }
    float sv[8];
    float mx = -INFINITY;
    // a page every query of the tile sees whole (the common case far from the diagonal) needs no per-score masks
    const bool whole = nq == 64 && 32 * kb + 31 <= p_first && (window <= 0 || 32 * kb > p_last - window);
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int j = 32 * kb + (r < 4 ? 4 * g4 + r : 16 + 4 * g4 + (r - 4));
      float v = (r < 4 ? sa[r] : sb[r - 4]) * qmul;
      if (pen) v -= r1h * __builtin_amdgcn_logf(1.f + r2h * (float)max(pq - j, 0));
      if (!whole) {
        const bool ok = qvalid && j <= pq && (window <= 0 || j > pq - window);
        v = ok ? v : -INFINITY;
      }
      sv[r] = v;
      mx = fmaxf(mx, v);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mn = fmaxf(m, mx);
    const float mu = mn == -INFINITY ? 0.f : mn;          // nothing visible yet: keep everything at zero
    const float corr = fast_exp2(m - mu);
    m = mn;
    bf16x8 ph, plo;
    float ps = 0.f;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const float pv = fast_exp2(sv[r] - mu);
      ps += pv;
      const uint16_t hi = f2bf(pv);
      ph[r] = (short)hi;
      plo[r] = (short)f2bf(pv - bf2f(hi));
    }
    l = l * corr + ps;
#pragma unroll
    for (int i = 0; i < MTMAX; ++i) {
      if (i < MT) {
        const bf16x8 vf = *reinterpret_cast<const bf16x8*>(Vt + (16 * i + c) * VST + 8 * g4);
        f32x4 a = acc[i];
        a[0] *= corr; a[1] *= corr; a[2] *= corr; a[3] *= corr;
        a = mfma16(vf, ph, a);
        acc[i] = mfma16(vf, plo, a);
      }
    }
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!qvalid) return;
  if (sink != nullptr) l += fast_exp2(sink[h] * 1.4426950408889634f - m);
  const float rl = (gate != nullptr ? 1.f / (1.f + expf(-bf2f(gate[tq * g_ts + h]))) : 1.f) / l;
  uint16_t* orow = out + tq * o_ts + h * o_hs;
#pragma unroll
  for (int i = 0; i < MTMAX; ++i) {
    if (i < MT) {
      bf16x4 o;
#pragma unroll
      for (int r = 0; r < 4; ++r) o[r] = (short)f2bf(acc[i][r] * rl);
      *reinterpret_cast<bf16x4*>(orow + 16 * i + 4 * g4) = o;
    }
  }
}

// ------------------------------------------------------------------------------------------------ attention, decode rows, heads as columns
// bf16 only; for mixers whose query heads share a key / value head in groups of 8 or more (latent attention: all of them).
// One workgroup per (token, group of up to 16 heads, slice of the key range): the 16 MFMA columns are the HEADS of one
// token, so a key row fetched once meets every head on the matrix cores.  Pages are staged as in tile_attention_kernel
// (K rows, V transposed into the MFMA slot order); all four waves compute the same Sᵀ = K·Qᵀ tile and online softmax, and
// each accumulates its own quarter of the value columns, so nothing is merged inside the workgroup.  gridDim.z slices of
// the key range leave (max, sum, unnormalised output) in `part` for token_attention_merge_kernel.
template <int KSMAX, int MTQ>
__global__ __launch_bounds__(NT) void head_decode_attention_kernel(
    uint16_t* __restrict__ out, int64_t o_ts, int64_t o_hs, const uint16_t* __restrict__ q1, int64_t q1_ts, int64_t q1_hs, int D1,
    const uint16_t* __restrict__ q2, int64_t q2_ts, int64_t q2_hs, int D2, const uint16_t* __restrict__ kc, int rowk,
    const uint16_t* __restrict__ vc, int rowv, int vhead, int Dv, const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ positions, const int* __restrict__ token_seq, int H, int G, int groups, float scale, int window,
    const float* __restrict__ temp, const float* __restrict__ r1, const float* __restrict__ r2, int nsplit,
    float* __restrict__ part, const uint16_t* __restrict__ gate, int64_t g_ts, const float* __restrict__ sink) {
  extern __shared__ __align__(16) uint16_t tl[];
  const int64_t t = blockIdx.x;
  const int seq = token_seq[t];
  if (seq < 0) return;
  const int per = H / G;
  const int g = blockIdx.y / groups, grp = blockIdx.y - g * groups;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63, g4 = lane >> 4, c = lane & 15;
  const bool hvalid = 16 * grp + c < per;
  const int h = g * per + min(16 * grp + c, per - 1);
  const int Dk = D1 + D2;
  const int KS = (Dk + 31) >> 5, MT = Dv >> 4;
  const int MTW = (MT + 3) >> 2;                         // value tiles per wave
  const int KST = KS * 32 + 8;
  constexpr int VST = 40;
  uint16_t* Ks = tl;
  uint16_t* Vt = tl + 32 * KST;
  for (int i = threadIdx.x; i < 32 * (KS * 32 - Dk); i += NT) {
    const int row = i / (KS * 32 - Dk), col = Dk + i % (KS * 32 - Dk);
    Ks[row * KST + col] = 0;
  }
  bf16x8 qf[KSMAX];
#pragma unroll
  for (int s = 0; s < KSMAX; ++s) {
    const int d = 32 * s + 8 * g4;
    bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (s < KS && hvalid && d < Dk)
      v = d < D1 ? *reinterpret_cast<const bf16x8*>(q1 + t * q1_ts + h * q1_hs + d)
                 : *reinterpret_cast<const bf16x8*>(q2 + t * q2_ts + h * q2_hs + (d - D1));
    qf[s] = v;
  }
  const float qmul = scale * (temp != nullptr ? temp[h] : 1.f) * 1.4426950408889634f;     // log2 domain, as in the tile kernel
  const float r1h = r1 != nullptr ? r1[h] : 0.f, r2h = r1 != nullptr ? r2[h] : 0.f;
  const bool pen = r1 != nullptr;
  const int p = positions[t];
  const int lo = window > 0 ? max(p - window + 1, 0) : 0;
  const int kb_lo = lo >> 5, kb_hi = p >> 5;
  const int per_split = (kb_hi - kb_lo + nsplit) / nsplit;
  const int kb_begin = kb_lo + blockIdx.z * per_split, kb_end = min(kb_begin + per_split - 1, kb_hi);
  const int* bt = block_tables + (int64_t)seq * max_blocks;

  float m = -INFINITY, l = 0.f;
  f32x4 acc[MTQ];
#pragma unroll
  for (int i = 0; i < MTQ; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int kchunks = Dk >> 3, vchunks = Dv >> 3;
  const bool vfromk = vc == kc && rowv == rowk && vhead == Dk;     // latent attention: one row is key and value
  for (int kb = kb_begin; kb <= kb_end; ++kb) {
    __syncthreads();
    const int64_t page_row = (int64_t)bt[kb] * kBlockTokens;
    for (int i = threadIdx.x; i < 32 * kchunks; i += NT) {
      const int row = i / kchunks, ch = i - row * kchunks;
      *reinterpret_cast<bf16x8*>(Ks + row * KST + 8 * ch) =
          *reinterpret_cast<const bf16x8*>(kc + (page_row + row) * rowk + g * Dk + 8 * ch);
    }
    if (vfromk) __syncthreads();                          // values = leading columns of the key rows just staged
    for (int i = threadIdx.x; i < 32 * vchunks; i += NT) {
      const int row = i & 31, ch = i >> 5;
      const bf16x8 v = vfromk ? *reinterpret_cast<const bf16x8*>(Ks + row * KST + 8 * ch)
                              : *reinterpret_cast<const bf16x8*>(vc + (page_row + row) * rowv + g * vhead + 8 * ch);
      const int slot = ((row & 15) >> 2) * 8 + (row >> 4) * 4 + (row & 3);
#pragma unroll
      for (int j = 0; j < 8; ++j) Vt[(8 * ch + j) * VST + slot] = (uint16_t)v[j];
    }
    __syncthreads();
    f32x4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < KSMAX; ++s) {
      if (s < KS) {
        const bf16x8 ka = *reinterpret_cast<const bf16x8*>(Ks + c * KST + 32 * s + 8 * g4);
        const bf16x8 kb2 = *reinterpret_cast<const bf16x8*>(Ks + (16 + c) * KST + 32 * s + 8 * g4);
        sa = mfma16(ka, qf[s], sa);
        sb = mfma16(kb2, qf[s], sb);
      }
    }
    float sv[8];
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int j = 32 * kb + (r < 4 ? 4 * g4 + r : 16 + 4 * g4 + (r - 4));
      float v = (r < 4 ? sa[r] : sb[r - 4]) * qmul;
      if (pen) v -= r1h * __builtin_amdgcn_logf(1.f + r2h * (float)max(p - j, 0));
      v = (j >= lo && j <= p) ? v : -INFINITY;
      sv[r] = v;
      mx = fmaxf(mx, v);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mn = fmaxf(m, mx);
    const float mu = mn == -INFINITY ? 0.f : mn;
    const float corr = fast_exp2(m - mu);
    m = mn;
    bf16x8 ph, plo;
    float ps = 0.f;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const float pv = fast_exp2(sv[r] - mu);
      ps += pv;
      const uint16_t hi = f2bf(pv);
      ph[r] = (short)hi;
      plo[r] = (short)f2bf(pv - bf2f(hi));
    }
    l = l * corr + ps;
#pragma unroll
    for (int ii = 0; ii < MTQ; ++ii) {
      const int i = wave * MTW + ii;
      if (ii < MTW && i < MT) {
        const bf16x8 vf = *reinterpret_cast<const bf16x8*>(Vt + (16 * i + c) * VST + 8 * g4);
        f32x4 a = acc[ii];
        a[0] *= corr; a[1] *= corr; a[2] *= corr; a[3] *= corr;
        a = mfma16(vf, ph, a);
        acc[ii] = mfma16(vf, plo, a);
      }
    }
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!hvalid) return;
  if (nsplit == 1) {
    if (sink != nullptr) l += fast_exp2(sink[h] * 1.4426950408889634f - m);
    const float rl = (gate != nullptr ? 1.f / (1.f + expf(-bf2f(gate[t * g_ts + h]))) : 1.f) / l;
    uint16_t* orow = out + t * o_ts + h * o_hs;
#pragma unroll
    for (int ii = 0; ii < MTQ; ++ii) {
      const int i = wave * MTW + ii;
      if (ii < MTW && i < MT) {
        bf16x4 o;
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = (short)f2bf(acc[ii][r] * rl);
        *reinterpret_cast<bf16x4*>(orow + 16 * i + 4 * g4) = o;
      }
    }
  } else {
    // the merge kernel works with natural exponentials: hand it the maximum in that domain
    float* pr = part + ((t * H + h) * nsplit + blockIdx.z) * (int64_t)(Dv + 2);
    if (wave == 0 && g4 == 0) {
      pr[0] = m * 0.6931471805599453f;
      pr[1] = l;
    }
#pragma unroll
    for (int ii = 0; ii < MTQ; ++ii) {
      const int i = wave * MTW + ii;
      if (ii < MTW && i < MT) {
#pragma unroll
        for (int r = 0; r < 4; ++r) pr[2 + 16 * i + 4 * g4 + r] = acc[ii][r];
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------ linear attention
// S ← decay·S + act(k)·act(v)ᵀ, o = Sᵀ act(q), token by token, with S = a [D, Dv] fp32 state per (sequence, head); act is
// silu, or the identity with `plain` (retention: q and k arrive rotated and scaled, in fp32).
// One wave per (work item, head, 64 value columns): lane e keeps column e of the state in registers; the next token's
// q / k / v are fetched while the current one is applied.  DMAX: compile-time bound of D (registers per lane).
//
// A work item is either a whole sequence of the step (MODE 0: decode rows — and every sequence when the step has no
// block list) or one 64-token block of a prefill chunk (the prefill path, three launches so that the blocks of a long
// chunk run side by side instead of one after the other):
//   MODE 1  per block: the block's own contribution L = Σ_j decay^(n-1-j) k_j v_jᵀ (state from zero, no output) → ws[block]
//   prefix  per sequence (lightning_prefix_kernel): walks its blocks in order, leaves in ws[block] the state at the block's
//           START and in the sequence's state slot the state after its last token: S ← decay^n · S + L
//   MODE 2  per block: the recurrence again from ws[block], now with outputs.
// Blocks are the step's prefill tiles (tile_seq / tile_q0, 64 tokens); ws row of a block = (first token >> 6) + batch row
// (unique: rows of later sequences start at later tokens).
template <typename A, int DMAX, int MODE>
__global__ __launch_bounds__(64) void lightning_scan_kernel(const A* __restrict__ qkvg, int64_t row_stride,
                                                            float* __restrict__ state, const int* __restrict__ positions,
                                                            const int* __restrict__ qsl, const int* __restrict__ state_slots,
                                                            const int* __restrict__ counts, int H, int D, int Dv,
                                                            const float* __restrict__ decay, float* __restrict__ out,
                                                            const int* __restrict__ tile_seq, const int* __restrict__ tile_q0,
                                                            int num_tiles, float* __restrict__ ws, int single_only, int zs,
                                                            int DR, int64_t out_part, int plain) {
  __shared__ float qs[2][DMAX], ks[2][DMAX];
  int seq, t0, t1;
  if (MODE == 0) {
    seq = blockIdx.x;
    if (seq >= counts[3]) return;
    t0 = qsl[seq];
    t1 = qsl[seq + 1];
    if (single_only && t1 - t0 != 1) return;             // longer chunks take the block path
  } else {
    const int tile = blockIdx.x;
    if (tile >= min(counts[2], num_tiles)) return;
    seq = tile_seq[tile];
    t0 = qsl[seq] + tile_q0[tile];
    t1 = min(t0 + 64, qsl[seq + 1]);
  }
  const int slot = state_slots[seq];
  if (slot < 0 || t1 <= t0) return;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  // blockIdx.z = (part of the D rows, 64-column slice): this wave owns state rows dbase … dbase + DR - 1 (DR ≤ DMAX); the
  // partial outputs of the parts go to separate planes of `out` and are summed by the consumer (rms_gate_kernel)
  const int part = blockIdx.z / zs;
  const int e = (blockIdx.z - part * zs) * 64 + lane;
  const int dbase = part * DR;
  const int Dn = min(DR, D - dbase);                   // rows of this part
  if (Dn <= 0) return;
  out += part * out_part;
  const bool active = e < Dv;
  const float lam = decay[h];
  float S[DMAX];
  float* srow = (MODE == 0 ? state + ((int64_t)slot * H + h) * D * Dv
                           : ws + ((int64_t)((t0 >> 6) + seq) * H + h) * D * Dv) + (int64_t)dbase * Dv;
  const bool carry = MODE == 0 ? positions[t0] > 0 : MODE == 2;
#pragma unroll
  for (int d = 0; d < DMAX; ++d) S[d] = (carry && active && d < Dn) ? srow[(int64_t)d * Dv + e] : 0.f;

  const int64_t qoff = (int64_t)h * D + dbase, koff = (int64_t)H * D + (int64_t)h * D + dbase,
                voff = 2 * (int64_t)H * D + (int64_t)h * Dv;
  constexpr int PER = (DMAX + 63) / 64;
  float nq[PER], nk[PER], nv = 0.f;
  auto fetch = [&](int t) {
    const A* row = qkvg + (int64_t)t * row_stride;
#pragma unroll
    for (int r = 0; r < PER; ++r) {
      const int i = lane + 64 * r;
      nq[r] = (MODE != 1 && i < Dn) ? ldf<A>(row + qoff + i) : 0.f;
      nk[r] = i < Dn ? ldf<A>(row + koff + i) : 0.f;
    }
    nv = active ? ldf<A>(row + voff + e) : 0.f;
  };
  fetch(t0);
  for (int t = t0; t < t1; ++t) {
    const int buf = (t - t0) & 1;
#pragma unroll
    for (int r = 0; r < PER; ++r) {
      const int i = lane + 64 * r;
      if (i < DMAX) {
        if (MODE != 1) qs[buf][i] = plain ? nq[r] : silu_act<A>(nq[r]);
        ks[buf][i] = plain ? nk[r] : silu_act<A>(nk[r]);
      }
    }
    const float ve = plain ? nv : silu_act<A>(nv);
    if (t + 1 < t1) fetch(t + 1);
    __syncthreads();                       // one wave: publishes qs / ks of this token (the other buffer is being refilled next trip)
    float o = 0.f;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
      if (d < Dn) {
        S[d] = lam * S[d] + ks[buf][d] * ve;
        if (MODE != 1) o += S[d] * qs[buf][d];
      }
    }
    if (MODE != 1 && active) out[(int64_t)t * H * Dv + (int64_t)h * Dv + e] = o;
  }
  if (MODE != 2 && active) {
#pragma unroll
    for (int d = 0; d < DMAX; ++d)
      if (d < Dn) srow[(int64_t)d * Dv + e] = S[d];
  }
}

// per (sequence with a chunk of two tokens or more, head, 64 value columns): see above
__global__ __launch_bounds__(64) void lightning_prefix_kernel(float* __restrict__ state, float* __restrict__ ws,
                                                              const int* __restrict__ positions, const int* __restrict__ qsl,
                                                              const int* __restrict__ state_slots, const int* __restrict__ counts,
                                                              int H, int D, int Dv, const float* __restrict__ decay) {
  const int seq = blockIdx.x;
  if (seq >= counts[3]) return;
  const int t0 = qsl[seq], n = qsl[seq + 1] - t0;
  const int slot = state_slots[seq];
  if (slot < 0 || n < 2) return;
  const int h = blockIdx.y;
  const int zs = (Dv + 63) >> 6;
  const int d = blockIdx.z / zs;                       // grid.z = D · (64-column slices): the walk over blocks is per state row
  const int e = (blockIdx.z - d * zs) * 64 + threadIdx.x;
  if (e >= Dv) return;
  const float lam = decay[h];
  float lam64 = lam;
#pragma unroll
  for (int i = 0; i < 6; ++i) lam64 *= lam64;
  const int rest = n & 63;
  float lamr = 1.f;
  for (int i = 0; i < rest; ++i) lamr *= lam;
  const bool carry = positions[t0] > 0;
  const int blocks = (n + 63) >> 6;
  float* srow = state + (((int64_t)slot * H + h) * D + d) * Dv + e;
  float run = carry ? *srow : 0.f;
  for (int i = 0; i < blocks; ++i) {
    float* w = ws + (((int64_t)(((t0 + 64 * i) >> 6) + seq) * H + h) * D + d) * Dv + e;
    const float own = *w;
    *w = run;
    run = ((i == blocks - 1 && rest) ? lamr : lam64) * run + own;
  }
  *srow = run;
}

}  // namespace

// ================================================================================================ launchers
#define SM_DISPATCH_BF16(flag, T, ...) \
  do {                                 \
    if (flag) {                        \
      using T = uint16_t;              \
      __VA_ARGS__;                     \
    } else {                           \
      using T = float;                 \
      __VA_ARGS__;                     \
    }                                  \
  } while (0)

void launch_sm_layer_norm(const float* x, const float* w, const float* b, float eps, int rows, int W, void* out, bool out_bf16,
                          hipStream_t stream) {
  if (rows == 0) return;
  SM_DISPATCH_BF16(out_bf16, O, hipLaunchKernelGGL(layer_norm_kernel<O>, dim3(rows), dim3(NT), W * sizeof(float), stream, x, w, b,
                                                   eps, W, (O*)out));
}

void launch_sm_ln_shift(const float* x, const float* add, float* xout, const float* w, const float* b, const float* mix,
                        float* state, const int* positions, const int* token_seq, const int* qsl, const int* state_slots,
                        const int* counts, int rows, int seqs, float eps, int W, void* out, bool out_bf16, hipStream_t stream) {
  if (rows == 0) return;
  SM_DISPATCH_BF16(out_bf16, O, hipLaunchKernelGGL(ln_shift_kernel<O>, dim3(rows), dim3(NT), 2 * W * sizeof(float), stream, x, add,
                                                   xout, w, b, mix, (const float*)state, positions, token_seq, qsl, state_slots,
                                                   eps, W, (O*)out));
  if (seqs > 0)
    hipLaunchKernelGGL(ln_state_kernel, dim3(seqs), dim3(NT), W * sizeof(float), stream, x, add, w, b, state, qsl, state_slots,
                       counts, eps, W);
}

void launch_sm_add_ln(float* x, const void* y, bool y_bf16, int64_t y_stride, const float* w1, const float* b1, float mult,
                      const float* w2, const float* b2, float eps, int rows, int W, void* out, bool out_bf16,
                      hipStream_t stream) {
  if (rows == 0) return;
  SM_DISPATCH_BF16(y_bf16, Y, SM_DISPATCH_BF16(out_bf16, O, hipLaunchKernelGGL((add_ln_kernel<Y, O>), dim3(rows), dim3(NT),
                                                                                W * sizeof(float), stream, x, (const Y*)y,
                                                                                y_stride, w1, b1, mult, w2, b2, eps, W, (O*)out)));
}

void launch_sm_rms_gate(const float* o, int parts, const float* w, float eps, const void* gate, bool gate_bf16, int64_t gate_stride,
                        int rows, int N, void* out, bool out_bf16, int groups, bool silu, hipStream_t stream) {
  if (rows == 0) return;
  const int64_t ps = (int64_t)rows * N;
  SM_DISPATCH_BF16(gate_bf16, G, SM_DISPATCH_BF16(out_bf16, O, hipLaunchKernelGGL((rms_gate_kernel<G, O>), dim3(rows), dim3(NT),
                                                                                   N * sizeof(float), stream, o, parts, ps, w, eps,
                                                                                   (const G*)gate, gate_stride, N, (O*)out, groups,
                                                                                   silu ? 1 : 0)));
}

void launch_sm_relu2(const void* x, void* out, int64_t n, bool bf16, hipStream_t stream) {
  if (n == 0) return;
  const int blocks = (int)std::min<int64_t>((n + NT - 1) / NT, 4096);
  SM_DISPATCH_BF16(bf16, A, hipLaunchKernelGGL(relu2_kernel<A>, dim3(blocks), dim3(NT), 0, stream, (const A*)x, (A*)out, n));
}

void launch_sm_softcap(const void* x, bool bf16, float* out, float cap, int64_t n, hipStream_t stream) {
  if (n == 0) return;
  const int blocks = (int)std::min<int64_t>((n + NT - 1) / NT, 4096);
  SM_DISPATCH_BF16(bf16, A, hipLaunchKernelGGL(softcap_kernel<A>, dim3(blocks), dim3(NT), 0, stream, (const A*)x, out, cap, n));
}

void launch_sm_qk_norm_cache(void* qkv, bool bf16, int64_t row_stride, const float* qw, const float* kw, float eps,
                             const int* slot_mapping, void* k_cache, void* v_cache, int rows, int H, int G, int D, int Dv,
                             hipStream_t stream) {
  if (rows == 0) return;
  SM_DISPATCH_BF16(bf16, A, hipLaunchKernelGGL(qk_norm_cache_kernel<A>, dim3(rows), dim3(NT), 0, stream, (A*)qkv, row_stride, qw, kw,
                                               eps, slot_mapping, (A*)k_cache, (A*)v_cache, H, G, D, Dv));
}

void launch_sm_latent_prep(void* q, bool bf16, int64_t q_stride, const void* dkv, int64_t dkv_stride, const float* cw, float eps,
                           const int* positions, const double* inv_freq, int rot_dims, const int* slot_mapping, void* cache,
                           int rows, int H, int D, int R, int C, hipStream_t stream) {
  if (rows == 0) return;
  SM_DISPATCH_BF16(bf16, A, hipLaunchKernelGGL(latent_prep_kernel<A>, dim3(rows), dim3(NT), std::max(rot_dims, 2) * sizeof(float),
                                               stream, (A*)q, q_stride, (const A*)dkv, dkv_stride, cw, eps, positions, inv_freq,
                                               rot_dims, slot_mapping, (A*)cache, H, D, R, C));
}

template <typename A, int VPL>
static void token_attention_hg(int hg, dim3 grid, size_t lds, hipStream_t stream, A* out, int64_t o_ts, int64_t o_hs, const A* q1,
                               int64_t q1_ts, int64_t q1_hs, int D1, const A* q2, int64_t q2_ts, int64_t q2_hs, int D2, const A* kc,
                               int rowk, const A* vc, int rowv, int vhead, int Dv, const int* bt, int max_blocks, const int* pos,
                               const int* tseq, int H, int G, float scale, int window, const float* temp, const float* r1,
                               const float* r2, int nsplit, float* part, const A* gate, int64_t g_ts, const float* __restrict__ sink) {
#define SM_ATT(HGV)                                                                                                              \
  hipLaunchKernelGGL((token_attention_kernel<A, VPL, HGV>), grid, dim3(NT), lds, stream, out, o_ts, o_hs, q1, q1_ts, q1_hs, D1,  \
                     q2, q2_ts, q2_hs, D2, kc, rowk, vc, rowv, vhead, Dv, bt, max_blocks, pos, tseq, H, G, scale, window, temp,  \
                     r1, r2, nsplit, part, gate, g_ts, sink)
  if (hg == 1) SM_ATT(1);
  else if (hg == 2) SM_ATT(2);
  else SM_ATT(4);
#undef SM_ATT
}

void launch_sm_token_attention(void* out, int64_t o_ts, int64_t o_hs, const void* q1, int64_t q1_ts, int64_t q1_hs, int D1,
                               const void* q2, int64_t q2_ts, int64_t q2_hs, int D2, const void* kc, int rowk, const void* vc,
                               int rowv, int vhead, int Dv, const int* block_tables, int max_blocks, const int* positions,
                               const int* token_seq, int rows, int H, int G, float scale, int window, const float* temp,
                               const float* r1, const float* r2, bool bf16, int nsplit, float* part, const void* gate, int64_t g_ts, const float* sink,
                               hipStream_t stream) {
  if (rows == 0) return;
  if (Dv > 512) {
    // wider values than a lane's 8 columns × 64 lanes: slabs of 512 columns, each a launch of its own (scores recomputed)
    for (int e = 0; e < Dv; e += 512)
      launch_sm_token_attention(bf16 ? (void*)((uint16_t*)out + e) : (void*)((float*)out + e), o_ts, o_hs, q1, q1_ts, q1_hs, D1, q2,
                                q2_ts, q2_hs, D2, kc, rowk, bf16 ? (const void*)((const uint16_t*)vc + e) : (const void*)((const float*)vc + e),
                                rowv, vhead, std::min(512, Dv - e), block_tables, max_blocks, positions, token_seq, rows, H, G, scale,
                                window, temp, r1, r2, bf16, 1, nullptr, gate, g_ts, sink, stream);
    return;
  }
  // heads per workgroup: as many of the heads sharing a key / value head as divide their number and fit the LDS budget
  const int per = H / G, Dk = D1 + D2;
  int hg = per % 4 == 0 ? 4 : (per % 2 == 0 ? 2 : 1);
  auto lds_of = [&](int g) { return (size_t)(g * Dk + (NT / 64) * g * Dv + 2 * (NT / 64) * g) * sizeof(float); };
  while (hg > 1 && lds_of(hg) > 60 * 1024) hg >>= 1;
  const size_t lds = lds_of(hg);
  const dim3 grid(rows, H / hg, nsplit);
  const int nv = (Dv + 63) / 64;
#define SM_ATT_V(VPLV)                                                                                                            \
  SM_DISPATCH_BF16(bf16, A, (token_attention_hg<A, VPLV>(hg, grid, lds, stream, (A*)out, o_ts, o_hs, (const A*)q1, q1_ts, q1_hs, \
                                                         D1, (const A*)q2, q2_ts, q2_hs, D2, (const A*)kc, rowk, (const A*)vc,   \
                                                         rowv, vhead, Dv, block_tables, max_blocks, positions, token_seq, H, G,  \
                                                         scale, window, temp, r1, r2, nsplit, part, (const A*)gate, g_ts, sink)))
  if (nv <= 1) SM_ATT_V(1);
  else if (nv <= 2) SM_ATT_V(2);
  else if (nv <= 4) SM_ATT_V(4);
  else SM_ATT_V(8);
#undef SM_ATT_V
  if (nsplit > 1)
    SM_DISPATCH_BF16(bf16, A, hipLaunchKernelGGL(token_attention_merge_kernel<A>, dim3(rows, H), dim3(128), 0, stream, (A*)out, o_ts,
                                                 o_hs, (const float*)part, token_seq, H, Dv, nsplit, (const A*)gate, g_ts, sink));
}

// workgroups of a per-token attention launch over `rows` tokens: long key ranges are cut so that about 1024 exist
int sm_token_attention_splits(int rows, int H, int G) {
  const int per = H / G;
  const int hg = per % 4 == 0 ? 4 : (per % 2 == 0 ? 2 : 1);
  const int wgs = std::max(rows * (H / hg), 1);
  return std::max(1, std::min(8, 1024 / wgs));
}

// prefill tiles on the matrix cores (bf16; see tile_attention_kernel).  Returns false when the shapes do not fit its
// fragments (the caller then runs the per-token kernel over those rows instead).
bool launch_sm_tile_attention(void* out, int64_t o_ts, int64_t o_hs, const void* q1, int64_t q1_ts, int64_t q1_hs, int D1,
                              const void* q2, int64_t q2_ts, int64_t q2_hs, int D2, const void* kc, int rowk, const void* vc,
                              int rowv, int vhead, int Dv, const int* block_tables, int max_blocks, const int* seq_lens,
                              const int* qsl, const int* tile_seq, const int* tile_q0, int num_tiles, const int* counts, int H,
                              int G, float scale, int window, const float* temp, const float* r1, const float* r2,
                              const void* gate, int64_t g_ts, const float* sink, hipStream_t stream) {
  const int Dk = D1 + D2, KS = (Dk + 31) / 32, MT = Dv / 16;
  auto al = [](const void* p, int64_t a) { return p == nullptr || reinterpret_cast<uintptr_t>(p) % a == 0; };
  const bool ok = D1 % 8 == 0 && D2 % 8 == 0 && Dv % 16 == 0 && KS <= 18 && MT <= 32 && rowk % 8 == 0 && rowv % 8 == 0 &&
                  vhead % 8 == 0 && q1_ts % 8 == 0 && q1_hs % 8 == 0 && q2_ts % 8 == 0 && q2_hs % 8 == 0 && o_ts % 4 == 0 &&
                  o_hs % 4 == 0 && al(out, 8) && al(q1, 16) && al(q2, 16) && al(kc, 16) && al(vc, 16);
  if (!ok) return false;
  if (num_tiles == 0) return true;
  const size_t lds = (size_t)(32 * (KS * 32 + 8) + Dv * 40) * sizeof(uint16_t);
  // two heads of a key / value group per workgroup (8 waves) where the group has an even number of heads
  const int hw = (H / G) % 2 == 0 ? 2 : 1;
  const dim3 grid(num_tiles, H / hw);
#define SM_TILE_HW(KSM, MTM, HWV)                                                                                                \
  do {                                                                                                                           \
    static bool big = false;                                                                                                     \
    if (lds > 48 * 1024 && !big) {                                                                                               \
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&tile_attention_kernel<KSM, MTM, HWV>),                            \
                                hipFuncAttributeMaxDynamicSharedMemorySize, 100 * 1024);                                         \
      big = true;                                                                                                                \
    }                                                                                                                            \
    hipLaunchKernelGGL((tile_attention_kernel<KSM, MTM, HWV>), grid, dim3(NT * HWV), lds, stream, (uint16_t*)out, o_ts, o_hs,    \
                       (const uint16_t*)q1, q1_ts, q1_hs, D1, (const uint16_t*)q2, q2_ts, q2_hs, D2, (const uint16_t*)kc, rowk,  \
                       (const uint16_t*)vc, rowv, vhead, Dv, block_tables, max_blocks, seq_lens, qsl, tile_seq, tile_q0,        \
                       num_tiles, counts, H, G, scale, window, temp, r1, r2, (const uint16_t*)gate, g_ts, sink);                       \
  } while (0)
#define SM_TILE(KSM, MTM)              \
  do {                                 \
    if (hw == 2) SM_TILE_HW(KSM, MTM, 2); \
    else SM_TILE_HW(KSM, MTM, 1);      \
  } while (0)
  if (KS <= 4 && MT <= 8) SM_TILE(4, 8);
  else if (KS <= 8 && MT <= 16) SM_TILE(8, 16);
  else SM_TILE(18, 32);
#undef SM_TILE
#undef SM_TILE_HW
  return true;
}

// decode rows with heads as MFMA columns (bf16; see head_decode_attention_kernel).  False: shapes it does not take.
bool launch_sm_head_decode_attention(void* out, int64_t o_ts, int64_t o_hs, const void* q1, int64_t q1_ts, int64_t q1_hs, int D1,
                                     const void* q2, int64_t q2_ts, int64_t q2_hs, int D2, const void* kc, int rowk, const void* vc,
                                     int rowv, int vhead, int Dv, const int* block_tables, int max_blocks, const int* positions,
                                     const int* token_seq, int rows, int H, int G, float scale, int window, const float* temp,
                                     const float* r1, const float* r2, int nsplit, float* part, const void* gate, int64_t g_ts, const float* sink,
                                     hipStream_t stream) {
  const int Dk = D1 + D2, KS = (Dk + 31) / 32, MT = Dv / 16, per = H / G;
  auto al = [](const void* p, int64_t a) { return p == nullptr || reinterpret_cast<uintptr_t>(p) % a == 0; };
  const bool ok = per >= 8 && D1 % 8 == 0 && D2 % 8 == 0 && Dv % 16 == 0 && KS <= 18 && MT <= 32 && rowk % 8 == 0 && rowv % 8 == 0 &&
                  vhead % 8 == 0 && q1_ts % 8 == 0 && q1_hs % 8 == 0 && q2_ts % 8 == 0 && q2_hs % 8 == 0 && o_ts % 4 == 0 &&
                  o_hs % 4 == 0 && al(out, 8) && al(q1, 16) && al(q2, 16) && al(kc, 16) && al(vc, 16);
  if (!ok) return false;
  if (rows == 0) return true;
  const size_t lds = (size_t)(32 * (KS * 32 + 8) + Dv * 40) * sizeof(uint16_t);
  const int groups = (per + 15) / 16;
  const dim3 grid(rows, G * groups, nsplit);
#define SM_HD(KSM, MTQV)                                                                                                         \
  do {                                                                                                                           \
    static bool big = false;                                                                                                     \
    if (lds > 48 * 1024 && !big) {                                                                                               \
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&head_decode_attention_kernel<KSM, MTQV>),                         \
                                hipFuncAttributeMaxDynamicSharedMemorySize, 100 * 1024);                                         \
      big = true;                                                                                                                \
    }                                                                                                                            \
    hipLaunchKernelGGL((head_decode_attention_kernel<KSM, MTQV>), grid, dim3(NT), lds, stream, (uint16_t*)out, o_ts, o_hs,       \
                       (const uint16_t*)q1, q1_ts, q1_hs, D1, (const uint16_t*)q2, q2_ts, q2_hs, D2, (const uint16_t*)kc, rowk,  \
                       (const uint16_t*)vc, rowv, vhead, Dv, block_tables, max_blocks, positions, token_seq, H, G, groups, scale,\
                       window, temp, r1, r2, nsplit, part, (const uint16_t*)gate, g_ts, sink);                                         \
  } while (0)
  if (KS <= 4 && MT <= 8) SM_HD(4, 2);
  else if (KS <= 8 && MT <= 16) SM_HD(8, 4);
  else SM_HD(18, 8);
#undef SM_HD
  if (nsplit > 1)
    hipLaunchKernelGGL(token_attention_merge_kernel<uint16_t>, dim3(rows, H), dim3(128), 0, stream, (uint16_t*)out, o_ts, o_hs,
                       (const float*)part, token_seq, H, Dv, nsplit, (const uint16_t*)gate, g_ts, sink);
  return true;
}

// slices of the key range for that kernel: about 512 workgroups
int sm_head_decode_splits(int rows, int H, int G) {
  const int per = H / G;
  const int wgs = std::max(rows * G * ((per + 15) / 16), 1);
  return std::max(1, std::min(8, 512 / wgs));
}

// rows of the state one wave keeps: D is cut into parts so that a wave's per-token loop is short and more waves share the work
int sm_lightning_parts(int D) { return D >= 128 ? 4 : (D >= 64 ? 2 : 1); }

void launch_sm_lightning_scan(const void* qkvg, bool bf16, int64_t row_stride, float* state, const int* positions, const int* qsl,
                              const int* state_slots, const int* counts, int seqs, int H, int D, int Dv, const float* decay,
                              float* out, int64_t out_part, const int* tile_seq, const int* tile_q0, int num_tiles, float* ws,
                              bool plain_act, hipStream_t stream) {
  if (seqs == 0) return;
  const int zs = (Dv + 63) / 64;
  const int parts = sm_lightning_parts(D);
  const int DR = (D + parts - 1) / parts;
  const unsigned gz = zs * parts;
  const bool blocks = num_tiles > 0 && ws != nullptr;
  const int plain = plain_act ? 1 : 0;
#define SM_SCAN(DM)                                                                                                                  \
  SM_DISPATCH_BF16(bf16, A, {                                                                                                         \
    hipLaunchKernelGGL((lightning_scan_kernel<A, DM, 0>), dim3(seqs, H, gz), dim3(64), 0, stream, (const A*)qkvg, row_stride, state,  \
                       positions, qsl, state_slots, counts, H, D, Dv, decay, out, tile_seq, tile_q0, num_tiles, ws, blocks ? 1 : 0,  \
                       zs, DR, out_part, plain);                                                                                     \
    if (blocks) {                                                                                                                    \
      hipLaunchKernelGGL((lightning_scan_kernel<A, DM, 1>), dim3(num_tiles, H, gz), dim3(64), 0, stream, (const A*)qkvg, row_stride,  \
                         state, positions, qsl, state_slots, counts, H, D, Dv, decay, out, tile_seq, tile_q0, num_tiles, ws, 0, zs,  \
                         DR, out_part, plain);                                                                                       \
      hipLaunchKernelGGL(lightning_prefix_kernel, dim3(seqs, H, zs * D), dim3(64), 0, stream, state, ws, positions, qsl, state_slots, \
                         counts, H, D, Dv, decay);                                                                                   \
      hipLaunchKernelGGL((lightning_scan_kernel<A, DM, 2>), dim3(num_tiles, H, gz), dim3(64), 0, stream, (const A*)qkvg, row_stride,  \
                         state, positions, qsl, state_slots, counts, H, D, Dv, decay, out, tile_seq, tile_q0, num_tiles, ws, 0, zs,  \
                         DR, out_part, plain);                                                                                       \
    }                                                                                                                                \
  })
  if (DR <= 32) SM_SCAN(32);
  else if (DR <= 64) SM_SCAN(64);
  else if (DR <= 128) SM_SCAN(128);
  else SM_SCAN(256);
#undef SM_SCAN
}

}  // namespace dli
