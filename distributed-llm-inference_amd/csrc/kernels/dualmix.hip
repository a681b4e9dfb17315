// Kernels of the gated parallel layers (models/mixers.py: SinkTalkAttention, TimeMix, RoutedFF, GatedParallelLayer;
// ops/seqmix.py): scalar-gain RMS norms, blends with the previous token's input, whole-projection q/k norm + half-split
// rotation + cache write, attention with a sink and head-mixed weights over token-major pages, the decaying recurrence with
// per-token / per-channel decay, sigmoid routing, squared-ReLU experts and the gated residual update.
//
// Arithmetic: the residual stream, norm statistics, scores, softmax weights, rotation angles (double until reduced), decays,
// the recurrent state, router logits and every gate are fp32; activations are the template type A = float or bf16 (uint16_t
// bit pattern).  Small parameters (norm gains, per-head constants, biases, router rows) are fp32 tensors.
//
// Step metadata (int32, static device buffers): positions[T], slot_mapping[T] (cache row, < 0: padding), token_seq[T] (batch
// row of a token, < 0: padding), query_start_loc[B+1], state_slots[B] (< 0: none), counts[3] = number of valid batch rows.
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

__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }

// fp32 row in LDS · one row of A in global memory: 16-byte loads where the row allows them
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

// lane-strided dot of an fp32 LDS row with a global row of A (one wave per row; coalesced), summed over the wave
template <typename A>
__device__ __forceinline__ float wave_dot(const float* __restrict__ xs, const A* __restrict__ wr, int n) {
  float d = 0.f;
  for (int i = threadIdx.x & 63; i < n; i += 64) d += xs[i] * ldf<A>(wr + i);
  return wave_sum(d);
}

// ------------------------------------------------------------------------------------------------ scalar-gain RMS norms
template <typename O>
__global__ __launch_bounds__(NT) void rms_scale_kernel(const float* __restrict__ x, const float* __restrict__ g1,
                                                       const float* __restrict__ g2, float eps, int W, O* __restrict__ h1,
                                                       O* __restrict__ h2) {
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const float* row = x + t * W;
  float s = 0.f;
  for (int i = threadIdx.x; i < W; i += NT) s += row[i] * row[i];
  const float inv = 1.f / sqrtf(block_sum<NT>(s, red) / (float)W + eps);
  const float a = g1[0], b = g2 != nullptr ? g2[0] : 0.f;
  for (int i = threadIdx.x; i < W; i += NT) {
    const float n = row[i] * inv;
    stf<O>(h1 + t * W + i, n * a);
    if (g2 != nullptr) stf<O>(h2 + t * W + i, n * b);
  }
}

// ------------------------------------------------------------------------------------------------ blends with the previous token
template <typename A>
__global__ __launch_bounds__(NT) void shift_mix_kernel(const A* __restrict__ h, int64_t h_stride, const float* __restrict__ mu, int S,
                                                       const float* __restrict__ state, const int* __restrict__ positions,
                                                       const int* __restrict__ token_seq, const int* __restrict__ qsl,
                                                       const int* __restrict__ state_slots, int T, int W, A* __restrict__ out) {
  const int t = blockIdx.x;
  const int seq = token_seq[t];
  const A* row = h + (int64_t)t * h_stride;
  const A* above = nullptr;
  const float* srow = nullptr;
  if (seq >= 0 && positions[t] > 0) {
    if (t > qsl[seq]) above = h + (int64_t)(t - 1) * h_stride;
    else if (state_slots[seq] >= 0) srow = state + (int64_t)state_slots[seq] * W;
  }
  for (int i = threadIdx.x; i < W; i += NT) {
    const float hv = ldf<A>(row + i);
    const float pv = above != nullptr ? ldf<A>(above + i) : srow != nullptr ? srow[i] : (seq >= 0 ? 0.f : hv);
    const float d = pv - hv;
    for (int s = 0; s < S; ++s) stf<A>(out + ((int64_t)s * T + t) * W + i, hv + d * mu[s * W + i]);
  }
}

// state[slot] = h of every sequence's last token of the step (runs behind shift_mix_kernel)
template <typename A>
__global__ __launch_bounds__(NT) void shift_state_kernel(const A* __restrict__ h, int64_t h_stride, float* __restrict__ state,
                                                         const int* __restrict__ qsl, const int* __restrict__ state_slots,
                                                         const int* __restrict__ counts, int W) {
  const int seq = blockIdx.x;
  if (seq >= counts[3]) return;
  const int slot = state_slots[seq];
  const int t0 = qsl[seq], t1 = qsl[seq + 1];
  if (slot < 0 || t1 <= t0) return;
  for (int i = threadIdx.x; i < W; i += NT) state[(int64_t)slot * W + i] = ldf<A>(h + (int64_t)(t1 - 1) * h_stride + i);
}

// ------------------------------------------------------------------------------------------------ q/k norm + rotation + cache
// One workgroup per token.  LDS: normalised q row | normalised k row | cos | sin.
template <typename A>
__global__ __launch_bounds__(NT) void wide_norm_rope_cache_kernel(A* __restrict__ qkv, int64_t row_stride, const float* __restrict__ qw,
                                                                  const float* __restrict__ kw, float eps,
                                                                  const int* __restrict__ positions, const double* __restrict__ freq,
                                                                  float mag, int rot_dims, const int* __restrict__ slot_mapping,
                                                                  A* __restrict__ k_cache, A* __restrict__ v_cache, int H, int G, int D,
                                                                  int Dv) {
  extern __shared__ float sh[];
  __shared__ float red[NT / 64];
  const int t = blockIdx.x;
  const int nq = H * D, nk = G * D, half = rot_dims >> 1;
  float* qs = sh;
  float* ks = sh + nq;
  float* cs = ks + nk;
  float* sn = cs + half;
  A* row = qkv + (int64_t)t * row_stride;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < nq; i += NT) {
    const float v = ldf<A>(row + i);
    qs[i] = v;
    sq += v * v;
  }
  for (int i = threadIdx.x; i < nk; i += NT) {
    const float v = ldf<A>(row + nq + i);
    ks[i] = v;
    sk += v * v;
  }
  if (threadIdx.x < half && freq != nullptr) {
    const double two_pi = 6.283185307179586476925286766559;
    double a = (double)positions[t] * freq[threadIdx.x];
    a -= floor(a / two_pi) * two_pi;
    cs[threadIdx.x] = cosf((float)a) * mag;
    sn[threadIdx.x] = sinf((float)a) * mag;
  }
  const float iq = 1.f / sqrtf(block_sum<NT>(sq, red) / (float)nq + eps);
  const float ik = 1.f / sqrtf(block_sum<NT>(sk, red) / (float)max(nk, 1) + eps);        // nk = 0: queries only
  for (int i = threadIdx.x; i < nq; i += NT) qs[i] = qs[i] * iq * qw[i];
  for (int i = threadIdx.x; i < nk; i += NT) ks[i] = ks[i] * ik * kw[i];
  __syncthreads();
  const int slot = slot_mapping[t];
  for (int i = threadIdx.x; i < nq + nk; i += NT) {
    const float* src = i < nq ? qs : ks;
    const int e = i < nq ? i : i - nq;
    const int d = e % D;
    float v = src[e];
    if (d < half) v = v * cs[d] - src[e + half] * sn[d];
    else if (d < rot_dims) v = v * cs[d - half] + src[e - half] * sn[d - half];
    if (i < nq) stf<A>(row + i, v);
    else if (slot >= 0) stf<A>(k_cache + (int64_t)slot * nk + e, v);
  }
  if (slot >= 0 && G > 0)
    for (int i = threadIdx.x; i < G * Dv; i += NT) v_cache[(int64_t)slot * G * Dv + i] = row[nq + nk + i];
}

// 4 consecutive row entries ↔ fp32 (16-byte / 8-byte accesses)
template <typename A> __device__ __forceinline__ f32x4 ldv4(const A* p);
template <> __device__ __forceinline__ f32x4 ldv4<float>(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
template <> __device__ __forceinline__ f32x4 ldv4<uint16_t>(const uint16_t* p) {
  const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
  return f32x4{bf2f((uint16_t)v[0]), bf2f((uint16_t)v[1]), bf2f((uint16_t)v[2]), bf2f((uint16_t)v[3])};
}
template <typename A> __device__ __forceinline__ void stv4(A* p, f32x4 v);
template <> __device__ __forceinline__ void stv4<float>(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
template <> __device__ __forceinline__ void stv4<uint16_t>(uint16_t* p, f32x4 v) {
  bf16x4 o;
#pragma unroll
  for (int j = 0; j < 4; ++j) o[j] = (short)f2bf(v[j]);
  *reinterpret_cast<bf16x4*>(p) = o;
}

// The same with four entries per access, for rows whose pieces (q, k, v widths, head size, rotated half) are all multiples of
// four and 16-byte aligned: a vector of four then never straddles a head or the rotated / unrotated border.
template <typename A>
__global__ __launch_bounds__(NT) void wide_norm_rope_cache_v4_kernel(A* __restrict__ qkv, int64_t row_stride, const float* __restrict__ qw,
                                                                     const float* __restrict__ kw, float eps,
                                                                     const int* __restrict__ positions, const double* __restrict__ freq,
                                                                     float mag, int rot_dims, const int* __restrict__ slot_mapping,
                                                                     A* __restrict__ k_cache, A* __restrict__ v_cache, int H, int G, int D,
                                                                     int Dv) {
  extern __shared__ __align__(16) float sh[];
  __shared__ float red[NT / 64];
  const int t = blockIdx.x;
  const int nq = H * D, nk = G * D, half = rot_dims >> 1;
  float* qs = sh;
  float* ks = sh + nq;
  float* cs = ks + nk;
  float* sn = cs + half;
  A* row = qkv + (int64_t)t * row_stride;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x * 4; i < nq; i += NT * 4) {
    const f32x4 v = ldv4<A>(row + i);
    *reinterpret_cast<f32x4*>(qs + i) = v;
    sq += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
  }
  for (int i = threadIdx.x * 4; i < nk; i += NT * 4) {
    const f32x4 v = ldv4<A>(row + nq + i);
    *reinterpret_cast<f32x4*>(ks + i) = v;
    sk += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
  }
  if (threadIdx.x < half && freq != nullptr) {
    const double two_pi = 6.283185307179586476925286766559;
    double a = (double)positions[t] * freq[threadIdx.x];
    a -= floor(a / two_pi) * two_pi;
    cs[threadIdx.x] = cosf((float)a) * mag;
    sn[threadIdx.x] = sinf((float)a) * mag;
  }
  const float iq = 1.f / sqrtf(block_sum<NT>(sq, red) / (float)nq + eps);
  const float ik = 1.f / sqrtf(block_sum<NT>(sk, red) / (float)max(nk, 1) + eps);
  for (int i = threadIdx.x * 4; i < nq; i += NT * 4) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(qs + i), w = *reinterpret_cast<const f32x4*>(qw + i);
    *reinterpret_cast<f32x4*>(qs + i) = f32x4{v[0] * iq * w[0], v[1] * iq * w[1], v[2] * iq * w[2], v[3] * iq * w[3]};
  }
  for (int i = threadIdx.x * 4; i < nk; i += NT * 4) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(ks + i), w = *reinterpret_cast<const f32x4*>(kw + i);
    *reinterpret_cast<f32x4*>(ks + i) = f32x4{v[0] * ik * w[0], v[1] * ik * w[1], v[2] * ik * w[2], v[3] * ik * w[3]};
  }
  __syncthreads();
  const int slot = slot_mapping[t];
  for (int i = threadIdx.x * 4; i < nq + nk; i += NT * 4) {
    const float* src = i < nq ? qs : ks;
    const int e = i < nq ? i : i - nq;
    const int d = e % D;
    f32x4 v = *reinterpret_cast<const f32x4*>(src + e);
    if (d < half) {
      const f32x4 o = *reinterpret_cast<const f32x4*>(src + e + half), c = *reinterpret_cast<const f32x4*>(cs + d),
                  s_ = *reinterpret_cast<const f32x4*>(sn + d);
      v = f32x4{v[0] * c[0] - o[0] * s_[0], v[1] * c[1] - o[1] * s_[1], v[2] * c[2] - o[2] * s_[2], v[3] * c[3] - o[3] * s_[3]};
    } else if (d < rot_dims) {
      const f32x4 o = *reinterpret_cast<const f32x4*>(src + e - half), c = *reinterpret_cast<const f32x4*>(cs + d - half),
                  s_ = *reinterpret_cast<const f32x4*>(sn + d - half);
      v = f32x4{v[0] * c[0] + o[0] * s_[0], v[1] * c[1] + o[1] * s_[1], v[2] * c[2] + o[2] * s_[2], v[3] * c[3] + o[3] * s_[3]};
    }
    if (i < nq) stv4<A>(row + i, v);
    else if (slot >= 0) stv4<A>(k_cache + (int64_t)slot * nk + e, v);
  }
  if (slot >= 0 && G > 0)
    for (int i = threadIdx.x * 4; i < G * Dv; i += NT * 4)
      stv4<A>(v_cache + (int64_t)slot * G * Dv + i, ldv4<A>(row + nq + nk + i));
}

// ------------------------------------------------------------------------------------------------ attention: sink + mixed heads
// One workgroup per token; two passes over the sequence's keys in chunks of 64 (a lane per key).  Pass 1: per head the
// maximum and the denominator (sink included).  Pass 2: normalised weights of all heads for a chunk in LDS, mixed across
// heads, applied to the values (threads over output columns).  Wave w owns heads w, w+4, … in the score passes.
constexpr int TA_CHUNK = 64;
constexpr int TA_MAX_HPW = 16;      // heads per wave  → H ≤ 64
constexpr int TA_MAX_OUT = 32;      // output columns per thread → H·Dv ≤ 8192

template <typename A>
__global__ __launch_bounds__(NT) void talk_attention_kernel(A* __restrict__ out, int64_t o_stride, const A* __restrict__ q, int64_t q_ts,
                                                            int64_t q_hs, const A* __restrict__ gate, int64_t g_stride,
                                                            const A* __restrict__ k_cache, const A* __restrict__ v_cache,
                                                            const int* __restrict__ block_tables, int max_blocks,
                                                            const int* __restrict__ positions, const int* __restrict__ token_seq,
                                                            const float* __restrict__ sink, const float* __restrict__ talk, int H, int G,
                                                            int D, int Dv, float scale) {
  extern __shared__ float sh[];
  const int t = blockIdx.x;
  const int seq = token_seq[t];
  if (seq < 0) {                                               // padding row of a captured step: zeros, not what the buffer held
    for (int o = threadIdx.x; o < H * Dv; o += NT) stf<A>(out + (int64_t)t * o_stride + o, 0.f);
    return;
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int L = positions[t] + 1;
  const int rep = H / G;
  float* qs = sh;                                  // [H·D], scaled
  float* P = qs + H * D;                           // [H][64] normalised weights of a chunk
  float* Pm = P + H * TA_CHUNK;                    // [H][64] mixed
  float* tk = Pm + H * TA_CHUNK;                   // [H·H] mixing matrix (identity without one)
  float* hm = tk + H * H;                          // [H] maximum
  float* hl = hm + H;                              // [H] 1 / denominator
  int* rows = reinterpret_cast<int*>(hl + H);      // [64] cache rows of the chunk
  for (int i = threadIdx.x; i < H * D; i += NT) qs[i] = ldf<A>(q + (int64_t)t * q_ts + (i / D) * q_hs + (i % D)) * scale;
  for (int i = threadIdx.x; i < H * H; i += NT) tk[i] = talk != nullptr ? talk[i] : (i / H == i % H ? 1.f : 0.f);
  __syncthreads();
  const int* bt = block_tables + (int64_t)seq * max_blocks;
  const int n_chunks = (L + TA_CHUNK - 1) / TA_CHUNK;
  const int64_t krow = (int64_t)G * D, vrow = (int64_t)G * Dv;

  // ---- pass 1
  float m[TA_MAX_HPW], l[TA_MAX_HPW];
#pragma unroll
  for (int hi = 0; hi < TA_MAX_HPW; ++hi) { m[hi] = -3.0e38f; l[hi] = 0.f; }
  for (int c = 0; c < n_chunks; ++c) {
    const int j = c * TA_CHUNK + lane;
    if (j >= L) continue;
    const int64_t r = (int64_t)bt[j / kBlockTokens] * kBlockTokens + j % kBlockTokens;
#pragma unroll
    for (int hi = 0; hi < TA_MAX_HPW; ++hi) {
      const int h = wave + 4 * hi;
      if (h < H) {
        const float s = dot_row<A>(qs + h * D, k_cache + r * krow + (h / rep) * D, D);
        const float nm = fmaxf(m[hi], s);
        l[hi] = l[hi] * expf(m[hi] - nm) + expf(s - nm);
        m[hi] = nm;
      }
    }
  }
#pragma unroll
  for (int hi = 0; hi < TA_MAX_HPW; ++hi) {
    const int h = wave + 4 * hi;
    if (h < H) {                                              // wave-uniform
      float wm = wave_max(m[hi]);
      const float sk = sink != nullptr ? sink[h] : -3.0e38f;
      wm = fmaxf(wm, sk);
      float wl = wave_sum(l[hi] * expf(m[hi] - wm));
      if (sink != nullptr) wl += expf(sk - wm);
      if (lane == 0) { hm[h] = wm; hl[h] = 1.f / wl; }
    }
  }
  __syncthreads();

  // ---- pass 2
  float acc[TA_MAX_OUT];
#pragma unroll
  for (int i = 0; i < TA_MAX_OUT; ++i) acc[i] = 0.f;
  const int n_out = H * Dv;
  for (int c = 0; c < n_chunks; ++c) {
    const int j = c * TA_CHUNK + lane;
    int64_t r = -1;
    if (j < L) r = (int64_t)bt[j / kBlockTokens] * kBlockTokens + j % kBlockTokens;
    if (wave == 0) rows[lane] = (int)r;
#pragma unroll
    for (int hi = 0; hi < TA_MAX_HPW; ++hi) {
      const int h = wave + 4 * hi;
      if (h < H) {
        float p = 0.f;
        if (r >= 0) p = expf(dot_row<A>(qs + h * D, k_cache + r * krow + (h / rep) * D, D) - hm[h]) * hl[h];
        P[h * TA_CHUNK + lane] = p;
      }
    }
    __syncthreads();
#pragma unroll
    for (int hi = 0; hi < TA_MAX_HPW; ++hi) {
      const int h = wave + 4 * hi;
      if (h < H) {
        float s = 0.f;
        for (int g = 0; g < H; ++g) s += tk[h * H + g] * P[g * TA_CHUNK + lane];
        Pm[h * TA_CHUNK + lane] = s;
      }
    }
    __syncthreads();
    const int nj = min(TA_CHUNK, L - c * TA_CHUNK);
#pragma unroll
    for (int i = 0; i < TA_MAX_OUT; ++i) {
      const int o = threadIdx.x + i * NT;
      if (o < n_out) {
        const int h = o / Dv, e = o - h * Dv;
        const A* vp = v_cache + (h / rep) * Dv + e;
        const float* pm = Pm + h * TA_CHUNK;
        float a = acc[i];
        for (int jj = 0; jj < nj; ++jj) a += pm[jj] * ldf<A>(vp + (int64_t)rows[jj] * vrow);
        acc[i] = a;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TA_MAX_OUT; ++i) {
    const int o = threadIdx.x + i * NT;
    if (o < n_out) {
      float v = acc[i];
      if (gate != nullptr) v *= sigmoid_f(ldf<A>(gate + (int64_t)t * g_stride + o));
      stf<A>(out + (int64_t)t * o_stride + o, v);
    }
  }
}

// ------------------------------------------------------------------------------------------------ attention: prefill tiles (bf16)
// The same two passes on the matrix cores.  A workgroup owns 16 queries of one chunk and up to 16 output heads (grid.y:
// groups of 16 heads); it computes the scores of ALL heads (the mixing needs them), a wave taking heads w, w+4, ….
// Sᵀ = K·Qᵀ per head on v_mfma_f32_16x16x32_bf16 from a page of K rows staged in LDS (KG key heads per round); pass 1
// keeps each head's running maximum and denominator per query; pass 2 writes the normalised fp32 weights of a page
// to LDS [head][lane][8] — a lane's eight values (two 16-key tiles) are, in that order, its B fragment of the P·V k-step
// — mixes them across heads in fp32 for the wave's own output heads, rounds the mixed weights to bf16 and accumulates
// Oᵀ += Vᵀ·Pᵀ against the staged V page.  KS = D / 32, DVT = Dv / 16.
constexpr int TT_MAX_HW = 8;        // score heads per wave → H ≤ 32
constexpr int TT_HEADS = 16;        // output heads per workgroup
constexpr int TT_MAX_HO = 4;        // output heads per wave

template <int KS, int DVT>
__global__ __launch_bounds__(NT) void talk_tile_kernel(
    uint16_t* __restrict__ out, int64_t o_stride, const uint16_t* __restrict__ q, int64_t q_ts, int64_t q_hs,
    const uint16_t* __restrict__ gate, int64_t g_stride, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
    const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ seq_lens, const int* __restrict__ qsl,
    const int* __restrict__ tile_seq, const int* __restrict__ tile_q0, int num_tiles, const int* __restrict__ counts,
    const float* __restrict__ sink, const float* __restrict__ talk, int H, int G, int KG, int NVmax, float scale) {
  extern __shared__ __align__(16) uint16_t tl[];
  constexpr int D = 32 * KS, Dv = 16 * DVT;
  const int ntiles = counts != nullptr ? min(counts[2], num_tiles) : num_tiles;
  const int tile = num_tiles - 1 - (int)(blockIdx.x >> 2);        // the host lists causal tiles so that the END is longest
  if (tile >= ntiles) return;
  const int seq = tile_seq[tile];
  const int q0 = tile_q0[tile] + 16 * (int)(blockIdx.x & 3);
  const int t_begin = qsl[seq];
  const int n_chunk = qsl[seq + 1] - t_begin;
  const int nq = min(16, n_chunk - q0);
  if (nq <= 0) return;
  const int p0 = seq_lens[seq] - n_chunk;                          // position of the chunk's first token
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63, g4 = lane >> 4, c = lane & 15;
  const int rep = H / G;
  const int hb = blockIdx.y * TT_HEADS, nh = min(TT_HEADS, H - hb);
  const int per = (nh + 3) >> 2;                                   // output heads per wave
  const int c_lo = hb / rep, NV = (hb + nh - 1) / rep - c_lo + 1;  // value heads this workgroup reads
  const int KST = KG * D + 8, VST = NVmax * Dv + 8;                // LDS row strides (elements): +16 bytes against bank conflicts
  uint16_t* Ks = tl;
  uint16_t* Vs = Ks + 32 * KST;
  float* Pl = reinterpret_cast<float*>(Vs + 32 * VST);             // [H][64][8]
  float* Tk = Pl + H * 512;                                        // [nh][H]
  float* St = Tk + TT_HEADS * H;                                   // [H][16][2]: maximum, 1 / denominator
  for (int i = threadIdx.x; i < nh * H; i += NT) {
    const int h = hb + i / H, g = i % H;
    Tk[i] = talk != nullptr ? talk[h * H + g] : (h == g ? 1.f : 0.f);
  }
  const bool qvalid = c < nq;
  const int64_t tq = t_begin + q0 + (qvalid ? c : 0);
  const int pos_q = qvalid ? p0 + q0 + c : 0x7fffffff;             // rows past the chunk: nothing masked, nothing stored
  const int n_kb = (p0 + q0 + nq - 1) / kBlockTokens + 1;
  const int* bt = block_tables + (int64_t)seq * max_blocks;
  const int rounds = (G + KG - 1) / KG;
  const int64_t krow = (int64_t)G * D, vrow = (int64_t)G * Dv;

  // scores of head g for the staged K page: two 16-key tiles, natural units, masked entries → -inf
#define TT_SCORES(g_, kvl_, kb_, s0_, s1_)                                                                         \
  {                                                                                                                \
    f32x4 a0_ = {0.f, 0.f, 0.f, 0.f}, a1_ = {0.f, 0.f, 0.f, 0.f};                                                  \
    _Pragma("unroll") for (int ks_ = 0; ks_ < KS; ++ks_) {                                                         \
      const bf16x8 qf_ = *reinterpret_cast<const bf16x8*>(q + tq * q_ts + (g_) * q_hs + ks_ * 32 + 8 * g4);        \
      const bf16x8 k0_ = *reinterpret_cast<const bf16x8*>(Ks + c * KST + (kvl_) * D + ks_ * 32 + 8 * g4);          \
      const bf16x8 k1_ = *reinterpret_cast<const bf16x8*>(Ks + (16 + c) * KST + (kvl_) * D + ks_ * 32 + 8 * g4);   \
      a0_ = mfma16(k0_, qf_, a0_);                                                                                 \
      a1_ = mfma16(k1_, qf_, a1_);                                                                                 \
    }                                                                                                              \
    _Pragma("unroll") for (int r_ = 0; r_ < 4; ++r_) {                                                             \
      const int j_ = (kb_) * kBlockTokens + 4 * g4 + r_;                                                           \
      s0_[r_] = j_ <= pos_q ? a0_[r_] * scale : -INFINITY;                                                         \
      s1_[r_] = j_ + 16 <= pos_q ? a1_[r_] * scale : -INFINITY;                                                    \
    }                                                                                                              \
  }
#define TT_STAGE_K(page_, r_)                                                                                      \
  {                                                                                                                \
    const int kg_ = min(KG, G - (r_) * KG), cpr_ = kg_ * D / 8;                                                    \
    for (int i_ = threadIdx.x; i_ < 32 * cpr_; i_ += NT) {                                                         \
      const int row_ = i_ / cpr_, ch_ = i_ - row_ * cpr_;                                                          \
      *reinterpret_cast<bf16x8*>(Ks + row_ * KST + ch_ * 8) =                                                      \
          *reinterpret_cast<const bf16x8*>(kc + ((int64_t)(page_) * kBlockTokens + row_) * krow + (r_) * KG * D + ch_ * 8); \
    }                                                                                                              \
  }

  // ---- pass 1: maximum and denominator of every head
  float m[TT_MAX_HW], l[TT_MAX_HW];
#pragma unroll
  for (int i = 0; i < TT_MAX_HW; ++i) { m[i] = -3.0e38f; l[i] = 0.f; }
  for (int kb = 0; kb < n_kb; ++kb) {
    const int page = bt[kb];
    for (int r = 0; r < rounds; ++r) {
      __syncthreads();
      TT_STAGE_K(page, r);
      __syncthreads();
      const int g_lo = r * KG * rep, g_hi = min(H, g_lo + KG * rep);
#pragma unroll
      for (int i = 0; i < TT_MAX_HW; ++i) {
        const int g = 4 * i + wave;
        if (g >= g_lo && g < g_hi) {                              // wave-uniform
          f32x4 s0, s1;
          TT_SCORES(g, g / rep - r * KG, kb, s0, s1);
          float mx = m[i];
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) mx = fmaxf(mx, fmaxf(s0[rr], s1[rr]));
          float add = 0.f;
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) add += __expf(s0[rr] - mx) + __expf(s1[rr] - mx);
          l[i] = l[i] * __expf(m[i] - mx) + add;
          m[i] = mx;
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < TT_MAX_HW; ++i) {
    const int g = 4 * i + wave;
    if (g < H) {
      float mx = fmaxf(m[i], __shfl_xor(m[i], 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float sk = sink != nullptr ? sink[g] : -3.0e38f;
      mx = fmaxf(mx, sk);
      float ls = l[i] * __expf(m[i] - mx);
      ls += __shfl_xor(ls, 16, 64);
      ls += __shfl_xor(ls, 32, 64);
      if (sink != nullptr) ls += __expf(sk - mx);
      if (g4 == 0) {
        St[(g * 16 + c) * 2] = mx;
        St[(g * 16 + c) * 2 + 1] = 1.f / ls;
      }
    }
  }

  // ---- pass 2
  f32x4 acc[TT_MAX_HO][DVT];
#pragma unroll
  for (int i = 0; i < TT_MAX_HO; ++i)
#pragma unroll
    for (int d = 0; d < DVT; ++d) acc[i][d] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int kb = 0; kb < n_kb; ++kb) {
    const int page = bt[kb];
    for (int r = 0; r < rounds; ++r) {
      __syncthreads();                                            // everyone is done with the previous K / V / weights (and St is written)
      TT_STAGE_K(page, r);
      if (r == 0) {
        const int cpr = NV * Dv / 8;
        for (int i = threadIdx.x; i < 32 * cpr; i += NT) {
          const int row = i / cpr, ch = i - row * cpr;
          *reinterpret_cast<bf16x8*>(Vs + row * VST + ch * 8) =
              *reinterpret_cast<const bf16x8*>(vc + ((int64_t)page * kBlockTokens + row) * vrow + c_lo * Dv + ch * 8);
        }
      }
      __syncthreads();
      const int g_lo = r * KG * rep, g_hi = min(H, g_lo + KG * rep);
#pragma unroll
      for (int i = 0; i < TT_MAX_HW; ++i) {
        const int g = 4 * i + wave;
        if (g >= g_lo && g < g_hi) {
          f32x4 s0, s1;
          TT_SCORES(g, g / rep - r * KG, kb, s0, s1);
          const float mx = St[(g * 16 + c) * 2], il = St[(g * 16 + c) * 2 + 1];
          f32x4 pa, pb;
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) {
            pa[rr] = __expf(s0[rr] - mx) * il;
            pb[rr] = __expf(s1[rr] - mx) * il;
          }
          *reinterpret_cast<f32x4*>(Pl + (g * 64 + lane) * 8) = pa;
          *reinterpret_cast<f32x4*>(Pl + (g * 64 + lane) * 8 + 4) = pb;
        }
      }
    }
    __syncthreads();                                              // the page's weights of all heads are in LDS
    int cur_c = -1;
    bf16x8 vf[DVT];
#pragma unroll
    for (int i = 0; i < TT_MAX_HO; ++i) {
      const int hl = wave * per + i;                              // wave-uniform
      if (i < per && hl < nh) {
        const float* trow = Tk + hl * H;
        f32x4 ma = {0.f, 0.f, 0.f, 0.f}, mb = {0.f, 0.f, 0.f, 0.f};
        for (int g = 0; g < H; ++g) {
          const float tw = trow[g];
          const f32x4 pa = *reinterpret_cast<const f32x4*>(Pl + (g * 64 + lane) * 8);
          const f32x4 pb = *reinterpret_cast<const f32x4*>(Pl + (g * 64 + lane) * 8 + 4);
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) {
            ma[rr] += tw * pa[rr];
            mb[rr] += tw * pb[rr];
          }
        }
        bf16x8 pf;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          pf[rr] = (short)f2bf(ma[rr]);
          pf[4 + rr] = (short)f2bf(mb[rr]);
        }
        const int cl = (hb + hl) / rep - c_lo;
        if (cl != cur_c) {
          cur_c = cl;
#pragma unroll
          for (int d = 0; d < DVT; ++d) {
            const uint16_t* vp = Vs + cl * Dv + d * 16 + c;
            bf16x8 v;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              v[j] = (short)vp[(4 * g4 + j) * VST];
              v[4 + j] = (short)vp[(16 + 4 * g4 + j) * VST];
            }
            vf[d] = v;
          }
        }
#pragma unroll
        for (int d = 0; d < DVT; ++d) acc[i][d] = mfma16(vf[d], pf, acc[i][d]);
      }
    }
  }
#undef TT_SCORES
#undef TT_STAGE_K
  if (!qvalid) return;
#pragma unroll
  for (int i = 0; i < TT_MAX_HO; ++i) {
    const int hl = wave * per + i;
    if (i < per && hl < nh) {
#pragma unroll
      for (int d = 0; d < DVT; ++d) {
        const int col = (hb + hl) * Dv + d * 16 + 4 * g4;
        f32x4 o = acc[i][d];
        if (gate != nullptr) {
          const bf16x4 gv = *reinterpret_cast<const bf16x4*>(gate + tq * g_stride + col);
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) o[rr] *= sigmoid_f(bf2f((uint16_t)gv[rr]));
        }
        bf16x4 ov;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) ov[rr] = (short)f2bf(o[rr]);
        *reinterpret_cast<bf16x4*>(out + tq * o_stride + col) = ov;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------ decay
// w[t, c] = exp(-exp(Σ_l w2[c, l] · tanh(a[t, l]) + w0[c]))
template <typename A>
__global__ __launch_bounds__(NT) void decay_kernel(const A* __restrict__ a, int64_t a_stride, const A* __restrict__ w2,
                                                   const float* __restrict__ w0, int Lr, int C, float* __restrict__ out) {
  extern __shared__ float sh[];
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < Lr; i += NT) sh[i] = tanhf(ldf<A>(a + t * a_stride + i));
  __syncthreads();
  for (int c = threadIdx.x; c < C; c += NT) {
    float s = 0.f;
    for (int i = 0; i < Lr; ++i) s += sh[i] * ldf<A>(w2 + (int64_t)c * Lr + i);
    out[t * C + c] = expf(-expf(s + w0[c]));
  }
}

// ------------------------------------------------------------------------------------------------ recurrence
// One workgroup per (sequence, head).  Thread = (value column e, row group rg): it keeps the state rows d = rg, rg+R, … of
// column e in registers (R = NT / D row groups, at most MAXR rows each) and walks the sequence's tokens of this step in order.
template <typename A, int MAXR>
__global__ __launch_bounds__(NT) void wkv_scan_kernel(const A* __restrict__ rkv, int64_t plane, const float* __restrict__ w,
                                                      const float* __restrict__ u, float* __restrict__ state,
                                                      const int* __restrict__ positions, const int* __restrict__ qsl,
                                                      const int* __restrict__ state_slots, const int* __restrict__ counts, int H,
                                                      int D, float* __restrict__ out) {
  extern __shared__ float sh[];
  const int seq = blockIdx.x, h = blockIdx.y;
  if (seq >= counts[3]) return;
  const int slot = state_slots[seq];
  const int t0 = qsl[seq], t1 = qsl[seq + 1];
  if (slot < 0 || t1 <= t0) return;
  const int R = NT / D;                                       // row groups (≥ 1: the launcher checks D ≤ NT)
  const int e = threadIdx.x % D, rg = threadIdx.x / D;
  const bool active = rg < R;
  const int C = H * D;
  float* rs = sh;                                             // [D] receptance
  float* ks = rs + D;                                         // [D] key
  float* ws = ks + D;                                         // [D] decay
  float* us = ws + D;                                         // [D] bonus
  float* part = us + D;                                       // [R][D] partial outputs
  float S[MAXR];
  float* srow = state + ((int64_t)slot * H + h) * D * D;
  const bool fresh = positions[t0] == 0;
#pragma unroll
  for (int i = 0; i < MAXR; ++i) {
    const int d = rg + i * R;
    S[i] = (active && d < D && !fresh) ? srow[d * D + e] : 0.f;
  }
  if (threadIdx.x < D) us[threadIdx.x] = u[h * D + threadIdx.x];
  for (int t = t0; t < t1; ++t) {
    const int64_t base = (int64_t)t * C + h * D;
    if (threadIdx.x < D) {
      rs[threadIdx.x] = ldf<A>(rkv + base + threadIdx.x);
      ks[threadIdx.x] = ldf<A>(rkv + plane + base + threadIdx.x);
      ws[threadIdx.x] = w[base + threadIdx.x];
    }
    __syncthreads();
    if (active) {
      const float v = ldf<A>(rkv + 2 * plane + base + e);
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < MAXR; ++i) {
        const int d = rg + i * R;
        if (d < D) {
          const float kv = ks[d] * v;
          o += rs[d] * (S[i] + us[d] * kv);
          S[i] = ws[d] * S[i] + kv;
        }
      }
      part[rg * D + e] = o;
    }
    __syncthreads();
    if (threadIdx.x < D) {
      float o = 0.f;
      for (int g = 0; g < R; ++g) o += part[g * D + threadIdx.x];
      out[base + threadIdx.x] = o;
    }
  }
  if (active) {
#pragma unroll
    for (int i = 0; i < MAXR; ++i) {
      const int d = rg + i * R;
      if (d < D) srow[d * D + e] = S[i];
    }
  }
}

// ------------------------------------------------------------------------------------------------ per-group unit RMS · w · silu(gate)
template <typename G, typename O>
__global__ __launch_bounds__(NT) void group_rms_gate_kernel(const float* __restrict__ o, int groups, const float* __restrict__ w, float eps,
                                                            const G* __restrict__ gate, int64_t g_stride, int C, O* __restrict__ out) {
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int Dg = C / groups;
  for (int g = wave; g < groups; g += NT / 64) {
    const float* row = o + t * C + g * Dg;
    float s = 0.f;
    for (int i = lane; i < Dg; i += 64) s += row[i] * row[i];
    const float inv = 1.f / sqrtf(wave_sum(s) / (float)Dg + eps);
    for (int i = lane; i < Dg; i += 64) {
      const float z = ldf<G>(gate + t * g_stride + g * Dg + i);
      stf<O>(out + t * C + g * Dg + i, row[i] * inv * w[g * Dg + i] * (z * sigmoid_f(z)));
    }
  }
}

// ------------------------------------------------------------------------------------------------ sigmoid routing
// One workgroup per token: fp32 logits of all router rows (a wave per row), then wave 0 picks the top-k scores
// (ties → lowest expert id).  Rows beyond E: the per-token extra gate.
template <typename A>
__global__ __launch_bounds__(NT) void sigmoid_route_kernel(const A* __restrict__ h, int64_t h_stride, const float* __restrict__ router,
                                                           int rows, int E, int K, float scale, int W, int* __restrict__ ids,
                                                           float* __restrict__ wts, float* __restrict__ extra) {
  extern __shared__ float sh[];
  __shared__ float z[65];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < W; i += NT) sh[i] = ldf<A>(h + t * h_stride + i);
  __syncthreads();
  for (int r = wave; r < rows; r += NT / 64) {
    const float d = wave_dot<float>(sh, router + (int64_t)r * W, W);
    if (lane == 0) z[r] = d;
  }
  __syncthreads();
  if (wave != 0) return;
  if (rows > E && lane == 0) extra[t] = sigmoid_f(z[E]);
  // Picked by logit (the order of the scores, no saturated ties).  Every pass takes an expert that is still free, whatever
  // the logits hold: a row of padding can carry NaNs, and an id outside the experts would index past their weights.  A lane
  // that cannot be picked (no expert, or taken) offers -inf under an index past every expert; a NaN logit counts as -inf.
  float p = -INFINITY;
  if (lane < E) {
    const float v = z[lane];
    p = v == v ? v : -INFINITY;
  }
  bool free_lane = lane < E;
  for (int k = 0; k < K; ++k) {
    float bv = free_lane ? p : -INFINITY;
    int bi = free_lane ? lane : 64 + lane;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    // (value, index) is a total order without NaNs: every lane now holds the same pick
    if (lane == 0) {
      ids[t * K + k] = min(bi, E - 1);
      wts[t * K + k] = sigmoid_f(bv) * scale;
    }
    if (lane == bi) free_lane = false;
  }
}

// ------------------------------------------------------------------------------------------------ experts, any shape
// act[p, f] for the routed pair p = t·K + slot.  ACT 0: relu(up[e_p, f, :] · h[t])².  Gated forms: an expert's rows are F gate
// rows, then F up rows; with g = gate[e_p, f, :] · h[t] and u = up[e_p, f, :] · h[t], ACT 1: silu(g) · u; ACT 2 (clamped):
// g' = min(g, limit), u' = clamp(u, ±limit), g' · sigmoid(1.702 g') · (u' + 1).  A pair whose id is not one of the E experts
// (an identity expert) has no row to compute.
template <typename A, int ACT>
__global__ __launch_bounds__(NT) void expert_up_kernel(const A* __restrict__ h, int64_t h_stride, const int* __restrict__ ids, int K,
                                                       const A* __restrict__ up, int F, int W, A* __restrict__ act, int E, float limit) {
  extern __shared__ float sh[];
  const int64_t p = blockIdx.x;
  const int64_t t = p / K;
  const int e = ids[p];
  if (e < 0 || e >= E) return;
  for (int i = threadIdx.x; i < W; i += NT) sh[i] = ldf<A>(h + t * h_stride + i);
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const A* we = up + (int64_t)e * (ACT ? 2 : 1) * F * W;
  for (int f = wave; f < F; f += NT / 64) {
    if (ACT == 1) {
      const float g = wave_dot<A>(sh, we + (int64_t)f * W, W), u = wave_dot<A>(sh, we + (int64_t)(F + f) * W, W);
      if (lane == 0) stf<A>(act + p * F + f, g * sigmoid_f(g) * u);
    } else if (ACT == 2) {
      const float g = fminf(wave_dot<A>(sh, we + (int64_t)f * W, W), limit);
      const float u = fminf(fmaxf(wave_dot<A>(sh, we + (int64_t)(F + f) * W, W), -limit), limit);
      if (lane == 0) stf<A>(act + p * F + f, g * sigmoid_f(1.702f * g) * (u + 1.f));
    } else {
      const float d = fmaxf(wave_dot<A>(sh, we + (int64_t)f * W, W), 0.f);
      if (lane == 0) stf<A>(act + p * F + f, d * d);
    }
  }
}

// out[t, c] = Σ_slots wts[t, s] · down[e_s, c, :] · act[t·K + s, :]; a slot whose id is not one of the E experts adds
// wts[t, s] · hid[t, c] instead (identity expert; hid may be null when every id is an expert's)
template <typename A>
__global__ __launch_bounds__(NT) void expert_down_kernel(const A* __restrict__ act, const int* __restrict__ ids, const float* __restrict__ wts,
                                                         int K, const A* __restrict__ down, int F, int W, A* __restrict__ out, int E,
                                                         const A* __restrict__ hid, int64_t hid_stride) {
  extern __shared__ float sh[];
  const int64_t t = blockIdx.x;
  float idw = 0.f;
  for (int k = 0; k < K; ++k) {
    const int e = ids[t * K + k];
    const bool real = e >= 0 && e < E;
    if (!real && hid != nullptr) idw += wts[t * K + k];
    for (int i = threadIdx.x; i < F; i += NT) sh[k * F + i] = real ? ldf<A>(act + (t * K + k) * F + i) : 0.f;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int c = wave; c < W; c += NT / 64) {
    float s = 0.f;
    for (int k = 0; k < K; ++k) {
      const int e = ids[t * K + k];
      if (e >= 0 && e < E) s += wts[t * K + k] * wave_dot<A>(sh + k * F, down + ((int64_t)e * W + c) * F, F);
    }
    if (lane == 0) stf<A>(out + t * W + c, idw != 0.f ? s + idw * ldf<A>(hid + t * hid_stride + c) : s);
  }
}

template <typename A>
__global__ __launch_bounds__(NT) void relu2_rows_kernel(const A* __restrict__ x, int64_t x_stride, int F, int64_t n, A* __restrict__ out) {
  for (int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x; i < n; i += (int64_t)gridDim.x * NT) {
    const float v = fmaxf(ldf<A>(x + (i / F) * x_stride + i % F), 0.f);
    stf<A>(out + i, v * v);
  }
}

// ------------------------------------------------------------------------------------------------ gated residual update
// x += mult · (sigmoid(g1 + b1) · (s0·p0 + s1·p1) + sigmoid(g2 + b2) · (ff + sg · shared))
template <typename A>
__global__ __launch_bounds__(NT) void gated_combine_kernel(float* __restrict__ x, float mult, const A* __restrict__ p0,
                                                           const A* __restrict__ p1, float s0, float s1, const A* __restrict__ g1,
                                                           int64_t g1_stride, const float* __restrict__ b1, const A* __restrict__ ff,
                                                           const A* __restrict__ shared, const float* __restrict__ sg,
                                                           const A* __restrict__ g2, int64_t g2_stride, const float* __restrict__ b2,
                                                           int W) {
  const int64_t t = blockIdx.x;
  const float sgt = sg != nullptr ? sg[t] : 1.f;
  for (int i = threadIdx.x; i < W; i += NT) {
    const int64_t k = t * W + i;
    float y = sigmoid_f(ldf<A>(g1 + t * g1_stride + i) + b1[i]) * (s0 * ldf<A>(p0 + k) + s1 * ldf<A>(p1 + k));
    if (g2 != nullptr) {
      float f = ff != nullptr ? ldf<A>(ff + k) : 0.f;
      if (shared != nullptr) f += sgt * ldf<A>(shared + k);
      y += sigmoid_f(ldf<A>(g2 + t * g2_stride + i) + b2[i]) * f;
    }
    x[k] += mult * y;
  }
}

#define DM_BF16(flag, T, ...) \
  do {                        \
    if (flag) {               \
      using T = uint16_t;     \
      __VA_ARGS__;            \
    } else {                  \
      using T = float;        \
      __VA_ARGS__;            \
    }                         \
  } while (0)

}  // namespace

// ================================================================================================ launchers
void launch_dm_rms_scale(const float* x, const float* g1, const float* g2, float eps, int rows, int W, void* h1, void* h2, bool out_bf16,
                         hipStream_t stream) {
  if (rows == 0) return;
  DM_BF16(out_bf16, O, hipLaunchKernelGGL(rms_scale_kernel<O>, dim3(rows), dim3(NT), 0, stream, x, g1, g2, eps, W, (O*)h1, (O*)h2));
}

void launch_dm_shift_mix(const void* h, bool bf16, int64_t h_stride, const float* mu, int S, float* state, const int* positions,
                         const int* token_seq, const int* qsl, const int* state_slots, const int* counts, int T, int seqs, int W,
                         void* out, hipStream_t stream) {
  if (T == 0) return;
  DM_BF16(bf16, A, {
    hipLaunchKernelGGL(shift_mix_kernel<A>, dim3(T), dim3(NT), 0, stream, (const A*)h, h_stride, mu, S, state, positions, token_seq, qsl,
                       state_slots, T, W, (A*)out);
    if (seqs > 0)
      hipLaunchKernelGGL(shift_state_kernel<A>, dim3(seqs), dim3(NT), 0, stream, (const A*)h, h_stride, state, qsl, state_slots, counts, W);
  });
}

void launch_dm_wide_norm_rope_cache(void* qkv, bool bf16, int64_t row_stride, const float* qw, const float* kw, float eps,
                                    const int* positions, const double* freq, float mag, int rot_dims, const int* slot_mapping,
                                    void* k_cache, void* v_cache, int rows, int H, int G, int D, int Dv, hipStream_t stream) {
  if (rows == 0) return;
  const size_t lds = (size_t)(H * D + G * D + rot_dims) * sizeof(float);
  auto al = [](const void* p) { return p == nullptr || reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool wide = D % 4 == 0 && Dv % 4 == 0 && rot_dims % 8 == 0 && row_stride % 4 == 0 && al(qkv) && al(qw) && al(kw) && al(k_cache) &&
                    al(v_cache);
  if (wide)
    DM_BF16(bf16, A, hipLaunchKernelGGL(wide_norm_rope_cache_v4_kernel<A>, dim3(rows), dim3(NT), lds, stream, (A*)qkv, row_stride, qw, kw,
                                        eps, positions, freq, mag, rot_dims, slot_mapping, (A*)k_cache, (A*)v_cache, H, G, D, Dv));
  else
    DM_BF16(bf16, A, hipLaunchKernelGGL(wide_norm_rope_cache_kernel<A>, dim3(rows), dim3(NT), lds, stream, (A*)qkv, row_stride, qw, kw, eps,
                                        positions, freq, mag, rot_dims, slot_mapping, (A*)k_cache, (A*)v_cache, H, G, D, Dv));
}

size_t dm_talk_attention_lds(int H, int D) { return (size_t)(H * D + 2 * H * TA_CHUNK + H * H + 2 * H + TA_CHUNK) * sizeof(float); }
int dm_talk_attention_max_heads() { return 4 * TA_MAX_HPW; }
int dm_talk_attention_max_out() { return NT * TA_MAX_OUT; }

void launch_dm_talk_attention(void* out, int64_t o_stride, const void* q, int64_t q_ts, int64_t q_hs, const void* gate, int64_t g_stride,
                              const void* k_cache, const void* v_cache, bool bf16, const int* block_tables, int max_blocks,
                              const int* positions, const int* token_seq, const float* sink, const float* talk, int rows, int H, int G,
                              int D, int Dv, float scale, hipStream_t stream) {
  if (rows == 0) return;
  DM_BF16(bf16, A, hipLaunchKernelGGL(talk_attention_kernel<A>, dim3(rows), dim3(NT), dm_talk_attention_lds(H, D), stream, (A*)out, o_stride,
                                      (const A*)q, q_ts, q_hs, (const A*)gate, g_stride, (const A*)k_cache, (const A*)v_cache,
                                      block_tables, max_blocks, positions, token_seq, sink, talk, H, G, D, Dv, scale));
}

// More than 64 KiB of dynamic LDS needs an opt-in per kernel.  Done once, for every instantiation, and callable ahead of time
// (model construction) so that the attribute call never falls inside a stream capture.
void dm_prepare_kernels() {
  static const bool done = [] {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&talk_tile_kernel<2, 4>), hipFuncAttributeMaxDynamicSharedMemorySize,
                              150 * 1024);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&talk_tile_kernel<4, 8>), hipFuncAttributeMaxDynamicSharedMemorySize,
                              150 * 1024);
    return true;
  }();
  (void)done;
}

// Prefill tiles of a bf16 step on the matrix cores; false: shapes the tile kernel does not cover (the caller runs the
// per-token kernel on every row instead).
bool launch_dm_talk_tile_attention(void* out, int64_t o_stride, const void* q, int64_t q_ts, int64_t q_hs, const void* gate,
                                   int64_t g_stride, const void* k_cache, const void* v_cache, const int* block_tables, int max_blocks,
                                   const int* seq_lens, const int* qsl, const int* tile_seq, const int* tile_q0, int num_tiles,
                                   const int* counts, const float* sink, const float* talk, int H, int G, int D, int Dv, float scale,
                                   hipStream_t stream) {
  if (num_tiles <= 0) return true;
  const bool shape = (D == 64 && Dv == 64) || (D == 128 && Dv == 128);
  if (!shape || H > 4 * TT_MAX_HW || H % G != 0) return false;
  auto al = [](const void* p, int a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; };
  if (!al(q, 16) || q_ts % 8 || q_hs % 8 || !al(out, 8) || o_stride % 4 || (gate != nullptr && (!al(gate, 8) || g_stride % 4)) ||
      !al(k_cache, 16) || !al(v_cache, 16))
    return false;
  const int rep = H / G;
  // key heads staged per round: the whole row when it fits 32 KiB, else groups whose query heads are a multiple of the 4 waves
  int KG = G;
  while (32 * KG * D * 2 > 32 * 1024 && KG % 2 == 0 && (KG / 2 * rep) % 4 == 0) KG /= 2;
  if (32 * KG * D * 2 > 40 * 1024) return false;
  const int groups = (H + TT_HEADS - 1) / TT_HEADS;
  const int NVmax = std::min(G, (TT_HEADS + rep - 1) / rep + 1);
  const size_t lds = (size_t)32 * (KG * D + 8) * 2 + (size_t)32 * (NVmax * Dv + 8) * 2 +
                     (size_t)(H * 512 + TT_HEADS * H + H * 32) * sizeof(float);
  if (lds > 150 * 1024) return false;
  dm_prepare_kernels();
#define DM_TT(KSV, DVTV)                                                                                                       \
  do {                                                                                                                         \
    hipLaunchKernelGGL((talk_tile_kernel<KSV, DVTV>), dim3(num_tiles * 4, groups), dim3(NT), lds, stream, (uint16_t*)out, o_stride, \
                       (const uint16_t*)q, q_ts, q_hs, (const uint16_t*)gate, g_stride, (const uint16_t*)k_cache,              \
                       (const uint16_t*)v_cache, block_tables, max_blocks, seq_lens, qsl, tile_seq, tile_q0, num_tiles, counts, \
                       sink, talk, H, G, KG, NVmax, scale);                                                                    \
  } while (0)
  if (D == 64) DM_TT(2, 4);
  else DM_TT(4, 8);
#undef DM_TT
  return true;
}

void launch_dm_decay(const void* a, bool bf16, int64_t a_stride, const void* w2, const float* w0, int rows, int Lr, int C, float* out,
                     hipStream_t stream) {
  if (rows == 0) return;
  DM_BF16(bf16, A, hipLaunchKernelGGL(decay_kernel<A>, dim3(rows), dim3(NT), Lr * sizeof(float), stream, (const A*)a, a_stride,
                                      (const A*)w2, w0, Lr, C, out));
}

void launch_dm_wkv_scan(const void* rkv, bool bf16, int64_t plane, const float* w, const float* u, float* state, const int* positions,
                        const int* qsl, const int* state_slots, const int* counts, int seqs, int H, int D, float* out,
                        hipStream_t stream) {
  if (seqs == 0) return;
  const int R = NT / D;
  const size_t lds = (size_t)(4 * D + R * D) * sizeof(float);
  const int rows_per_thread = (D + R - 1) / R;
  DM_BF16(bf16, A, {
    if (rows_per_thread <= 16)
      hipLaunchKernelGGL((wkv_scan_kernel<A, 16>), dim3(seqs, H), dim3(NT), lds, stream, (const A*)rkv, plane, w, u, state, positions, qsl,
                         state_slots, counts, H, D, out);
    else
      hipLaunchKernelGGL((wkv_scan_kernel<A, 64>), dim3(seqs, H), dim3(NT), lds, stream, (const A*)rkv, plane, w, u, state, positions, qsl,
                         state_slots, counts, H, D, out);
  });
}

void launch_dm_group_rms_gate(const float* o, int groups, const float* w, float eps, const void* gate, bool gate_bf16, int64_t g_stride,
                              int rows, int C, void* out, bool out_bf16, hipStream_t stream) {
  if (rows == 0) return;
  DM_BF16(gate_bf16, G, DM_BF16(out_bf16, O, hipLaunchKernelGGL((group_rms_gate_kernel<G, O>), dim3(rows), dim3(NT), 0, stream, o, groups,
                                                                w, eps, (const G*)gate, g_stride, C, (O*)out)));
}

void launch_dm_sigmoid_route(const void* h, bool bf16, int64_t h_stride, const float* router, int router_rows, int E, int K, float scale,
                             int rows, int W, int* ids, float* wts, float* extra, hipStream_t stream) {
  if (rows == 0) return;
  DM_BF16(bf16, A, hipLaunchKernelGGL(sigmoid_route_kernel<A>, dim3(rows), dim3(NT), W * sizeof(float), stream, (const A*)h, h_stride,
                                      router, router_rows, E, K, scale, W, ids, wts, extra));
}

void launch_dm_experts(const void* h, bool bf16, int64_t h_stride, const int* ids, const float* wts, int K, const void* up,
                       const void* down, int rows, int F, int W, void* act, void* out, int act_kind, int E, float limit,
                       hipStream_t stream) {
  if (rows == 0) return;
  DM_BF16(bf16, A, {
    if (act_kind == 2)
      hipLaunchKernelGGL((expert_up_kernel<A, 2>), dim3(rows * K), dim3(NT), W * sizeof(float), stream, (const A*)h, h_stride, ids, K,
                         (const A*)up, F, W, (A*)act, E, limit);
    else if (act_kind == 1)
      hipLaunchKernelGGL((expert_up_kernel<A, 1>), dim3(rows * K), dim3(NT), W * sizeof(float), stream, (const A*)h, h_stride, ids, K,
                         (const A*)up, F, W, (A*)act, E, limit);
    else
      hipLaunchKernelGGL((expert_up_kernel<A, 0>), dim3(rows * K), dim3(NT), W * sizeof(float), stream, (const A*)h, h_stride, ids, K,
                         (const A*)up, F, W, (A*)act, E, limit);
    hipLaunchKernelGGL(expert_down_kernel<A>, dim3(rows), dim3(NT), (size_t)K * F * sizeof(float), stream, (const A*)act, ids, wts, K,
                       (const A*)down, F, W, (A*)out, E, act_kind == 2 ? (const A*)h : (const A*)nullptr, h_stride);
  });
}

void launch_dm_relu2_rows(const void* x, bool bf16, int64_t x_stride, int rows, int F, void* out, hipStream_t stream) {
  const int64_t n = (int64_t)rows * F;
  if (n == 0) return;
  const int blocks = (int)std::min<int64_t>((n + NT - 1) / NT, 8192);
  DM_BF16(bf16, A, hipLaunchKernelGGL(relu2_rows_kernel<A>, dim3(blocks), dim3(NT), 0, stream, (const A*)x, x_stride, F, n, (A*)out));
}

void launch_dm_gated_combine(float* x, float mult, const void* p0, const void* p1, float s0, float s1, const void* g1, int64_t g1_stride,
                             const float* b1, const void* ff, const void* shared, const float* sg, const void* g2, int64_t g2_stride,
                             const float* b2, bool bf16, int rows, int W, hipStream_t stream) {
  if (rows == 0) return;
  DM_BF16(bf16, A, hipLaunchKernelGGL(gated_combine_kernel<A>, dim3(rows), dim3(NT), 0, stream, x, mult, (const A*)p0, (const A*)p1, s0, s1,
                                      (const A*)g1, g1_stride, b1, (const A*)ff, (const A*)shared, sg, (const A*)g2, g2_stride, b2, W));
}

}  // namespace dli
