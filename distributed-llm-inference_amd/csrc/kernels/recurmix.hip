// Kernels of the stacks that alternate gated linear recurrences with gated latent attention (models/mixers.py:
// GatedLinearRecurrence, GatedLatentAttention; ops/seqmix.py): the causal per-channel convolution in front of the recurrence
// with its per-sequence input rows, the recurrence itself (gates, decay, state, output branch), the norms / rotation / cache
// write of the attention's latents, the rotation of its queries and its element-wise output gate.  (Attention with a sink,
// the layer norm over several stream copies, score routing and the clamped experts of these stacks are extensions of the
// kernels in seqmix.hip / hypermix.hip / dualmix.hip.)
//
// Arithmetic: convolution sums, gates, decays, the recurrent state, norm statistics and rotation angles (double until
// reduced) are fp32; activations between GEMMs are the template type float or bf16 (uint16_t bit pattern).
//
// Step metadata (int32, static device buffers): positions[T], token_seq[T] (batch row of a token, < 0: padding),
// query_start_loc[B+1], state_slots[B] (< 0: none), counts[3] = number of valid batch rows.
#include <algorithm>

#include "common.h"
#include "kernels.h"

namespace dli {

namespace {

constexpr int NT = 256;
constexpr int RM_MAX_TAPS = 64;

template <typename A> __device__ __forceinline__ float ldf(const A* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf2f(*p); }
template <typename A> __device__ __forceinline__ void stf(A* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f2bf(v); }

// sigmoid, exp and the tanh-form GELU on the hardware's exp2 / reciprocal (about one ulp each); 0.5 · (1 + tanh v) = sigmoid(2v)
__device__ __forceinline__ float sigmoid_f(float z) { return fast_rcp(1.f + fast_exp2(-1.4426950408889634f * z)); }
__device__ __forceinline__ float exp_f(float z) { return fast_exp2(1.4426950408889634f * z); }
__device__ __forceinline__ float gelu_tanh_f(float z) { return z * sigmoid_f(1.5957691216057308f * (z + 0.044715f * z * z * z)); }
// 1 − exp(x) for x ≤ 0 without the cancellation near zero (three terms of the series below 0.1: relative error < 5e-6 · x)
__device__ __forceinline__ float one_minus_exp(float x) {
  return x > -0.1f ? -x * (1.f + x * (0.5f + x * (0.16666667f + x * 0.041666668f))) : 1.f - exp_f(x);
}

// V consecutive row elements ↔ fp32: V = 4 takes 16-byte / 8-byte accesses (the launchers check divisibility and alignment)
template <typename A, int V> struct Vec {
  float v[V];
  __device__ __forceinline__ void load(const A* p) {
    if constexpr (V == 4) {
      if constexpr (sizeof(A) == 4) {
        const f32x4 t = *reinterpret_cast<const f32x4*>(p);
        v[0] = t[0]; v[1] = t[1]; v[2] = t[2]; v[3] = t[3];
      } else {
        const bf16x4 t = *reinterpret_cast<const bf16x4*>(p);
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = bf2f((uint16_t)t[j]);
      }
    } else {
#pragma unroll
      for (int j = 0; j < V; ++j) v[j] = ldf<A>(p + j);
    }
  }
  __device__ __forceinline__ void store(A* p) const {
    if constexpr (V == 4) {
      if constexpr (sizeof(A) == 4) {
        *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
      } else {
        bf16x4 t;
#pragma unroll
        for (int j = 0; j < 4; ++j) t[j] = (short)f2bf(v[j]);
        *reinterpret_cast<bf16x4*>(p) = t;
      }
    } else {
#pragma unroll
      for (int j = 0; j < V; ++j) stf<A>(p + j, v[j]);
    }
  }
};

// ------------------------------------------------------------------------------------------------ convolution
// out[t, c] = bias[c] + Σ_j w[j, c] · x[t - taps + 1 + j, c] over the rows of the token's own sequence: rows of this step's
// chunk, the sequence's state rows (its last taps-1 inputs, oldest first: positions p0-taps+1 … p0-1 for a chunk starting at
// p0) before the chunk, nothing before position 0 (so a reused slot needs no clearing).  One workgroup per token; a thread
// keeps one channel per trip, so all taps of a channel are coalesced row reads.
template <typename A, typename O, int V>
__global__ __launch_bounds__(NT) void causal_conv_kernel(const A* __restrict__ x, int64_t x_stride, const float* __restrict__ w,
                                                         const float* __restrict__ bias, int taps, const float* __restrict__ state,
                                                         const int* __restrict__ positions, const int* __restrict__ token_seq,
                                                         const int* __restrict__ qsl, const int* __restrict__ state_slots, int C,
                                                         O* __restrict__ out) {
  const int64_t t = blockIdx.x;
  const int seq = token_seq[t];
  if (seq < 0 || state_slots[seq] < 0) {                         // padding row
    for (int c = threadIdx.x; c < C; c += NT) stf<O>(out + t * C + c, 0.f);
    return;
  }
  const int p = positions[t];
  const int back = (int)t - qsl[seq];                             // rows of the chunk above this one
  const float* st = state + (int64_t)state_slots[seq] * (taps - 1) * C;
  const A* xr = x + t * x_stride;
  for (int c = threadIdx.x * V; c < C; c += NT * V) {
    Vec<float, V> a;
    if (bias != nullptr) a.load(bias + c);
    else
#pragma unroll
      for (int k = 0; k < V; ++k) a.v[k] = 0.f;
#pragma unroll 4
    for (int j = max(taps - 1 - p, 0); j < taps; ++j) {           // taps that would reach before position 0 are skipped
      const int d = taps - 1 - j;                                  // how far back the tap reaches
      Vec<float, V> v, wj;
      if (d <= back) {
        Vec<A, V> xv;
        xv.load(xr - (int64_t)d * x_stride + c);
#pragma unroll
        for (int k = 0; k < V; ++k) v.v[k] = xv.v[k];
      } else {
        v.load(st + (int64_t)(taps - 1 - (d - back)) * C + c);
      }
      wj.load(w + (int64_t)j * C + c);
#pragma unroll
      for (int k = 0; k < V; ++k) a.v[k] += wj.v[k] * v.v[k];
    }
    Vec<O, V> o;
#pragma unroll
    for (int k = 0; k < V; ++k) o.v[k] = a.v[k];
    o.store(out + t * C + c);
  }
}

// One workgroup per batch row, after the kernel above has read the old rows: the state becomes the sequence's last taps-1
// inputs.  New row r holds chunk row n-(taps-1)+r when that exists, else old row n+r (written in increasing r by the thread
// that owns the column, so an old row is read before its turn to be replaced).
template <typename A>
__global__ __launch_bounds__(NT) void conv_rows_kernel(const A* __restrict__ x, int64_t x_stride, int taps, float* __restrict__ state,
                                                       const int* __restrict__ qsl, const int* __restrict__ state_slots,
                                                       const int* __restrict__ counts, int C) {
  const int seq = blockIdx.x;
  if (seq >= counts[3]) return;
  const int slot = state_slots[seq];
  const int t0 = qsl[seq], n = qsl[seq + 1] - t0;
  if (slot < 0 || n <= 0) return;
  float* st = state + (int64_t)slot * (taps - 1) * C;
  for (int c = threadIdx.x; c < C; c += NT)
    for (int r = 0; r < taps - 1; ++r) {
      const int i = n - (taps - 1) + r;
      st[(int64_t)r * C + c] = i >= 0 ? ldf<A>(x + (int64_t)(t0 + i) * x_stride + c) : st[(int64_t)(n + r) * C + c];
    }
}

// ------------------------------------------------------------------------------------------------ recurrence
// Per (sequence of the step, channel c = b·n + j), token by token in fp32:
//   r = sigmoid(z[b, t, j] + gb[c]),  i = sigmoid(z[b, t, n + j] + gb[C + c]),  log a = -rate[c] · r,
//   S ← exp(log a) · S + sqrt(1 - exp(2 log a)) · i · u[t, c],   out[t, c] = S · gelu_tanh(y[t, c])
// with S the sequence's state row (zero at position 0), written back after its last token of the step.
//
// A work item is either a whole sequence of the step (rglru_scan_kernel: one-token rows — and every sequence when the step
// has no block list) or one 64-token block of a longer chunk (three launches, so that the blocks of a long chunk run side by
// side instead of one after the other):
//   MODE 1  per block (rglru_block_kernel): Σ log a over the block and the block's own contribution L (state from zero, no
//           output) → ws[block]
//   prefix  per sequence (rglru_prefix_kernel): walks its blocks in order, leaves in ws[block] the state at the block's START
//           and in the sequence's state slot the state after its last token: S ← exp(Σ log a) · S + L
//   MODE 2  per block: the recurrence again from ws[block], now with outputs.
// Blocks are the step's prefill tiles (tile_seq / tile_q0, 64 tokens); ws row of a block = (first token >> 6) + batch row
// (unique: rows of later sequences start at later tokens); a ws row is [2][C] = (Σ log a | L, then the start state).
//
// Whole sequences: a thread owns one channel of one sequence and fetches four tokens' operands at a time.
template <typename A, typename O>
__global__ __launch_bounds__(NT) void rglru_scan_kernel(const A* __restrict__ z, const A* __restrict__ u, const A* __restrict__ y,
                                                        int64_t y_stride, const float* __restrict__ gb, const float* __restrict__ rate,
                                                        float* __restrict__ state, const int* __restrict__ positions,
                                                        const int* __restrict__ qsl, const int* __restrict__ state_slots,
                                                        const int* __restrict__ counts, int T, int B, int n, O* __restrict__ out,
                                                        int single_only) {
  const int seq = blockIdx.y;
  if (seq >= counts[3]) return;
  const int t0 = qsl[seq], t1 = qsl[seq + 1];
  if (single_only && t1 - t0 != 1) return;                 // longer chunks take the block path
  const int slot = state_slots[seq];
  if (slot < 0 || t1 <= t0) return;
  const int C = B * n;
  const int c = blockIdx.x * NT + threadIdx.x;
  if (c >= C) return;
  const int b = c / n, j = c - b * n;
  const float br = gb[c], bi = gb[C + c], rt = rate[c];
  float* sp = state + (int64_t)slot * C + c;
  float S = positions[t0] > 0 ? *sp : 0.f;
  const A* zp = z + ((int64_t)b * T + t0) * 2 * n + j;
  for (int t = t0; t < t1; t += 4) {
    float zr[4], zi[4], uu[4], yy[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const bool live = t + k < t1;
      zr[k] = live ? ldf<A>(zp + (int64_t)k * 2 * n) : 0.f;
      zi[k] = live ? ldf<A>(zp + (int64_t)k * 2 * n + n) : 0.f;
      uu[k] = live ? ldf<A>(u + (int64_t)(t + k) * C + c) : 0.f;
      yy[k] = live ? ldf<A>(y + (int64_t)(t + k) * y_stride + c) : 0.f;
    }
    zp += 8 * n;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (t + k < t1) {
        const float la = -rt * sigmoid_f(zr[k] + br);
        S = exp_f(la) * S + sqrtf(one_minus_exp(2.f * la)) * sigmoid_f(zi[k] + bi) * uu[k];
        stf<O>(out + (int64_t)(t + k) * C + c, S * gelu_tanh_f(yy[k]));
      }
    }
  }
  *sp = S;
}

// MODE 1 / MODE 2 of a 64-token block on a workgroup of four waves over 64 channels: wave w takes the block's tokens
// 16w … 16w+15 — every operand of a wave's tokens is in flight at once, and the sequential chain is 16 steps, not 64.  Each
// wave computes its tokens' decays and inputs once (kept in registers), leaves (Σ log a, own contribution) of its quarter in
// LDS, and either wave 0 combines the four into the block's summary (MODE 1) or every wave starts from the block's start
// state advanced over the quarters before its own and writes its outputs (MODE 2).
template <typename A, typename O, int MODE>
__global__ __launch_bounds__(NT) void rglru_block_kernel(const A* __restrict__ z, const A* __restrict__ u, const A* __restrict__ y,
                                                         int64_t y_stride, const float* __restrict__ gb, const float* __restrict__ rate,
                                                         const int* __restrict__ qsl, const int* __restrict__ state_slots,
                                                         const int* __restrict__ counts, int T, int B, int n, O* __restrict__ out,
                                                         const int* __restrict__ tile_seq, const int* __restrict__ tile_q0,
                                                         int num_tiles, float* __restrict__ ws) {
  __shared__ float sLA[4][64], sL[4][64];
  const int tile = blockIdx.y;
  if (tile >= min(counts[2], num_tiles)) return;
  const int seq = tile_seq[tile];
  const int s0 = qsl[seq], s1 = qsl[seq + 1];
  if (s1 - s0 < 2 || state_slots[seq] < 0) return;           // one-token rows belong to the per-sequence kernel
  const int t0 = s0 + tile_q0[tile];
  const int t1 = min(t0 + 64, s1);
  if (t1 <= t0) return;
  const int C = B * n;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c_raw = blockIdx.x * 64 + lane;
  const bool ok = c_raw < C;
  const int c = ok ? c_raw : 0;
  const int b = c / n, j = c - b * n;
  const float br = gb[c], bi = gb[C + c], rt = rate[c];
  const int tb = t0 + 16 * wave;
  float av[16], bv[16], gv[16];
  float LA = 0.f, L = 0.f;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    float zr[4], zi[4], uu[4], yy[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int t = tb + 4 * g + k;
      const bool live = t < t1;
      const A* zp = z + ((int64_t)b * T + t) * 2 * n + j;
      zr[k] = live ? ldf<A>(zp) : 0.f;
      zi[k] = live ? ldf<A>(zp + n) : 0.f;
      uu[k] = live ? ldf<A>(u + (int64_t)t * C + c) : 0.f;
      yy[k] = (MODE == 2 && live) ? ldf<A>(y + (int64_t)t * y_stride + c) : 0.f;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const bool live = tb + 4 * g + k < t1;
      const float la = live ? -rt * sigmoid_f(zr[k] + br) : 0.f;
      const float a = exp_f(la);
      const float bb = live ? sqrtf(one_minus_exp(2.f * la)) * sigmoid_f(zi[k] + bi) * uu[k] : 0.f;
      av[4 * g + k] = a;
      bv[4 * g + k] = bb;
      gv[4 * g + k] = gelu_tanh_f(yy[k]);
      LA += la;
      L = a * L + bb;
    }
  }
  sLA[wave][lane] = LA;
  sL[wave][lane] = L;
  __syncthreads();
  float* wr = ws + ((int64_t)((t0 >> 6) + seq) * 2) * C + c;
  if (MODE == 1) {
    if (wave == 0 && ok) {
      float la = sLA[0][lane], l = sL[0][lane];
#pragma unroll
      for (int v = 1; v < 4; ++v) {
        l = exp_f(sLA[v][lane]) * l + sL[v][lane];
        la += sLA[v][lane];
      }
      wr[0] = la;
      wr[C] = l;
    }
  } else {
    if (!ok) return;
    float S = wr[C];
    for (int v = 0; v < wave; ++v) S = exp_f(sLA[v][lane]) * S + sL[v][lane];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      S = av[i] * S + bv[i];
      if (tb + i < t1) stf<O>(out + (int64_t)(tb + i) * C + c, S * gv[i]);
    }
  }
}

// per (sequence with a chunk of two tokens or more, channel): see above
__global__ __launch_bounds__(NT) void rglru_prefix_kernel(float* __restrict__ state, float* __restrict__ ws,
                                                          const int* __restrict__ positions, const int* __restrict__ qsl,
                                                          const int* __restrict__ state_slots, const int* __restrict__ counts, int C) {
  const int seq = blockIdx.y;
  if (seq >= counts[3]) return;
  const int t0 = qsl[seq], nt = qsl[seq + 1] - t0;
  const int slot = state_slots[seq];
  if (slot < 0 || nt < 2) return;
  const int c = blockIdx.x * NT + threadIdx.x;
  if (c >= C) return;
  float* sp = state + (int64_t)slot * C + c;
  float run = positions[t0] > 0 ? *sp : 0.f;
  const int blocks = (nt + 63) >> 6;
  for (int i = 0; i < blocks; ++i) {
    float* wr = ws + ((int64_t)(((t0 + 64 * i) >> 6) + seq) * 2) * C + c;
    const float la = wr[0], own = wr[C];
    wr[C] = run;
    run = exp_f(la) * run + own;
  }
  *sp = run;
}

// ------------------------------------------------------------------------------------------------ latents: norms, rotation, cache
// One workgroup per token.  proj row = [query latent (Q) | key / value latent (C) | shared key part (R) | …]: the query latent
// leaves as cq[t] = v / sqrt(mean(v²) + eps) · qw; with a cache, the key / value latent (normed the same way with cw) and the
// key part — entries i and i + rot_dims/2 turned by position · freq[i], cosine and sine times mag — go to the cache row
// slot_mapping[t] (< 0: none).
template <typename A>
__global__ __launch_bounds__(NT) void latent_norm_cache_kernel(const A* __restrict__ proj, int64_t p_stride, int Q,
                                                               const float* __restrict__ qw, const float* __restrict__ cw, float eps,
                                                               const int* __restrict__ positions, const double* __restrict__ freq,
                                                               float mag, int rot_dims, const int* __restrict__ slot_mapping,
                                                               A* __restrict__ cache, int C, int R, A* __restrict__ cq) {
  extern __shared__ float sh[];          // cos[rot_dims/2], sin[rot_dims/2]
  __shared__ float red[NT / 64];
  const int64_t t = blockIdx.x;
  const int half = rot_dims >> 1;
  const A* row = proj + t * p_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < Q; i += NT) {
    const float v = ldf<A>(row + i);
    ss += v * v;
  }
  const float qinv = 1.f / sqrtf(block_sum<NT>(ss, red) / (float)Q + eps);
  for (int i = threadIdx.x; i < Q; i += NT) stf<A>(cq + t * Q + i, ldf<A>(row + i) * qinv * qw[i]);
  if (cache == nullptr) return;
  const int slot = slot_mapping[t];
  if (slot < 0) return;                                             // whole workgroup
  const double pos = (double)positions[t];
  for (int i = threadIdx.x; i < half; i += NT) {
    double a = pos * freq[i];
    a -= 6.283185307179586476925 * floor(a * 0.15915494309189533577);    // reduced in double, then exact enough in fp32
    double sn, cs;
    sincos(a, &sn, &cs);
    sh[i] = (float)cs * mag;
    sh[half + i] = (float)sn * mag;
  }
  const A* crow = row + Q;
  ss = 0.f;
  for (int i = threadIdx.x; i < C; i += NT) {
    const float v = ldf<A>(crow + i);
    ss += v * v;
  }
  const float inv = 1.f / sqrtf(block_sum<NT>(ss, red) / (float)C + eps);      // (block_sum's barriers also publish sh)
  A* dst = cache + (int64_t)slot * (C + R);
  for (int i = threadIdx.x; i < C; i += NT) stf<A>(dst + i, ldf<A>(crow + i) * inv * cw[i]);
  for (int i = threadIdx.x; i < R; i += NT) {
    float v = ldf<A>(crow + C + i);
    if (i < half) {
      const float o = ldf<A>(crow + C + i + half);
      v = v * sh[i] - o * sh[half + i];
    } else if (i < rot_dims) {
      const float o = ldf<A>(crow + C + i - half);
      v = v * sh[i - half] + o * sh[i];
    }
    stf<A>(dst + C + i, v);
  }
}

// In place on q [T, H·(D+R)]: entries D+i and D+i+rot_dims/2 of every head turned by position · freq[i], cosine and sine
// times mag.  One workgroup per token, a thread per pair and trip (both entries read before either is written).
template <typename A>
__global__ __launch_bounds__(NT) void rotate_heads_kernel(A* __restrict__ q, int64_t q_stride, const int* __restrict__ positions,
                                                          const double* __restrict__ freq, float mag, int rot_dims, int H, int D, int R) {
  extern __shared__ float sh[];
  const int64_t t = blockIdx.x;
  const int half = rot_dims >> 1;
  const double pos = (double)positions[t];
  for (int i = threadIdx.x; i < half; i += NT) {
    double a = pos * freq[i];
    a -= 6.283185307179586476925 * floor(a * 0.15915494309189533577);
    double sn, cs;
    sincos(a, &sn, &cs);
    sh[i] = (float)cs * mag;
    sh[half + i] = (float)sn * mag;
  }
  __syncthreads();
  A* row = q + t * q_stride;
  for (int idx = threadIdx.x; idx < H * half; idx += NT) {
    const int h = idx / half, i = idx - h * half;
    A* p = row + (int64_t)h * (D + R) + D + i;
    const float a = ldf<A>(p), b = ldf<A>(p + half);
    stf<A>(p, a * sh[i] - b * sh[half + i]);
    stf<A>(p + half, b * sh[i] + a * sh[half + i]);
  }
}

// out[t, h·Dv + d] = o[h, t, d] · sigmoid(gate[t, h·Dv + d]); V entries of a head per thread and trip
template <typename A, int V>
__global__ __launch_bounds__(NT) void gate_heads_kernel(const A* __restrict__ o, const A* __restrict__ gate, int64_t g_stride, int H,
                                                        int T, int Dv, A* __restrict__ out) {
  const int64_t n = (int64_t)T * H * Dv;
  for (int64_t i = ((int64_t)blockIdx.x * NT + threadIdx.x) * V; i < n; i += (int64_t)gridDim.x * NT * V) {
    const int64_t t = i / (H * Dv);
    const int r = (int)(i - t * (H * Dv));
    const int h = r / Dv, d = r - h * Dv;
    Vec<A, V> ov, gv, res;
    ov.load(o + ((int64_t)h * T + t) * Dv + d);
    gv.load(gate + t * g_stride + r);
#pragma unroll
    for (int k = 0; k < V; ++k) res.v[k] = ov.v[k] * sigmoid_f(gv.v[k]);
    res.store(out + i);
  }
}

// out[t, :] += (Σ over the slots of token t whose id is not one of the E experts of wts[t, slot]) · h[t, :] — the identity
// experts of a routed feed-forward whose real experts ran elsewhere
template <typename A, int V>
__global__ __launch_bounds__(NT) void identity_add_kernel(A* __restrict__ out, const A* __restrict__ h, int64_t h_stride,
                                                          const int* __restrict__ ids, const float* __restrict__ wts, int K, int E, int W) {
  const int64_t t = blockIdx.x;
  float idw = 0.f;
  for (int k = 0; k < K; ++k) {
    const int e = ids[t * K + k];
    if (e < 0 || e >= E) idw += wts[t * K + k];
  }
  if (idw == 0.f) return;
  for (int c = threadIdx.x * V; c < W; c += NT * V) {
    Vec<A, V> ov, hv;
    ov.load(out + t * W + c);
    hv.load(h + t * h_stride + c);
#pragma unroll
    for (int k = 0; k < V; ++k) ov.v[k] += idw * hv.v[k];
    ov.store(out + t * W + c);
  }
}

}  // namespace

// ================================================================================================ launchers
#define RM_BF16(flag, T, ...) \
  do {                        \
    if (flag) {               \
      using T = uint16_t;     \
      __VA_ARGS__;            \
    } else {                  \
      using T = float;        \
      __VA_ARGS__;            \
    }                         \
  } while (0)

int rm_max_taps() { return RM_MAX_TAPS; }

static bool al16(const void* p) { return p == nullptr || reinterpret_cast<uintptr_t>(p) % 16 == 0; }

void launch_rm_causal_conv(const void* x, bool bf16, int64_t x_stride, const float* w, const float* bias, int taps, float* state,
                           const int* positions, const int* token_seq, const int* qsl, const int* state_slots, const int* counts,
                           int rows, int seqs, int C, void* out, bool out_bf16, hipStream_t stream) {
  if (rows == 0) return;
  if (C % 4 == 0 && x_stride % 4 == 0 && al16(x) && al16(w) && al16(bias) && al16(state) && al16(out))
    RM_BF16(bf16, A, RM_BF16(out_bf16, O, hipLaunchKernelGGL((causal_conv_kernel<A, O, 4>), dim3(rows), dim3(NT), 0, stream, (const A*)x,
                                                             x_stride, w, bias, taps, state, positions, token_seq, qsl, state_slots, C,
                                                             (O*)out)));
  else
    RM_BF16(bf16, A, RM_BF16(out_bf16, O, hipLaunchKernelGGL((causal_conv_kernel<A, O, 1>), dim3(rows), dim3(NT), 0, stream, (const A*)x,
                                                             x_stride, w, bias, taps, state, positions, token_seq, qsl, state_slots, C,
                                                             (O*)out)));
  if (taps > 1 && seqs > 0)
    RM_BF16(bf16, A, hipLaunchKernelGGL(conv_rows_kernel<A>, dim3(seqs), dim3(NT), 0, stream, (const A*)x, x_stride, taps, state, qsl,
                                        state_slots, counts, C));
}

int64_t rm_rglru_ws_floats(int rows, int seqs, int C) { return (int64_t)((rows >> 6) + seqs + 1) * 2 * C; }

void launch_rm_rglru_scan(const void* z, const void* u, const void* y, bool bf16, int64_t y_stride, const float* gate_bias,
                          const float* rate, float* state, const int* positions, const int* qsl, const int* state_slots,
                          const int* counts, int rows, int seqs, int B, int n, void* out, bool out_bf16, const int* tile_seq,
                          const int* tile_q0, int num_tiles, float* ws, hipStream_t stream) {
  if (rows == 0 || seqs == 0) return;
  const int C = B * n, cb = (C + NT - 1) / NT;
  const bool blocks = num_tiles > 0 && ws != nullptr;
#define RM_BLOCK(MODE)                                                                                                                 \
  RM_BF16(bf16, A, RM_BF16(out_bf16, O, hipLaunchKernelGGL((rglru_block_kernel<A, O, MODE>), dim3((C + 63) / 64, num_tiles), dim3(NT), 0, \
                                                           stream, (const A*)z, (const A*)u, (const A*)y, y_stride, gate_bias, rate,  \
                                                           qsl, state_slots, counts, rows, B, n, (O*)out, tile_seq, tile_q0,         \
                                                           num_tiles, ws)))
  RM_BF16(bf16, A, RM_BF16(out_bf16, O, hipLaunchKernelGGL((rglru_scan_kernel<A, O>), dim3(cb, seqs), dim3(NT), 0, stream, (const A*)z,
                                                           (const A*)u, (const A*)y, y_stride, gate_bias, rate, state, positions, qsl,
                                                           state_slots, counts, rows, B, n, (O*)out, blocks ? 1 : 0)));
  if (blocks) {
    RM_BLOCK(1);
    hipLaunchKernelGGL(rglru_prefix_kernel, dim3(cb, seqs), dim3(NT), 0, stream, state, ws, positions, qsl, state_slots, counts, C);
    RM_BLOCK(2);
  }
#undef RM_BLOCK
}

void launch_rm_latent_norm_cache(const void* proj, bool bf16, int64_t p_stride, int Q, const float* qw, const float* cw, float eps,
                                 const int* positions, const double* freq, float mag, int rot_dims, const int* slot_mapping, void* cache,
                                 int rows, int C, int R, void* cq, hipStream_t stream) {
  if (rows == 0) return;
  RM_BF16(bf16, A, hipLaunchKernelGGL(latent_norm_cache_kernel<A>, dim3(rows), dim3(NT), std::max(rot_dims, 2) * sizeof(float), stream,
                                      (const A*)proj, p_stride, Q, qw, cw, eps, positions, freq, mag, rot_dims, slot_mapping, (A*)cache,
                                      C, R, (A*)cq));
}

void launch_rm_rotate_heads(void* q, bool bf16, int64_t q_stride, const int* positions, const double* freq, float mag, int rot_dims,
                            int rows, int H, int D, int R, hipStream_t stream) {
  if (rows == 0 || rot_dims == 0) return;
  RM_BF16(bf16, A, hipLaunchKernelGGL(rotate_heads_kernel<A>, dim3(rows), dim3(NT), rot_dims * sizeof(float), stream, (A*)q, q_stride,
                                      positions, freq, mag, rot_dims, H, D, R));
}

void launch_rm_identity_add(void* out, const void* h, bool bf16, int64_t h_stride, const int* ids, const float* wts, int K, int E,
                            int rows, int W, hipStream_t stream) {
  if (rows == 0) return;
  if (W % 4 == 0 && h_stride % 4 == 0 && al16(out) && al16(h))
    RM_BF16(bf16, A, hipLaunchKernelGGL((identity_add_kernel<A, 4>), dim3(rows), dim3(NT), 0, stream, (A*)out, (const A*)h, h_stride, ids,
                                        wts, K, E, W));
  else
    RM_BF16(bf16, A, hipLaunchKernelGGL((identity_add_kernel<A, 1>), dim3(rows), dim3(NT), 0, stream, (A*)out, (const A*)h, h_stride, ids,
                                        wts, K, E, W));
}

void launch_rm_gate_heads(const void* o, const void* gate, bool bf16, int64_t g_stride, int H, int rows, int Dv, void* out,
                          hipStream_t stream) {
  const int64_t n = (int64_t)rows * H * Dv;
  if (n == 0) return;
  const bool wide = Dv % 4 == 0 && g_stride % 4 == 0 && al16(o) && al16(gate) && al16(out);
  const int64_t items = wide ? n / 4 : n;
  const int blocks = (int)std::min<int64_t>((items + NT - 1) / NT, 16384);
  if (wide)
    RM_BF16(bf16, A, hipLaunchKernelGGL((gate_heads_kernel<A, 4>), dim3(blocks), dim3(NT), 0, stream, (const A*)o, (const A*)gate, g_stride,
                                        H, rows, Dv, (A*)out));
  else
    RM_BF16(bf16, A, hipLaunchKernelGGL((gate_heads_kernel<A, 1>), dim3(blocks), dim3(NT), 0, stream, (const A*)o, (const A*)gate, g_stride,
                                        H, rows, Dv, (A*)out));
}

}  // namespace dli
