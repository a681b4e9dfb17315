// Kernels of the hyper-connected stacks (models/mixers.py: HyperLayer, Retention, GatedDenseFF, SoftmaxRoutedFF;
// ops/seqmix.py): the write-back / read / RMS norm over several fp32 copies of the residual stream, the causal per-channel
// convolution in front of a mixer with its per-sequence input rows, rotation and key scale of retention's q / k, the gated
// feed-forward activation and softmax-over-the-chosen routing.  (Attention, the decayed scan, the per-head unit norm and the
// experts of these stacks are extensions of the kernels in seqmix.hip / dualmix.hip / moe.hip.)
//
// Arithmetic: streams, norm statistics, convolution inputs and state, rotation angles (double until reduced), router logits
// and weights are fp32; activations handed to GEMMs are the template type float or bf16 (uint16_t bit pattern).
//
// Step metadata (int32, static device buffers): positions[T], token_seq[T] (batch row of a token, < 0: padding),
// query_start_loc[B+1], state_slots[B] (< 0: none), counts[3] = number of valid batch rows.
#include <algorithm>

#include "common.h"
#include "kernels.h"

namespace dli {

namespace {

constexpr int NT = 256;
constexpr int HM_MAX_S = 16;      // copies of the stream
constexpr int HM_MAX_TAPS = 64;   // taps of the input convolution

template <typename A> __device__ __forceinline__ float ldf(const A* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf2f(*p); }
template <typename A> __device__ __forceinline__ void stf(A* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f2bf(v); }

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

// ------------------------------------------------------------------------------------------------ streams: write, read, norm
// One workgroup per token over x [T, S, W].  With y: x_t ← Σ_s mix[s, t] x_s + out_w[t] · y for all t at once (every column's
// S values are read before any is written).  With in_w: u = Σ_s in_w[s] x_s of the updated streams is kept in LDS and leaves
// as u / sqrt(mean(u²) + eps) · (w_offset + norm_w) — or, with `center`, as the layer norm (u − mean) / sqrt(var + eps) ·
// (w_offset + norm_w), the variance taken over the deviations in a second pass over the LDS row.  MS: compile-time bound of S;
// a thread takes V columns per trip.
template <typename Y, typename O, int MS, int V>
__global__ __launch_bounds__(NT) void stream_mix_norm_kernel(float* __restrict__ x, const Y* __restrict__ y, int64_t y_stride,
                                                             const float* __restrict__ mix, const float* __restrict__ out_w,
                                                             const float* __restrict__ in_w, const float* __restrict__ norm_w,
                                                             float eps, float w_offset, int S, int W, O* __restrict__ out,
                                                             int center) {
  extern __shared__ float us[];
  __shared__ float red[NT / 64];
  __shared__ float cm[MS * MS], co[MS], ci[MS];
  const int64_t t = blockIdx.x;
  if (threadIdx.x < S * S && y != nullptr) cm[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    co[threadIdx.x] = y != nullptr ? out_w[threadIdx.x] : 0.f;
    ci[threadIdx.x] = in_w != nullptr ? in_w[threadIdx.x] : 0.f;
  }
  __syncthreads();
  float* xr = x + t * S * W;
  float sq = 0.f, su = 0.f;
  for (int c = threadIdx.x * V; c < W; c += NT * V) {
    Vec<float, V> xs[MS];
#pragma unroll
    for (int s = 0; s < MS; ++s)
      if (s < S) xs[s].load(xr + (int64_t)s * W + c);
    if (y != nullptr) {
      Vec<Y, V> yv;
      yv.load(y + t * y_stride + c);
      Vec<float, V> nx[MS];
#pragma unroll
      for (int to = 0; to < MS; ++to) {
        if (to < S) {
#pragma unroll
          for (int j = 0; j < V; ++j) nx[to].v[j] = co[to] * yv.v[j];
#pragma unroll
          for (int s = 0; s < MS; ++s)
            if (s < S) {
              const float m = cm[s * S + to];
#pragma unroll
              for (int j = 0; j < V; ++j) nx[to].v[j] += m * xs[s].v[j];
            }
        }
      }
#pragma unroll
      for (int to = 0; to < MS; ++to)
        if (to < S) {
          nx[to].store(xr + (int64_t)to * W + c);
          xs[to] = nx[to];
        }
    }
    if (in_w != nullptr) {
#pragma unroll
      for (int j = 0; j < V; ++j) {
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < MS; ++s)
          if (s < S) u += ci[s] * xs[s].v[j];
        us[c + j] = u;
        sq += u * u;
        su += u;
      }
    }
  }
  if (in_w == nullptr) return;
  float mean = 0.f;
  if (center) {                                                   // every thread re-reads the columns it wrote itself
    mean = block_sum<NT>(su, red) / (float)W;
    sq = 0.f;
    for (int c = threadIdx.x * V; c < W; c += NT * V)
#pragma unroll
      for (int j = 0; j < V; ++j) {
        const float d = us[c + j] - mean;
        sq += d * d;
      }
  }
  const float inv = 1.f / sqrtf(block_sum<NT>(sq, red) / (float)W + eps);
  for (int c = threadIdx.x * V; c < W; c += NT * V) {
    Vec<float, V> nw;
    nw.load(norm_w + c);
    Vec<O, V> o;
#pragma unroll
    for (int j = 0; j < V; ++j) o.v[j] = (us[c + j] - mean) * inv * (w_offset + nw.v[j]);
    o.store(out + t * W + c);
  }
}

// ------------------------------------------------------------------------------------------------ input convolution
// out[t] = h[t] + Σ_j w[j, :] · h[t - taps + 1 + j] (w [taps, W]: a tap's weights are one contiguous row) over the rows of the token's own sequence: rows of this step's chunk, the
// sequence's state rows (its last taps-1 inputs, oldest first: positions p0-taps+1 … p0-1 for a chunk starting at p0) before
// the chunk, zero before position 0 (so a reused slot needs no clearing).  One workgroup per token, V columns per thread and trip.
template <typename O, int V>
__global__ __launch_bounds__(NT) void causal_conv_add_kernel(const float* __restrict__ h, const float* __restrict__ w, int taps,
                                                             const float* __restrict__ state, const int* __restrict__ positions,
                                                             const int* __restrict__ token_seq, const int* __restrict__ qsl,
                                                             const int* __restrict__ state_slots, int W, O* __restrict__ out) {
  const int64_t t = blockIdx.x;
  const int seq = token_seq[t];
  const float* hr = h + t * W;
  if (seq < 0 || state_slots[seq] < 0) {                         // padding row
    for (int c = threadIdx.x * V; c < W; c += NT * V) {
      Vec<float, V> a;
      a.load(hr + c);
      Vec<O, V> o;
#pragma unroll
      for (int j = 0; j < V; ++j) o.v[j] = a.v[j];
      o.store(out + t * W + c);
    }
    return;
  }
  const int p = positions[t];
  const int t0 = qsl[seq];
  const int back = (int)t - t0;                                   // rows of the chunk above this one
  const float* st = state + (int64_t)state_slots[seq] * (taps - 1) * W;
  for (int c = threadIdx.x * V; c < W; c += NT * V) {
    Vec<float, V> a;
    a.load(hr + c);
#pragma unroll 4
    for (int j = max(taps - 1 - p, 0); j < taps; ++j) {          // taps that would reach before position 0 are skipped
      const int d = taps - 1 - j;                                 // how far back the tap reaches
      // state row of position p - d: its index counts from the chunk's first position minus (taps - 1)
      Vec<float, V> v, wj;
      v.load(d <= back ? hr + c - (int64_t)d * W : st + (int64_t)(taps - 1 - (d - back)) * W + c);
      wj.load(w + (int64_t)j * W + c);
#pragma unroll
      for (int k = 0; k < V; ++k) a.v[k] += wj.v[k] * v.v[k];
    }
    Vec<O, V> o;
#pragma unroll
    for (int k = 0; k < V; ++k) o.v[k] = a.v[k];
    o.store(out + t * W + c);
  }
}

// One workgroup per batch row, after the kernel above has read the old rows: the state becomes the sequence's last taps-1
// inputs.  New row r holds chunk row n-(taps-1)+r when that exists, else old row n+r (written in increasing r by the thread
// that owns the column, so an old row is read before its turn to be replaced).
__global__ __launch_bounds__(NT) void conv_state_kernel(const float* __restrict__ h, int taps, float* __restrict__ state,
                                                        const int* __restrict__ qsl, const int* __restrict__ state_slots,
                                                        const int* __restrict__ counts, int W) {
  const int seq = blockIdx.x;
  if (seq >= counts[3]) return;
  const int slot = state_slots[seq];
  const int t0 = qsl[seq], n = qsl[seq + 1] - t0;
  if (slot < 0 || n <= 0) return;
  float* st = state + (int64_t)slot * (taps - 1) * W;
  for (int c = threadIdx.x; c < W; c += NT)
    for (int r = 0; r < taps - 1; ++r) {
      const int i = n - (taps - 1) + r;
      st[(int64_t)r * W + c] = i >= 0 ? h[(int64_t)(t0 + i) * W + c] : st[(int64_t)(n + r) * W + c];
    }
}

// ------------------------------------------------------------------------------------------------ retention: rotation, key scale
// out [T, 2·H·D + H·Dv] fp32 = [q' | k' | v]: entries i and i + rot_dims/2 (i < rot_dims/2) of every q and k head turned by
// position · freq[i]; k' also times k_scale.  One workgroup per token: first the rotated pairs (a thread reads and writes both
// entries of a pair), then everything that passes unchanged, V entries at a time.
template <typename A, int V>
__global__ __launch_bounds__(NT) void retention_prep_kernel(const A* __restrict__ qkvg, int64_t row_stride,
                                                            const int* __restrict__ positions, const double* __restrict__ freq,
                                                            int rot_dims, int H, int D, int Dv, float k_scale,
                                                            float* __restrict__ out) {
  extern __shared__ float cs[];                                   // cos [half] | sin [half]
  const int64_t t = blockIdx.x;
  const int half = rot_dims >> 1;
  float* sn = cs + half;
  for (int i = threadIdx.x; i < half; i += NT) {
    const double two_pi = 6.283185307179586476925286766559;
    double a = (double)positions[t] * freq[i];
    a -= floor(a / two_pi) * two_pi;
    cs[i] = cosf((float)a);
    sn[i] = sinf((float)a);
  }
  __syncthreads();
  const A* row = qkvg + t * row_stride;
  const int nqk = 2 * H * D, n = nqk + H * Dv;
  float* orow = out + t * n;
#pragma unroll 4
  for (int p = threadIdx.x; p < 2 * H * half; p += NT) {
    const int hh = p / half, i = p - hh * half;
    const int e = hh * D + i;
    const float a = ldf<A>(row + e), b = ldf<A>(row + e + half);
    const float m = hh >= H ? k_scale : 1.f;
    orow[e] = (a * cs[i] - b * sn[i]) * m;
    orow[e + half] = (b * cs[i] + a * sn[i]) * m;
  }
  // the unrotated tail of every q / k head
  const int tail = D - rot_dims;
#pragma unroll 4
  for (int p = threadIdx.x; p < 2 * H * tail; p += NT) {
    const int hh = p / tail, e = hh * D + rot_dims + (p - hh * tail);
    orow[e] = ldf<A>(row + e) * (hh >= H ? k_scale : 1.f);
  }
  for (int i = threadIdx.x * V; i < H * Dv; i += NT * V) {
    Vec<A, V> a;
    a.load(row + nqk + i);
    Vec<float, V> o;
#pragma unroll
    for (int j = 0; j < V; ++j) o.v[j] = a.v[j];
    o.store(orow + nqk + i);
  }
}

// ------------------------------------------------------------------------------------------------ gated activation
// out[r, f] = act(x[r, f]) · x[r, F + f]; act: tanh-form GELU, or silu.  V entries per thread and trip.
template <typename A, int V>
__global__ __launch_bounds__(NT) void act_mul_kernel(const A* __restrict__ x, int64_t x_stride, int F, int64_t n, int silu,
                                                     A* __restrict__ out) {
  for (int64_t i = ((int64_t)blockIdx.x * NT + threadIdx.x) * V; i < n; i += (int64_t)gridDim.x * NT * V) {
    const int64_t r = i / F;
    const int f = (int)(i - r * F);
    Vec<A, V> z, u, o;
    z.load(x + r * x_stride + f);
    u.load(x + r * x_stride + F + f);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float zz = z.v[j];
      const float a = silu ? zz / (1.f + expf(-zz)) : 0.5f * zz * (1.f + tanhf(0.7978845608028654f * (zz + 0.044715f * zz * zz * zz)));
      o.v[j] = a * u.v[j];
    }
    o.store(out + i);
  }
}

// ------------------------------------------------------------------------------------------------ softmax routing
// One workgroup per TPB tokens (their rows in LDS): fp32 logits router · h + bias — a wave per expert row, which it reads once
// for all TPB tokens — then wave k picks token k's top-k logits (ties → lowest expert id) and normalises exp(logit − largest)
// over the picks.  Every pass takes an expert that is still free, whatever the logits hold (a row of padding can carry NaNs;
// an id outside the experts would index past their weights).  V router entries per lane and trip.
// `all`: the scores are the softmax over ALL E logits; `bias` is not part of the logits but added to the scores for the choice
// only, and the weights are the chosen scores divided by their sum (+ 1e-20).
template <typename A, int TPB, int V>
__global__ __launch_bounds__(NT) void softmax_route_kernel(const A* __restrict__ h, int64_t h_stride, const float* __restrict__ router,
                                                           const float* __restrict__ bias, int E, int K, int T, int W,
                                                           int* __restrict__ ids, float* __restrict__ wts, int all) {
  extern __shared__ float sh[];                                   // TPB rows of W
  __shared__ float z[TPB][64];
  const int64_t tb = (int64_t)blockIdx.x * TPB;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int k = 0; k < TPB; ++k) {
    const bool live = tb + k < T;
    for (int i = threadIdx.x * V; i < W; i += NT * V) {
      Vec<A, V> a;
      if (live) a.load(h + (tb + k) * h_stride + i);
#pragma unroll
      for (int j = 0; j < V; ++j) sh[k * W + i + j] = live ? a.v[j] : 0.f;
    }
  }
  __syncthreads();
  for (int r = wave; r < E; r += NT / 64) {
    float d[TPB];
#pragma unroll
    for (int k = 0; k < TPB; ++k) d[k] = 0.f;
#pragma unroll 4
    for (int i = lane * V; i < W; i += 64 * V) {
      Vec<float, V> rw;
      rw.load(router + (int64_t)r * W + i);
#pragma unroll
      for (int k = 0; k < TPB; ++k)
#pragma unroll
        for (int j = 0; j < V; ++j) d[k] += sh[k * W + i + j] * rw.v[j];
    }
    const float b = bias != nullptr && !all ? bias[r] : 0.f;
#pragma unroll
    for (int k = 0; k < TPB; ++k) {
      const float s = wave_sum(d[k]);
      if (lane == 0) z[k][r] = s + b;
    }
  }
  __syncthreads();
  for (int k = wave; k < TPB; k += NT / 64) {
    const int64_t t = tb + k;
    if (t >= T) continue;                                         // whole wave
    float p = -INFINITY;
    if (lane < E) {
      const float v = z[k][lane];
      p = v == v ? v : -INFINITY;
    }
    float score = 0.f;
    if (all) {
      const float mx = wave_max(p);
      const float ex = (lane < E && mx != -INFINITY) ? expf(p - mx) : 0.f;
      const float tot = wave_sum(ex);
      score = tot > 0.f ? ex / tot : 0.f;
      if (lane < E) p = score + (bias != nullptr ? bias[lane] : 0.f);
      if (!(p == p)) p = -INFINITY;
    }
    bool free_lane = lane < E;
    float my_v = -INFINITY, top_v = -INFINITY;
    int my_id = 0;
    for (int kk = 0; kk < K; ++kk) {
      float bv = free_lane ? p : -INFINITY;
      int bi = free_lane ? lane : 64 + lane;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, 64);
        const int oi = __shfl_xor(bi, o, 64);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
      }
      if (kk == 0) top_v = bv;
      const float sv = __shfl(score, min(bi, E - 1) & 63, 64);        // the chosen output's score (softmax over all)
      if (lane == kk) { my_v = all ? sv : bv; my_id = min(bi, E - 1); }
      if (lane == bi) free_lane = false;
    }
    float e = 0.f;
    if (all) {
      if (lane < K) e = my_v;
    } else if (lane < K) {
      e = top_v == -INFINITY ? 1.f : expf(my_v - top_v);                // no finite logit at all: equal shares
    }
    const float sum = wave_sum(e) + (all ? 1e-20f : 0.f);
    if (lane < K) {
      ids[t * K + lane] = my_id;
      wts[t * K + lane] = e / sum;
    }
  }
}

}  // namespace

// ================================================================================================ launchers
#define HM_BF16(flag, T, ...) \
  do {                        \
    if (flag) {               \
      using T = uint16_t;     \
      __VA_ARGS__;            \
    } else {                  \
      using T = float;        \
      __VA_ARGS__;            \
    }                         \
  } while (0)

int hm_max_streams() { return HM_MAX_S; }
int hm_max_taps() { return HM_MAX_TAPS; }

static bool al16(const void* p) { return p == nullptr || reinterpret_cast<uintptr_t>(p) % 16 == 0; }

void launch_hm_stream_mix_norm(float* x, const void* y, bool y_bf16, int64_t y_stride, const float* mix, const float* out_w,
                               const float* in_w, const float* norm_w, float eps, float w_offset, int rows, int S, int W, void* out,
                               bool out_bf16, bool center, hipStream_t stream) {
  if (rows == 0) return;
  const size_t lds = in_w != nullptr ? (size_t)W * sizeof(float) : 0;
  const bool wide = W % 4 == 0 && y_stride % 4 == 0 && al16(x) && al16(y) && al16(norm_w) && al16(out);
#define HM_SMN(MS, V)                                                                                                               \
  HM_BF16(y_bf16, Y, HM_BF16(out_bf16, O, hipLaunchKernelGGL((stream_mix_norm_kernel<Y, O, MS, V>), dim3(rows), dim3(NT), lds, stream, \
                                                             x, (const Y*)y, y_stride, mix, out_w, in_w, norm_w, eps, w_offset, S, \
                                                             W, (O*)out, center ? 1 : 0)))
#define HM_SMN_S(V)            \
  do {                         \
    if (S <= 2) HM_SMN(2, V);  \
    else if (S <= 4) HM_SMN(4, V); \
    else if (S <= 8) HM_SMN(8, V); \
    else HM_SMN(16, V);        \
  } while (0)
  if (wide) HM_SMN_S(4);
  else HM_SMN_S(1);
#undef HM_SMN_S
#undef HM_SMN
}

void launch_hm_causal_conv_add(const float* h, const float* w, int taps, float* state, const int* positions, const int* token_seq,
                               const int* qsl, const int* state_slots, const int* counts, int rows, int seqs, int W, void* out,
                               bool out_bf16, hipStream_t stream) {
  if (rows == 0) return;
  if (W % 4 == 0 && al16(h) && al16(state) && al16(out) && al16(w))
    HM_BF16(out_bf16, O, hipLaunchKernelGGL((causal_conv_add_kernel<O, 4>), dim3(rows), dim3(NT), 0, stream, h, w, taps, state, positions,
                                            token_seq, qsl, state_slots, W, (O*)out));
  else
    HM_BF16(out_bf16, O, hipLaunchKernelGGL((causal_conv_add_kernel<O, 1>), dim3(rows), dim3(NT), 0, stream, h, w, taps, state, positions,
                                            token_seq, qsl, state_slots, W, (O*)out));
  if (taps > 1 && seqs > 0)
    hipLaunchKernelGGL(conv_state_kernel, dim3(seqs), dim3(NT), 0, stream, h, taps, state, qsl, state_slots, counts, W);
}

void launch_hm_retention_prep(const void* qkvg, bool bf16, int64_t row_stride, const int* positions, const double* freq, int rot_dims,
                              int rows, int H, int D, int Dv, float k_scale, float* out, hipStream_t stream) {
  if (rows == 0) return;
  const size_t lds = (size_t)rot_dims * sizeof(float);
  const bool wide = (H * Dv) % 4 == 0 && (2 * H * D) % 4 == 0 && row_stride % 4 == 0 && al16(qkvg) && al16(out);
  if (wide)
    HM_BF16(bf16, A, hipLaunchKernelGGL((retention_prep_kernel<A, 4>), dim3(rows), dim3(NT), lds, stream, (const A*)qkvg, row_stride,
                                        positions, freq, rot_dims, H, D, Dv, k_scale, out));
  else
    HM_BF16(bf16, A, hipLaunchKernelGGL((retention_prep_kernel<A, 1>), dim3(rows), dim3(NT), lds, stream, (const A*)qkvg, row_stride,
                                        positions, freq, rot_dims, H, D, Dv, k_scale, out));
}

void launch_hm_act_mul(const void* x, bool bf16, int64_t x_stride, int rows, int F, bool silu, void* out, hipStream_t stream) {
  const int64_t n = (int64_t)rows * F;
  if (n == 0) return;
  const bool wide = F % 4 == 0 && x_stride % 4 == 0 && al16(x) && al16(out);
  const int64_t items = wide ? n / 4 : n;
  const int blocks = (int)std::min<int64_t>((items + NT - 1) / NT, 16384);
  if (wide)
    HM_BF16(bf16, A, hipLaunchKernelGGL((act_mul_kernel<A, 4>), dim3(blocks), dim3(NT), 0, stream, (const A*)x, x_stride, F, n,
                                        silu ? 1 : 0, (A*)out));
  else
    HM_BF16(bf16, A, hipLaunchKernelGGL((act_mul_kernel<A, 1>), dim3(blocks), dim3(NT), 0, stream, (const A*)x, x_stride, F, n,
                                        silu ? 1 : 0, (A*)out));
}

void launch_hm_softmax_route(const void* h, bool bf16, int64_t h_stride, const float* router, const float* bias, int E, int K, int rows,
                             int W, int* ids, float* wts, bool all, hipStream_t stream) {
  if (rows == 0) return;
  const bool wide = W % 4 == 0 && h_stride % 4 == 0 && al16(h) && al16(router);
  // four tokens share a pass over the router rows where their inputs fit the LDS budget together
  const bool four = (size_t)W * 4 * sizeof(float) <= 60 * 1024;
#define HM_ROUTE(TPB, V)                                                                                                      \
  HM_BF16(bf16, A, hipLaunchKernelGGL((softmax_route_kernel<A, TPB, V>), dim3((rows + TPB - 1) / TPB), dim3(NT),              \
                                      (size_t)TPB * W * sizeof(float), stream, (const A*)h, h_stride, router, bias, E, K, rows, W, \
                                      ids, wts, all ? 1 : 0))
  if (four && wide) HM_ROUTE(4, 4);
  else if (four) HM_ROUTE(4, 1);
  else if (wide) HM_ROUTE(1, 4);
  else HM_ROUTE(1, 1);
#undef HM_ROUTE
}

}  // namespace dli
