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
constexpr int HM_MAX_S = 8;       // copies of the stream
constexpr int HM_MAX_TAPS = 8;    // taps of the input convolution

template <typename A> __device__ __forceinline__ float ldf(const A* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p) { return bf2f(*p); }
template <typename A> __device__ __forceinline__ void stf(A* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<uint16_t>(uint16_t* p, float v) { *p = f2bf(v); }

// ------------------------------------------------------------------------------------------------ streams: write, read, norm
// One workgroup per token over x [T, S, W].  With y: x_t ← Σ_s mix[s, t] x_s + out_w[t] · y for all t at once (every column's
// S values are read before any is written).  With in_w: u = Σ_s in_w[s] x_s of the updated streams is kept in LDS and leaves
// as u / sqrt(mean(u²) + eps) · (w_offset + norm_w).
template <typename Y, typename O>
__global__ __launch_bounds__(NT) void stream_mix_norm_kernel(float* __restrict__ x, const Y* __restrict__ y, int64_t y_stride,
                                                             const float* __restrict__ mix, const float* __restrict__ out_w,
                                                             const float* __restrict__ in_w, const float* __restrict__ norm_w,
                                                             float eps, float w_offset, int S, int W, O* __restrict__ out) {
  extern __shared__ float us[];
  __shared__ float red[NT / 64];
  __shared__ float cm[HM_MAX_S * HM_MAX_S], co[HM_MAX_S], ci[HM_MAX_S];
  const int64_t t = blockIdx.x;
  if (threadIdx.x < S * S && y != nullptr) cm[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    co[threadIdx.x] = y != nullptr ? out_w[threadIdx.x] : 0.f;
    ci[threadIdx.x] = in_w != nullptr ? in_w[threadIdx.x] : 0.f;
  }
  __syncthreads();
  float* xr = x + t * S * W;
  float sq = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) {
    float xs[HM_MAX_S];
#pragma unroll
    for (int s = 0; s < HM_MAX_S; ++s) xs[s] = s < S ? xr[(int64_t)s * W + c] : 0.f;
    if (y != nullptr) {
      const float yv = ldf<Y>(y + t * y_stride + c);
      float nx[HM_MAX_S];
#pragma unroll
      for (int to = 0; to < HM_MAX_S; ++to) {
        float a = 0.f;
        if (to < S) {
          a = co[to] * yv;
#pragma unroll
          for (int s = 0; s < HM_MAX_S; ++s)
            if (s < S) a += cm[s * S + to] * xs[s];
          xr[(int64_t)to * W + c] = a;
        }
        nx[to] = a;
      }
#pragma unroll
      for (int s = 0; s < HM_MAX_S; ++s) xs[s] = nx[s];
    }
    if (in_w != nullptr) {
      float u = 0.f;
#pragma unroll
      for (int s = 0; s < HM_MAX_S; ++s)
        if (s < S) u += ci[s] * xs[s];
      us[c] = u;
      sq += u * u;
    }
  }
  if (in_w == nullptr) return;
  const float inv = 1.f / sqrtf(block_sum<NT>(sq, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += NT) stf<O>(out + t * W + c, us[c] * inv * (w_offset + norm_w[c]));
}

// ------------------------------------------------------------------------------------------------ input convolution
// out[t] = h[t] + Σ_j w[:, j] · h[t - taps + 1 + j] over the rows of the token's own sequence: rows of this step's chunk, the
// sequence's state rows (its last taps-1 inputs, oldest first: positions p0-taps+1 … p0-1 for a chunk starting at p0) before
// the chunk, zero before position 0 (so a reused slot needs no clearing).  One workgroup per token.
template <typename O>
__global__ __launch_bounds__(NT) void causal_conv_add_kernel(const float* __restrict__ h, const float* __restrict__ w, int taps,
                                                             const float* __restrict__ state, const int* __restrict__ positions,
                                                             const int* __restrict__ token_seq, const int* __restrict__ qsl,
                                                             const int* __restrict__ state_slots, int W, O* __restrict__ out) {
  const int64_t t = blockIdx.x;
  const int seq = token_seq[t];
  const float* hr = h + t * W;
  if (seq < 0 || state_slots[seq] < 0) {                         // padding row
    for (int c = threadIdx.x; c < W; c += NT) stf<O>(out + t * W + c, hr[c]);
    return;
  }
  const int p = positions[t];
  const int t0 = qsl[seq];
  const int back = (int)t - t0;                                   // rows of the chunk above this one
  const float* st = state + (int64_t)state_slots[seq] * (taps - 1) * W;
  for (int c = threadIdx.x; c < W; c += NT) {
    float a = hr[c];
    for (int j = 0; j < taps; ++j) {
      const int d = taps - 1 - j;                                 // how far back the tap reaches
      if (p - d < 0) continue;
      // state row of position p - d: its index counts from the chunk's first position minus (taps - 1)
      const float v = d <= back ? hr[c - (int64_t)d * W] : st[(int64_t)(taps - 1 - (d - back)) * W + c];
      a += w[c * taps + j] * v;
    }
    stf<O>(out + t * W + c, a);
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
// position · freq[i]; k' also times k_scale.  One workgroup per token.
template <typename A>
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
  for (int i = threadIdx.x; i < n; i += NT) {
    float v = ldf<A>(row + i);
    if (i < nqk) {
      const int d = i % D;
      if (d < half) v = v * cs[d] - ldf<A>(row + i + half) * sn[d];
      else if (d < rot_dims) v = v * cs[d - half] + ldf<A>(row + i - half) * sn[d - half];
      if (i >= H * D) v *= k_scale;
    }
    orow[i] = v;
  }
}

// ------------------------------------------------------------------------------------------------ gated activation
// out[r, f] = act(x[r, f]) · x[r, F + f]; act: tanh-form GELU, or silu
template <typename A>
__global__ __launch_bounds__(NT) void act_mul_kernel(const A* __restrict__ x, int64_t x_stride, int F, int64_t n, int silu,
                                                     A* __restrict__ out) {
  for (int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x; i < n; i += (int64_t)gridDim.x * NT) {
    const int64_t r = i / F;
    const int f = (int)(i - r * F);
    const float z = ldf<A>(x + r * x_stride + f), u = ldf<A>(x + r * x_stride + F + f);
    float a;
    if (silu) a = z / (1.f + expf(-z));
    else a = 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    stf<A>(out + i, a * u);
  }
}

// ------------------------------------------------------------------------------------------------ softmax routing
// One workgroup per token: fp32 logits router · h + bias (a wave per expert row), then wave 0 picks the top-k logits (ties →
// lowest expert id) and normalises exp(logit − largest) over the picks.  Every pass takes an expert that is still free,
// whatever the logits hold (a row of padding can carry NaNs; an id outside the experts would index past their weights).
template <typename A>
__global__ __launch_bounds__(NT) void softmax_route_kernel(const A* __restrict__ h, int64_t h_stride, const float* __restrict__ router,
                                                           const float* __restrict__ bias, int E, int K, int W,
                                                           int* __restrict__ ids, float* __restrict__ wts) {
  extern __shared__ float sh[];
  __shared__ float z[64];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < W; i += NT) sh[i] = ldf<A>(h + t * h_stride + i);
  __syncthreads();
  for (int r = wave; r < E; r += NT / 64) {
    float d = 0.f;
    for (int i = lane; i < W; i += 64) d += sh[i] * router[(int64_t)r * W + i];
    d = wave_sum(d);
    if (lane == 0) z[r] = d + (bias != nullptr ? bias[r] : 0.f);
  }
  __syncthreads();
  if (wave != 0) return;
  float p = -INFINITY;
  if (lane < E) {
    const float v = z[lane];
    p = v == v ? v : -INFINITY;
  }
  bool free_lane = lane < E;
  float my_v = -INFINITY, top_v = -INFINITY;
  int my_id = 0;
  for (int k = 0; k < K; ++k) {
    float bv = free_lane ? p : -INFINITY;
    int bi = free_lane ? lane : 64 + lane;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (k == 0) top_v = bv;
    if (lane == k) { my_v = bv; my_id = min(bi, E - 1); }
    if (lane == bi) free_lane = false;
  }
  float e = 0.f;
  if (lane < K) e = top_v == -INFINITY ? 1.f : expf(my_v - top_v);      // no finite logit at all: equal shares
  const float sum = wave_sum(e);
  if (lane < K) {
    ids[t * K + lane] = my_id;
    wts[t * K + lane] = e / sum;
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

void launch_hm_stream_mix_norm(float* x, const void* y, bool y_bf16, int64_t y_stride, const float* mix, const float* out_w,
                               const float* in_w, const float* norm_w, float eps, float w_offset, int rows, int S, int W, void* out,
                               bool out_bf16, hipStream_t stream) {
  if (rows == 0) return;
  const size_t lds = in_w != nullptr ? (size_t)W * sizeof(float) : 0;
  HM_BF16(y_bf16, Y, HM_BF16(out_bf16, O, hipLaunchKernelGGL((stream_mix_norm_kernel<Y, O>), dim3(rows), dim3(NT), lds, stream, x,
                                                             (const Y*)y, y_stride, mix, out_w, in_w, norm_w, eps, w_offset, S, W,
                                                             (O*)out)));
}

void launch_hm_causal_conv_add(const float* h, const float* w, int taps, float* state, const int* positions, const int* token_seq,
                               const int* qsl, const int* state_slots, const int* counts, int rows, int seqs, int W, void* out,
                               bool out_bf16, hipStream_t stream) {
  if (rows == 0) return;
  HM_BF16(out_bf16, O, hipLaunchKernelGGL(causal_conv_add_kernel<O>, dim3(rows), dim3(NT), 0, stream, h, w, taps, state, positions,
                                          token_seq, qsl, state_slots, W, (O*)out));
  if (taps > 1 && seqs > 0)
    hipLaunchKernelGGL(conv_state_kernel, dim3(seqs), dim3(NT), 0, stream, h, taps, state, qsl, state_slots, counts, W);
}

void launch_hm_retention_prep(const void* qkvg, bool bf16, int64_t row_stride, const int* positions, const double* freq, int rot_dims,
                              int rows, int H, int D, int Dv, float k_scale, float* out, hipStream_t stream) {
  if (rows == 0) return;
  HM_BF16(bf16, A, hipLaunchKernelGGL(retention_prep_kernel<A>, dim3(rows), dim3(NT), (size_t)rot_dims * sizeof(float), stream,
                                      (const A*)qkvg, row_stride, positions, freq, rot_dims, H, D, Dv, k_scale, out));
}

void launch_hm_act_mul(const void* x, bool bf16, int64_t x_stride, int rows, int F, bool silu, void* out, hipStream_t stream) {
  const int64_t n = (int64_t)rows * F;
  if (n == 0) return;
  const int blocks = (int)std::min<int64_t>((n + NT - 1) / NT, 16384);
  HM_BF16(bf16, A, hipLaunchKernelGGL(act_mul_kernel<A>, dim3(blocks), dim3(NT), 0, stream, (const A*)x, x_stride, F, n, silu ? 1 : 0,
                                      (A*)out));
}

void launch_hm_softmax_route(const void* h, bool bf16, int64_t h_stride, const float* router, const float* bias, int E, int K, int rows,
                             int W, int* ids, float* wts, hipStream_t stream) {
  if (rows == 0) return;
  HM_BF16(bf16, A, hipLaunchKernelGGL(softmax_route_kernel<A>, dim3(rows), dim3(NT), (size_t)W * sizeof(float), stream, (const A*)h,
                                      h_stride, router, bias, E, K, W, ids, wts));
}

}  // namespace dli
