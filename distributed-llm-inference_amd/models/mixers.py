"""Sequence mixers and the layer skeleton of heterogeneous decoder stacks.

Each mixer is a module with its sizes and constants as ``MixerSpec`` parameters, its own slice of the
runner's cache (token-major pages or per-sequence state rows, ``LayerCache``) and one ``forward(h, meta,
cache)`` that serves prefill chunks and decode rows of a mixed step alike:

* ``WindowAttention``   – grouped-query softmax attention, unit-RMS queries / keys, per-head temperature,
  logarithmic distance penalty, sliding window;
* ``LatentAttention``   – low-rank latent + shared rotated key cached per token; the key expansion is folded
  into the query and the value expansion applied after the softmax, so the cache is all the kernel reads;
* ``LightningAttention`` – linear attention with a per-head decay: a ``[D, Dv]`` fp32 state per head and sequence.

* ``SinkTalkAttention`` – causal grouped-query attention with whole-projection q / k norm, half-split partial
  rotation (optionally stretched frequencies), a per-head sink, weights mixed across heads, sigmoid output gate;
* ``TimeMix`` – recurrence with per-token, per-channel decay (low-rank projection), a bonus for the current token
  and a ``[D, D]`` fp32 state per head; its five projections read blends of the token's and the previous token's input;
* ``DualMixer`` – two of the above side by side on the same input, outputs summed with fixed weights.

``RoutedFF`` is a sigmoid-routed mixture of squared-ReLU experts with an optional gated shared expert;
``GatedParallelLayer`` runs a mixer and a feed-forward on two scalar-gain RMS norms of the same stream and adds
both, each through a sigmoid gate computed from its own input: ``x += m · (g1 ⊙ mixer(n1) + g2 ⊙ ff(n2))``.

* ``GatedAttention`` – causal grouped-query attention without positions: whole-projection q / k norm, one sigmoid output
  gate per head; optionally without key / value projections of its own, on another layer's cache;
* ``Retention`` – linear attention with a per-head decay and no activation: rotated q / k, scaled keys, a ``[D, Dv]``
  fp32 state per head, per-head unit RMS and a silu gate behind it.

* ``GatedLinearRecurrence`` – a per-channel recurrence ``S ← a ⊙ S + sqrt(1 - a²) ⊙ i ⊙ u`` behind a short causal convolution:
  decay and input gate from block-diagonal maps of ``u``, the fp32 state multiplied by a tanh-GELU branch;
* ``GatedLatentAttention`` – latent attention whose queries come from a normed latent too: half-split rotation with
  optionally stretched frequencies, a sliding window, a per-head sink in the softmax denominator, an element-wise sigmoid
  output gate; optionally without a key / value down-projection of its own, on another layer's cached latents.

``GatedDenseFF`` (``W_down (act(W_gate h) ⊙ W_up h)``, optionally with biases), ``SoftmaxRoutedFF`` (experts of that form
behind a biased fp32 router, softmax over the chosen logits) and ``ScoreRoutedFF`` (clamped gated experts and identity
experts chosen by softmax scores plus a correction) are the feed-forwards of ``HyperLayer``, which keeps several copies of
the fp32 stream: every sublayer reads a weighted sum of them through a norm (RMS with ``1 + w`` weights, or a layer norm
without bias; the mixer optionally also through a short causal convolution over time) and writes back through a mixing matrix.

``MixerLayer`` wraps one of the first three (and an optional dense feed-forward) in the sandwich
``x += m · norm_b(sublayer(norm(x)))`` with token shift in front of the mixer.  The residual stream ``x`` is
fp32; GEMM operands are the model dtype.  Tensor parallelism is not implemented for these stacks.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn as nn

from .. import ops
from ..config import KV_BLOCK_SIZE, MixerSpec
from ..ops import seqmix
from ..parallel.state import ParallelContext
from .layers import Weight


@dataclass
class LayerCache:
    """What one layer run keeps between steps: token-major pages (``k`` / ``v``; latent attention: ``k`` only), the
    recurrent ``state`` rows and the token-shift rows ``shift`` (previous token's normed input) — the latter two indexed
    by state slot."""
    k: Optional[torch.Tensor] = None
    v: Optional[torch.Tensor] = None
    state: Optional[torch.Tensor] = None
    shift: Optional[torch.Tensor] = None
    owns_pages: bool = True             # False: ``k`` / ``v`` are another layer's pages (a mixer without keys / values of its own)


def _param(shape, ctx, device) -> Weight:
    """Small fp32 parameter (norm weights / biases, per-head constants): these enter fp32 arithmetic only."""
    return Weight(tuple(shape), None, ctx, torch.float32, device)


def _matrix(out_f: int, in_f: int, ctx, dtype, device) -> Weight:
    return Weight((out_f, in_f), None, ctx, dtype, device)


class Norm(nn.Module):
    """Layer norm parameters (weight and bias over ``n`` features)."""

    def __init__(self, n: int, ctx, device):
        super().__init__()
        self.w, self.b = _param((n,), ctx, device), _param((n,), ctx, device)


class WindowAttention(nn.Module):
    def __init__(self, spec: MixerSpec, width: int, eps: float, ctx: ParallelContext, dtype, device):
        super().__init__()
        self.s, self.eps = spec, eps
        H, G, D, Dv = spec.heads, spec.kv_heads, spec.dim, spec.vdim
        assert H % G == 0, "query heads must be a multiple of the key/value heads"
        self.qkv = _matrix(H * D + G * D + G * Dv, width, ctx, dtype, device)
        self.o = _matrix(width, H * Dv, ctx, dtype, device)
        self.q_norm, self.k_norm = _param((D,), ctx, device), _param((D,), ctx, device)
        self.r1, self.r2, self.temp = (_param((H,), ctx, device) for _ in range(3))

    def weights(self, p):
        yield p + "qkv", self.qkv, "normal", [p + "q", p + "k", p + "v"]
        yield p + "o", self.o, "normal", None
        yield p + "q.norm", self.q_norm, "ones", None
        yield p + "k.norm", self.k_norm, "ones", None
        yield p + "r1", self.r1, "small", None
        yield p + "r2", self.r2, "small", None
        yield p + "temp", self.temp, "ones", None

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        s = self.s
        return LayerCache(k=torch.zeros(num_blocks, KV_BLOCK_SIZE, s.kv_heads * s.dim, dtype=dtype, device=device),
                          v=torch.zeros(num_blocks, KV_BLOCK_SIZE, s.kv_heads * s.vdim, dtype=dtype, device=device))

    def forward(self, h, meta, cache: LayerCache):
        s = self.s
        H, G, D, Dv = s.heads, s.kv_heads, s.dim, s.vdim
        T = h.shape[0]
        qkv = ops.linear(h, self.qkv.data)
        seqmix.qk_norm_cache(qkv, self.q_norm.data, self.k_norm.data, self.eps, meta.slot_mapping, cache.k, cache.v, H, G, D, Dv)
        out = torch.empty(T, H, Dv, dtype=h.dtype, device=h.device)
        seqmix.token_attention(out, qkv[:, :H * D].view(T, H, D), None, cache.k, cache.v, meta, G, Dv, s.scale, s.window,
                               self.temp.data, self.r1.data, self.r2.data)
        return ops.linear(out.view(T, H * Dv), self.o.data)


class LatentAttention(nn.Module):
    def __init__(self, spec: MixerSpec, width: int, eps: float, ctx: ParallelContext, dtype, device):
        super().__init__()
        self.s, self.eps = spec, eps
        H, D, R, Dv, C = spec.heads, spec.dim, spec.rot_dim, spec.vdim, spec.kv_rank
        assert spec.rot_dims <= R and spec.rot_dims % 2 == 0
        self.q_dkv = _matrix(H * (D + R) + C + R, width, ctx, dtype, device)
        self.c_norm = _param((C,), ctx, device)
        self.uk = _matrix(H * D, C, ctx, dtype, device)
        self.uv = _matrix(H * Dv, C, ctx, dtype, device)
        self.o = _matrix(width, H * Dv, ctx, dtype, device)
        self.register_buffer("inv_freq", seqmix.rotary_inv_freq(spec.rot_base, spec.rot_dims, device), persistent=False)

    def weights(self, p):
        yield p + "q_dkv", self.q_dkv, "normal", [p + "q", p + "dkv"]
        yield p + "dkv.norm", self.c_norm, "ones", None
        yield p + "uk", self.uk, "normal", None
        yield p + "uv", self.uv, "normal", None
        yield p + "o", self.o, "normal", None

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        s = self.s
        return LayerCache(k=torch.zeros(num_blocks, KV_BLOCK_SIZE, s.kv_rank + s.rot_dim, dtype=dtype, device=device))

    def forward(self, h, meta, cache: LayerCache):
        s = self.s
        H, D, R, Dv, C = s.heads, s.dim, s.rot_dim, s.vdim, s.kv_rank
        T = h.shape[0]
        both = ops.linear(h, self.q_dkv.data)
        q, dkv = both[:, :H * (D + R)], both[:, H * (D + R):]
        seqmix.latent_prep(q, dkv, self.c_norm.data, self.eps, meta.positions, self.inv_freq, s.rot_dims, meta.slot_mapping,
                           cache.k, H, D, R, C)
        q3 = q.view(T, H, D + R) if q.is_contiguous() else q.unflatten(1, (H, D + R))
        # key expansion folded into the query: (W_uk c) · q = c · (W_ukᵀ q) — one [D] → [C] product per head and token
        q_lat = torch.bmm(q3[:, :, :D].transpose(0, 1), self.uk.data.view(H, D, C))                  # [H, T, C]
        o_lat = torch.empty(H, T, C, dtype=h.dtype, device=h.device)
        seqmix.token_attention(o_lat.transpose(0, 1), q_lat.transpose(0, 1), q3[:, :, D:], cache.k, None, meta, 1, C, s.scale)
        # value expansion after the softmax: Σ p_j (W_uv c_j) = W_uv (Σ p_j c_j)
        out = torch.bmm(o_lat, self.uv.data.view(H, Dv, C).transpose(1, 2))                          # [H, T, Dv]
        return ops.linear(out.transpose(0, 1).reshape(T, H * Dv), self.o.data)


class LightningAttention(nn.Module):
    def __init__(self, spec: MixerSpec, width: int, eps: float, ctx: ParallelContext, dtype, device):
        super().__init__()
        self.s, self.eps = spec, eps
        H, D, Dv = spec.heads, spec.dim, spec.vdim
        assert len(spec.decay) == H, "one decay per head"
        self.qkvg = _matrix(2 * H * D + 2 * H * Dv, width, ctx, dtype, device)
        self.norm = _param((H * Dv,), ctx, device)
        self.o = _matrix(width, H * Dv, ctx, dtype, device)
        self.register_buffer("decay", torch.tensor(spec.decay, dtype=torch.float32, device=device), persistent=False)

    def weights(self, p):
        yield p + "qkvg", self.qkvg, "normal", [p + "q", p + "k", p + "v", p + "g"]
        yield p + "norm", self.norm, "ones", None
        yield p + "o", self.o, "normal", None

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        s = self.s
        return LayerCache(state=torch.zeros(num_slots, s.heads, s.dim, s.vdim, dtype=torch.float32, device=device))

    def forward(self, h, meta, cache: LayerCache):
        s = self.s
        H, D, Dv = s.heads, s.dim, s.vdim
        qkvg = ops.linear(h, self.qkvg.data)
        o = seqmix.lightning_scan(qkvg, cache.state, meta, H, D, Dv, self.decay)
        y = seqmix.rms_gate(o, self.norm.data, self.eps, qkvg[:, 2 * H * D + H * Dv:], h.dtype)
        return ops.linear(y, self.o.data)


class SinkTalkAttention(nn.Module):
    """``extra`` output columns are appended to the fused input projection (the layer's residual gate reads the same
    input): ``forward`` returns ``(attention output [T, H·Dv] before the output projection's caller-side scaling, extra)``."""

    def __init__(self, spec: MixerSpec, width: int, eps: float, ctx: ParallelContext, dtype, device, extra: int = 0):
        super().__init__()
        self.s, self.eps, self.extra = spec, eps, extra
        H, G, D, Dv = spec.heads, spec.kv_heads, spec.dim, spec.vdim
        assert H % G == 0, "query heads must be a multiple of the key/value heads"
        assert spec.rot_dims % 2 == 0 and spec.rot_dims <= D
        self.cols = (H * D, G * D, G * Dv, H * Dv, extra)           # q | k | v | output gate | extra
        self.qkvg = _matrix(sum(self.cols), width, ctx, dtype, device)
        self.o = _matrix(width, H * Dv, ctx, dtype, device)
        self.q_norm, self.k_norm = _param((H * D,), ctx, device), _param((G * D,), ctx, device)
        self.sink, self.talk = _param((H,), ctx, device), _param((H, H), ctx, device)
        freq, self.mag = seqmix.stretched_inv_freq(spec.rot_base, spec.rot_dims, spec.rot_scaling, device)
        self.register_buffer("inv_freq", freq, persistent=False)
        if torch.device(device).type == "cuda":
            seqmix._hip().dm_prepare()                      # kernel attributes are set outside any later stream capture

    def weights(self, p, extra_src=()):
        yield p + "qkvg", self.qkvg, "normal", [p + "q", p + "k", p + "v", p + "g", *extra_src]
        yield p + "o", self.o, "normal", None
        yield p + "q.norm", self.q_norm, "ones", None
        yield p + "k.norm", self.k_norm, "ones", None
        yield p + "sink", self.sink, "zeros", None
        yield p + "talk", self.talk, "eye", None

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        s = self.s
        return LayerCache(k=torch.zeros(num_blocks, KV_BLOCK_SIZE, s.kv_heads * s.dim, dtype=dtype, device=device),
                          v=torch.zeros(num_blocks, KV_BLOCK_SIZE, s.kv_heads * s.vdim, dtype=dtype, device=device))

    def forward(self, h, meta, cache: LayerCache):
        s = self.s
        H, G, D, Dv = s.heads, s.kv_heads, s.dim, s.vdim
        T = h.shape[0]
        nq, nk, nv, ng, _ = self.cols
        both = ops.linear(h, self.qkvg.data)
        seqmix.wide_norm_rope_cache(both, self.q_norm.data, self.k_norm.data, self.eps, meta.positions, self.inv_freq, self.mag,
                                    s.rot_dims, meta.slot_mapping, cache.k, cache.v, H, G, D, Dv)
        out = torch.zeros(T, H * Dv, dtype=h.dtype, device=h.device)     # padding rows of a captured step stay zero
        g0 = nq + nk + nv
        seqmix.talk_attention(out, both[:, :nq].unflatten(1, (H, D)), both[:, g0:g0 + ng], cache.k, cache.v, meta, G, Dv, s.scale,
                              self.sink.data, self.talk.data)
        return ops.linear(out, self.o.data), both[:, g0 + ng:]


class TimeMix(nn.Module):
    BLENDS = "rkvgw"                                     # order of the blend rows: receptance, key, value, gate, decay

    def __init__(self, spec: MixerSpec, width: int, eps: float, ctx: ParallelContext, dtype, device):
        super().__init__()
        self.s, self.eps = spec, eps
        H, D = spec.heads, spec.dim
        C = H * D
        assert spec.lora > 0, "the decay projection needs a rank"
        self.mu = _param((5, width), ctx, device)
        self.rkvg = Weight((4, C, width), None, ctx, dtype, device)         # one batched product for the four wide projections
        self.w1, self.w2 = _matrix(spec.lora, width, ctx, dtype, device), _matrix(C, spec.lora, ctx, dtype, device)
        self.w0, self.u, self.norm = _param((C,), ctx, device), _param((C,), ctx, device), _param((C,), ctx, device)
        self.o = _matrix(width, C, ctx, dtype, device)

    def weights(self, p):
        yield p + "mu", self.mu, "half", [[p + "mu." + s] for s in self.BLENDS]
        yield p + "rkvg", self.rkvg, "normal", [[p + s] for s in "rkvg"]
        yield p + "w1", self.w1, "normal", None
        yield p + "w2", self.w2, "normal", None
        yield p + "w0", self.w0, "zeros", None
        yield p + "u", self.u, "half", None
        yield p + "norm", self.norm, "ones", None
        yield p + "o", self.o, "normal", None

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        s = self.s
        return LayerCache(state=torch.zeros(num_slots, s.heads, s.dim, s.dim, dtype=torch.float32, device=device),
                          shift=torch.zeros(num_slots, self.mu.data.shape[1], dtype=torch.float32, device=device))

    def forward(self, h, meta, cache: LayerCache):
        s = self.s
        blends = seqmix.shift_mix(h, self.mu.data, cache.shift, meta)                    # [5, T, W]
        rkvg = torch.bmm(blends[:4], self.rkvg.data.transpose(1, 2))                     # [4, T, C]
        w = seqmix.decay_lora(ops.linear(blends[4], self.w1.data), self.w2.data, self.w0.data)
        o = seqmix.wkv_scan(rkvg, w, self.u.data, cache.state, meta, s.heads, s.dim)
        y = seqmix.group_rms_gate(o, s.heads, self.norm.data, self.eps, rkvg[3], h.dtype)
        return ops.linear(y, self.o.data)


class DualMixer(nn.Module):
    """Sink attention and a time mix on the same input; ``forward`` returns both outputs (the layer's combine step applies
    ``part_scales`` in fp32) and the extra columns of the attention's input projection."""

    def __init__(self, spec: MixerSpec, width: int, eps: float, ctx: ParallelContext, dtype, device, extra: int = 0):
        super().__init__()
        kinds = tuple(p.kind for p in spec.parts)
        if kinds != ("sink_attention", "time_mix"):
            raise ValueError(f"parallel mixers are sink attention beside a time mix, not {kinds}")
        self.s = spec
        self.left = SinkTalkAttention(spec.parts[0], width, eps, ctx, dtype, device, extra)
        self.right = TimeMix(spec.parts[1], width, eps, ctx, dtype, device)

    def weights(self, p, extra_src=()):
        yield from self.left.weights(p + "left.", extra_src)
        yield from self.right.weights(p + "right.")

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        a, b = self.left.cache(num_blocks, num_slots, dtype, device), self.right.cache(num_blocks, num_slots, dtype, device)
        return LayerCache(k=a.k, v=a.v, state=b.state, shift=b.shift)

    def forward(self, h, meta, cache: LayerCache):
        left, extra = self.left(h, meta, cache)
        return [left, self.right(h, meta, cache)], extra


class GatedAttention(nn.Module):
    """``spec.kv_from`` ≥ 0: no key / value projections; ``forward`` reads the pages it is handed (that layer's)."""

    def __init__(self, spec: MixerSpec, width: int, eps: float, ctx: ParallelContext, dtype, device):
        super().__init__()
        self.s, self.eps = spec, eps
        H, G, D, Dv = spec.heads, spec.kv_heads, spec.dim, spec.vdim
        assert H % G == 0, "query heads must be a multiple of the key/value heads"
        self.own_kv = spec.kv_from < 0
        Gp = G if self.own_kv else 0
        used = H * D + Gp * D + Gp * Dv + H
        # q | k | v | one output gate per head | unused rows: the tile kernels read query rows at 16-byte strides
        self.cols = (H * D, Gp * D, Gp * Dv, H, -used % 8)
        self.qkvg = _matrix(sum(self.cols), width, ctx, dtype, device)
        self.o = _matrix(width, H * Dv, ctx, dtype, device)
        self.q_norm = _param((H * D,), ctx, device)
        self.k_norm = _param((G * D,), ctx, device) if self.own_kv else None

    def weights(self, p):
        pad = [f"@zeros:{self.cols[4]}"] if self.cols[4] else []
        yield p + "qkvg", self.qkvg, "normal", [p + "q"] + ([p + "k", p + "v"] if self.own_kv else []) + [p + "g"] + pad
        yield p + "o", self.o, "normal", None
        yield p + "q.norm", self.q_norm, "ones", None
        if self.own_kv:
            yield p + "k.norm", self.k_norm, "ones", None

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        s = self.s
        if not self.own_kv:
            return LayerCache(owns_pages=False)
        return LayerCache(k=torch.zeros(num_blocks, KV_BLOCK_SIZE, s.kv_heads * s.dim, dtype=dtype, device=device),
                          v=torch.zeros(num_blocks, KV_BLOCK_SIZE, s.kv_heads * s.vdim, dtype=dtype, device=device))

    def forward(self, h, meta, cache: LayerCache):
        s = self.s
        H, G, D, Dv = s.heads, s.kv_heads, s.dim, s.vdim
        T = h.shape[0]
        nq, nk, nv, ng, _pad = self.cols
        both = ops.linear(h, self.qkvg.data)
        seqmix.wide_norm_rope_cache(both, self.q_norm.data, self.k_norm.data if self.own_kv else None, self.eps, meta.positions,
                                    None, 1.0, 0, meta.slot_mapping, cache.k, cache.v, H, G if self.own_kv else 0, D, Dv)
        out = torch.zeros(T, H, Dv, dtype=h.dtype, device=h.device)      # padding rows of a captured step stay zero
        seqmix.token_attention(out, both[:, :nq].unflatten(1, (H, D)), None, cache.k, cache.v, meta, G, Dv, s.scale,
                               gate=both[:, nq + nk + nv:nq + nk + nv + ng])
        return ops.linear(out.view(T, H * Dv), self.o.data)


class Retention(nn.Module):
    def __init__(self, spec: MixerSpec, width: int, eps: float, ctx: ParallelContext, dtype, device):
        super().__init__()
        self.s, self.eps = spec, eps
        H, D, Dv = spec.heads, spec.dim, spec.vdim
        assert len(spec.decay) == H, "one decay per head"
        assert spec.rot_dims % 2 == 0 and spec.rot_dims <= D
        self.qkvg = _matrix(2 * H * D + 2 * H * Dv, width, ctx, dtype, device)
        self.o = _matrix(width, H * Dv, ctx, dtype, device)
        self.register_buffer("decay", torch.tensor(spec.decay, dtype=torch.float32, device=device), persistent=False)
        self.register_buffer("inv_freq", seqmix.rotary_inv_freq(spec.rot_base, spec.rot_dims, device) if spec.rot_dims else None,
                             persistent=False)

    def weights(self, p):
        yield p + "qkvg", self.qkvg, "normal", [p + "q", p + "k", p + "v", p + "g"]
        yield p + "o", self.o, "normal", None

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        s = self.s
        return LayerCache(state=torch.zeros(num_slots, s.heads, s.dim, s.vdim, dtype=torch.float32, device=device))

    def forward(self, h, meta, cache: LayerCache):
        s = self.s
        H, D, Dv = s.heads, s.dim, s.vdim
        qkvg = ops.linear(h, self.qkvg.data)
        # rotation, key scale and everything behind them in fp32, whatever the model dtype
        qkv = seqmix.retention_prep(qkvg, meta.positions, self.inv_freq, s.rot_dims, H, D, Dv, D ** -0.5)
        o = seqmix.lightning_scan(qkv, cache.state, meta, H, D, Dv, self.decay, activation="none")
        y = seqmix.rms_gate(o, None, self.eps, qkvg[:, 2 * H * D + H * Dv:], h.dtype, groups=H, gate_act="silu")
        return ops.linear(y, self.o.data)


class GatedLinearRecurrence(nn.Module):
    """``W_o (S ⊙ gelu_tanh(W_y h + b_y))`` with ``S`` the per-channel fp32 state of ``S ← a ⊙ S + sqrt(1 - a²) ⊙ i ⊙ u``:
    ``u`` = causal convolution (``conv_taps`` taps, bias) of ``W_x h + b_x``; recurrence gate ``r`` and input gate ``i`` are
    sigmoids of block-diagonal maps of ``u`` (``heads`` blocks of ``dim`` channels, biases); ``a = exp(-8 · r · softplus(λ))``."""

    def __init__(self, spec: MixerSpec, width: int, eps: float, ctx: ParallelContext, dtype, device):
        super().__init__()
        self.s, self.dtype = spec, dtype
        B, n, taps = spec.heads, spec.dim, spec.conv_taps
        C = B * n
        assert taps >= 1, "the convolution has at least the current token's tap"
        self.yx, self.yx_b = _matrix(2 * C, width, ctx, dtype, device), Weight((2 * C,), None, ctx, dtype, device)
        self.conv, self.conv_b = _param((C, taps), ctx, device), _param((C,), ctx, device)
        self.gates = Weight((2 * B, n, n), None, ctx, dtype, device)        # the blocks of the recurrence gate, then those of the input gate
        self.gates_b = _param((2, C), ctx, device)
        self.lam = _param((C,), ctx, device)
        self.o = _matrix(width, C, ctx, dtype, device)
        self._taps = self._rate = self._gates_t = None                     # derived at first use (after loading)

    def weights(self, p):
        B = self.s.heads
        yield p + "yx", self.yx, "normal", [p + "y", p + "x"]
        yield p + "yx.b", self.yx_b, "zeros", [p + "y.b", p + "x.b"]
        yield p + "conv", self.conv, "small", None
        yield p + "conv.b", self.conv_b, "zeros", None
        yield p + "gates", self.gates, "normal", [p + "ra", p + "ri"]
        yield p + "gates.b", self.gates_b, "zeros", [p + "ra.b", p + "ri.b"]
        yield p + "lam", self.lam, "small", None
        yield p + "o", self.o, "normal", None

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        B, n, taps = self.s.heads, self.s.dim, self.s.conv_taps
        return LayerCache(state=torch.zeros(num_slots, B * n, dtype=torch.float32, device=device),
                          shift=torch.zeros(num_slots, max(taps - 1, 0), B * n, dtype=torch.float32, device=device))

    def forward(self, h, meta, cache: LayerCache):
        B, n = self.s.heads, self.s.dim
        C = B * n
        T = h.shape[0]
        if self._taps is None:
            self._taps = self.conv.data.t().contiguous()
            self._rate = 8.0 * torch.nn.functional.softplus(self.lam.data)
            # checkpoint order is [ra blocks | ri blocks]; the product wants a block's two gates side by side: [B, n, 2n]
            g = self.gates.data.view(2, B, n, n)
            self._gates_t = torch.cat([g[0].transpose(1, 2), g[1].transpose(1, 2)], dim=2).contiguous()
        yx = ops.linear(h, self.yx.data, self.yx_b.data)
        u = seqmix.causal_conv(yx[:, C:], self._taps, self.conv_b.data, cache.shift, meta, self.dtype)
        z = torch.bmm(u.view(T, B, n).transpose(0, 1), self._gates_t)                      # [B, T, 2n]
        out = seqmix.rglru_scan(z, u, yx[:, :C], self.gates_b.data, self._rate, cache.state, meta, self.dtype)
        return ops.linear(out, self.o.data)


class GatedLatentAttention(nn.Module):
    """Latent attention behind a normed query latent: ``c_q = rms(W_dq h)``, ``q = W_uq c_q``; keys and values are expanded from
    the cached latent ``c = rms(W_dkv h)[:C]`` and one rotated key part shared by the heads (the key expansion folded into
    the query, the value expansion applied after the softmax, so the cache rows are all the attention kernel reads).
    Half-split rotation with optionally stretched frequencies, sliding window, a per-head sink in the softmax denominator,
    element-wise sigmoid output gate ``W_g h``.  ``spec.kv_from`` ≥ 0: no ``W_dkv``; the layer reads that layer's cache rows."""

    def __init__(self, spec: MixerSpec, width: int, eps: float, ctx: ParallelContext, dtype, device):
        super().__init__()
        self.s, self.eps = spec, eps
        H, D, R, Dv, C, Q = spec.heads, spec.dim, spec.rot_dim, spec.vdim, spec.kv_rank, spec.q_rank
        assert spec.rot_dims <= R and spec.rot_dims % 2 == 0
        self.own_kv = spec.kv_from < 0
        kv = C + R if self.own_kv else 0
        used = Q + kv + H * Dv
        self.cols = (Q, kv, H * Dv, -used % 8)                  # query latent | latent + key part | output gate | alignment rows
        self.down = _matrix(sum(self.cols), width, ctx, dtype, device)
        self.q_norm = _param((Q,), ctx, device)
        self.c_norm = _param((C,), ctx, device) if self.own_kv else None
        self.uq = _matrix(H * (D + R), Q, ctx, dtype, device)
        self.uk = _matrix(H * D, C, ctx, dtype, device)
        self.uv = _matrix(H * Dv, C, ctx, dtype, device)
        self.sink = _param((H,), ctx, device) if spec.sink else None
        self.o = _matrix(width, H * Dv, ctx, dtype, device)
        freq, self.mag = seqmix.stretched_inv_freq(spec.rot_base, spec.rot_dims, spec.rot_scaling, device)
        self.register_buffer("inv_freq", freq, persistent=False)

    def weights(self, p):
        pad = [f"@zeros:{self.cols[3]}"] if self.cols[3] else []
        yield p + "down", self.down, "normal", [p + "dq"] + ([p + "dkv"] if self.own_kv else []) + [p + "g"] + pad
        yield p + "dq.norm", self.q_norm, "ones", None
        if self.own_kv:
            yield p + "dkv.norm", self.c_norm, "ones", None
        yield p + "uq", self.uq, "normal", None
        yield p + "uk", self.uk, "normal", None
        yield p + "uv", self.uv, "normal", None
        if self.sink is not None:
            yield p + "sink", self.sink, "zeros", None
        yield p + "o", self.o, "normal", None

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        s = self.s
        if not self.own_kv:
            return LayerCache(owns_pages=False)
        return LayerCache(k=torch.zeros(num_blocks, KV_BLOCK_SIZE, s.kv_rank + s.rot_dim, dtype=dtype, device=device))

    def forward(self, h, meta, cache: LayerCache):
        s = self.s
        H, D, R, Dv, C, Q = s.heads, s.dim, s.rot_dim, s.vdim, s.kv_rank, s.q_rank
        T = h.shape[0]
        nq, nkv, ng, _pad = self.cols
        both = ops.linear(h, self.down.data)
        cq = seqmix.latent_norm_cache(both, Q, self.q_norm.data, self.c_norm.data if self.own_kv else None, self.eps, meta.positions,
                                      self.inv_freq, self.mag, s.rot_dims, meta.slot_mapping, cache.k if self.own_kv else None, C, R)
        q = ops.linear(cq, self.uq.data)
        seqmix.rotate_heads(q, meta.positions, self.inv_freq, self.mag, s.rot_dims, H, D, R)
        q3 = q.view(T, H, D + R)
        # key expansion folded into the query: (W_uk c) · q = c · (W_ukᵀ q) — one [D] → [C] product per head and token
        q_lat = torch.bmm(q3[:, :, :D].transpose(0, 1), self.uk.data.view(H, D, C))                  # [H, T, C]
        o_lat = torch.zeros(H, T, C, dtype=h.dtype, device=h.device)     # padding rows of a captured step stay zero
        seqmix.token_attention(o_lat.transpose(0, 1), q_lat.transpose(0, 1), q3[:, :, D:], cache.k, None, meta, 1, C, s.scale,
                               s.window, sink=self.sink.data if self.sink is not None else None)
        # value expansion after the softmax: Σ p_j (W_uv c_j) = W_uv (Σ p_j c_j)
        out = torch.bmm(o_lat, self.uv.data.view(H, Dv, C).transpose(1, 2))                          # [H, T, Dv]
        return ops.linear(seqmix.gate_heads(out, both[:, nq + nkv:nq + nkv + ng]), self.o.data)


MIXERS = {"gated_attention": GatedAttention, "retention": Retention, "attention": WindowAttention, "latent_attention": LatentAttention, "lightning": LightningAttention,
          "sink_attention": SinkTalkAttention, "time_mix": TimeMix, "parallel": DualMixer, "rglru": GatedLinearRecurrence,
          "gated_latent_attention": GatedLatentAttention}


class DenseFF(nn.Module):
    """``W_down · relu(W_up h)²``."""

    def __init__(self, width: int, ff: int, ctx, dtype, device):
        super().__init__()
        self.up, self.down = _matrix(ff, width, ctx, dtype, device), _matrix(width, ff, ctx, dtype, device)

    def forward(self, h):
        return ops.linear(seqmix.relu2(ops.linear(h, self.up.data)), self.down.data)


class RoutedFF(nn.Module):
    """``Σ_chosen score · scale · expert(h)  +  sigmoid(w_sg · h) · shared(h)`` with ``expert(h) = W_down · relu(W_up h)²``;
    scores are sigmoids of fp32 router logits, the ``top`` largest are chosen and not renormalised.  ``extra`` output
    columns are appended to the shared expert's up projection (the layer's residual gate reads the same input)."""

    def __init__(self, spec: MixerSpec, width: int, ctx, dtype, device, extra: int = 0):
        super().__init__()
        self.s, self.extra = spec, extra
        E, F, Fs = spec.experts, spec.ff, spec.shared_ff
        assert 1 <= spec.top <= E
        self.up, self.down = Weight((E, F, width), None, ctx, dtype, device), Weight((E, width, F), None, ctx, dtype, device)
        self.router = _param((E + (1 if Fs else 0), width), ctx, device)     # fp32; last row: the shared expert's gate
        self.shared_up = _matrix(Fs + extra, width, ctx, dtype, device) if Fs + extra else None
        self.shared_down = _matrix(width, Fs, ctx, dtype, device) if Fs else None

    def weights(self, p, extra_src=()):
        E, Fs = self.s.experts, self.s.shared_ff
        yield p + "experts.up", self.up, "normal", [[p + f"e{e}.up"] for e in range(E)]
        yield p + "experts.down", self.down, "normal", [[p + f"e{e}.down"] for e in range(E)]
        yield p + "router", self.router, "normal", [p + "router"] + ([p + "shared.sg"] if Fs else [])
        if self.shared_up is not None:
            yield p + "shared.up", self.shared_up, "normal", ([p + "shared.up"] if Fs else []) + list(extra_src)
        if Fs:
            yield p + "shared.down", self.shared_down, "normal", None

    def forward(self, h):
        """Returns ``(routed sum [T, W], shared expert's output or None, its gate fp32 [T] or None, extra columns)``."""
        s = self.s
        ids, wts, sgate = seqmix.sigmoid_route(h, self.router.data, s.experts, s.top, s.router_scale)
        routed = seqmix.relu2_experts(h, ids, wts, self.up.data, self.down.data)
        shared = extra = None
        if self.shared_up is not None:
            both = ops.linear(h, self.shared_up.data)
            extra = both[:, s.shared_ff:]
            if s.shared_ff:
                shared = ops.linear(seqmix.relu2_rows(both[:, :s.shared_ff]), self.shared_down.data)
        return routed, shared, sgate, extra


class GatedDenseFF(nn.Module):
    """``W_down · (act(W_gate h) ⊙ W_up h)``; gate and up rows are one GEMM."""

    def __init__(self, width: int, ff: int, act: str, ctx, dtype, device, bias: bool = False):
        super().__init__()
        self.act = act
        self.gate_up, self.down = _matrix(2 * ff, width, ctx, dtype, device), _matrix(width, ff, ctx, dtype, device)
        self.gate_up_b = Weight((2 * ff,), None, ctx, dtype, device) if bias else None
        self.down_b = Weight((width,), None, ctx, dtype, device) if bias else None

    def weights(self, p):
        yield p + "gate_up", self.gate_up, "normal", [p + "gate", p + "up"]
        yield p + "down", self.down, "normal", None
        if self.gate_up_b is not None:
            yield p + "gate_up.b", self.gate_up_b, "zeros", [p + "gate.b", p + "up.b"]
            yield p + "down.b", self.down_b, "zeros", None

    def forward(self, h):
        if self.gate_up_b is None:
            return ops.linear(seqmix.act_mul(ops.linear(h, self.gate_up.data), self.act), self.down.data)
        return ops.linear(seqmix.act_mul(ops.linear(h, self.gate_up.data, self.gate_up_b.data), self.act), self.down.data, self.down_b.data)


class SoftmaxRoutedFF(nn.Module):
    """``Σ_chosen p_e · expert_e(h)``, ``expert(h) = W_down · (silu(W_gate h) ⊙ W_up h)``: the ``top`` experts with the largest
    fp32 router logits ``W_r h + b`` are chosen, ``p`` is the softmax over the chosen logits."""

    def __init__(self, spec: MixerSpec, width: int, ctx, dtype, device):
        super().__init__()
        self.s = spec
        E, F = spec.experts, spec.ff
        assert 1 <= spec.top <= E
        if spec.ff_act != "silu":
            raise ValueError(f"routed gated experts use silu, not {spec.ff_act!r}")
        self.gate_up, self.down = Weight((E, 2 * F, width), None, ctx, dtype, device), Weight((E, width, F), None, ctx, dtype, device)
        self.router, self.bias = _param((E, width), ctx, device), _param((E,), ctx, device)

    def weights(self, p):
        E = self.s.experts
        yield p + "experts.gate_up", self.gate_up, "normal", [[p + f"e{e}.gate", p + f"e{e}.up"] for e in range(E)]
        yield p + "experts.down", self.down, "normal", [[p + f"e{e}.down"] for e in range(E)]
        yield p + "router", self.router, "normal", None
        yield p + "router.b", self.bias, "zeros", None

    def forward(self, h):
        ids, wts = seqmix.softmax_route(h, self.router.data, self.bias.data, self.s.top)
        return seqmix.gated_experts(h, ids, wts, self.gate_up.data, self.down.data)


class ScoreRoutedFF(nn.Module):
    """``Σ_chosen w_e · expert_e(h)``: scores are the fp32 softmax of ``W_r h`` over all router outputs; the ``top`` outputs with
    the largest ``score + correction`` are chosen and weigh ``score / Σ_chosen score``.  The last ``identity_experts`` outputs
    are experts without tensors that return ``h`` itself; the others are clamped gated experts
    ``W_down (g · sigmoid(1.702 g) · (u + 1))`` with ``g = min(W_gate h, limit)``, ``u = clamp(W_up h, ±limit)``."""

    def __init__(self, spec: MixerSpec, width: int, ctx, dtype, device):
        super().__init__()
        self.s = spec
        E, F, I = spec.experts, spec.ff, spec.identity_experts
        assert 1 <= spec.top <= E + I and spec.ff_limit > 0.0
        self.gate_up, self.down = Weight((E, 2 * F, width), None, ctx, dtype, device), Weight((E, width, F), None, ctx, dtype, device)
        self.router, self.correction = _param((E + I, width), ctx, device), _param((E + I,), ctx, device)

    def weights(self, p):
        E = self.s.experts
        yield p + "experts.gate_up", self.gate_up, "normal", [[p + f"e{e}.gate", p + f"e{e}.up"] for e in range(E)]
        yield p + "experts.down", self.down, "normal", [[p + f"e{e}.down"] for e in range(E)]
        yield p + "router", self.router, "normal", None
        yield p + "correction", self.correction, "zeros", None

    def forward(self, h):
        ids, wts = seqmix.softmax_all_route(h, self.router.data, self.correction.data, self.s.top)
        return seqmix.gated_experts(h, ids, wts, self.gate_up.data, self.down.data, limit=self.s.ff_limit)


class StreamLinks(nn.Module):
    """How one sublayer reads and writes ``S`` copies of the stream: ``u = Σ_s in[s] x_s`` goes in; the result ``y`` comes back
    as ``x_t ← Σ_s mix[s, t] x_s + out[t] y``.  ``S = 1`` with all-ones weights is the plain residual sum."""

    def __init__(self, streams: int, ctx, device):
        super().__init__()
        self.w_in, self.w_out, self.mix = _param((streams,), ctx, device), _param((streams,), ctx, device), _param((streams, streams), ctx, device)
        with torch.no_grad():           # the plain residual sum until a checkpoint or the random initialisation says otherwise
            self.w_in.init_const(1.0)
            self.w_out.init_const(1.0)
            self.mix.load_full(torch.eye(streams, dtype=torch.float32, device=device))

    def weights(self, p):
        yield p + "in", self.w_in, "ones", None
        yield p + "out", self.w_out, "ones", None
        yield p + "mix", self.mix, "eye", None


class HyperLayer(nn.Module):
    """Pre-norm layer over ``S`` fp32 streams ``x [T, S, W]``: ``y = mixer(conv(norm1(Σ in·x)))`` written back through the first
    links, then ``y = ff(norm2(Σ in·x))`` through the second.  Norm weights are stored around zero (``1 + w``); ``conv`` adds a
    causal per-channel convolution over the sequence's last ``taps`` inputs (``taps`` = 0: none).  ``links`` False: one stream,
    plain residual sums (the link weights stay at one and are not part of a checkpoint)."""

    def __init__(self, spec: MixerSpec, width: int, eps: float, streams: int, taps: int, ctx: ParallelContext, dtype, device,
                 norm: str = "rms_offset"):
        super().__init__()
        if norm not in ("rms_offset", "layer"):
            raise ValueError(f"unknown norm {norm!r}")
        self.spec, self.eps, self.dtype, self.taps = spec, eps, dtype, taps
        # "rms_offset": u / rms(u) · (1 + w); "layer": (u - mean) / sqrt(var + eps) · w
        self.center, self.w_offset = norm == "layer", 0.0 if norm == "layer" else 1.0
        self.links = streams > 0
        S = max(streams, 1)
        self.norm1, self.hc1 = _param((width,), ctx, device), StreamLinks(S, ctx, device)
        self.conv = _param((width, taps), ctx, device) if taps else None    # as checkpoints store it: a channel's taps together
        self._conv_taps = None                                               # tap-major copy for the kernel, made at first use
        self.mixer = MIXERS[spec.kind](spec, width, eps, ctx, dtype, device)
        self.ff = None
        if spec.ff:
            self.norm2, self.hc2 = _param((width,), ctx, device), StreamLinks(S, ctx, device)
            if spec.ff_kind == "moe":
                if spec.router == "softmax":
                    self.ff = SoftmaxRoutedFF(spec, width, ctx, dtype, device)
                elif spec.router == "softmax_all":
                    self.ff = ScoreRoutedFF(spec, width, ctx, dtype, device)
                else:
                    raise ValueError(f"hyper-connected layers route by softmax, not {spec.router!r}")
            else:
                self.ff = GatedDenseFF(width, spec.ff, spec.ff_act, ctx, dtype, device, bias=spec.ff_bias)

    def weights(self, p):
        yield p + "norm1", self.norm1, "ones" if self.center else "zeros", None
        if self.links:
            yield from self.hc1.weights(p + "hc1.")
        if self.conv is not None:
            yield p + "canon1", self.conv, "small", None
        yield from self.mixer.weights(p + "mix.")
        if self.ff is not None:
            yield p + "norm2", self.norm2, "ones" if self.center else "zeros", None
            if self.links:
                yield from self.hc2.weights(p + "hc2.")
            yield from self.ff.weights(p + "mlp.")

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        c = self.mixer.cache(num_blocks, num_slots, dtype, device)
        if self.taps:               # the sequence's last taps-1 mixer inputs, oldest first
            assert c.shift is None, "the layer's input convolution and the mixer both want the shift rows"
            c.shift = torch.zeros(num_slots, self.taps - 1, self.norm1.data.shape[0], dtype=torch.float32, device=device)
        return c

    def read(self, x, y, prev: Optional[StreamLinks], out_dtype):
        """Write the previous sublayer's ``y`` back through its links ``prev`` (if any) and return this layer's mixer input
        before the convolution."""
        return seqmix.stream_mix_norm(x, y, prev.mix.data if prev else None, prev.w_out.data if prev else None, self.hc1.w_in.data,
                                      self.norm1.data, self.eps, self.w_offset, out_dtype, self.center)

    def forward(self, x, h, meta, cache: LayerCache):
        """``x``: fp32 streams ``[T, S, W]``, updated in place; ``h``: this layer's normed mixer input (``read``).  Returns the
        last sublayer's output and its links — the caller's next ``read`` (or the closing norm) writes them back."""
        if self.conv is not None:
            if self._conv_taps is None:
                self._conv_taps = self.conv.data.t().contiguous()
            h = seqmix.causal_conv_add(h, self._conv_taps, cache.shift, meta, self.dtype)
        y = self.mixer(h, meta, cache)
        if self.ff is None:
            return y, self.hc1
        h2 = seqmix.stream_mix_norm(x, y, self.hc1.mix.data, self.hc1.w_out.data, self.hc2.w_in.data, self.norm2.data, self.eps,
                                    self.w_offset, self.dtype, self.center)
        return self.ff(h2), self.hc2


class GatedParallelLayer(nn.Module):
    def __init__(self, spec: MixerSpec, width: int, eps: float, mult: float, ctx: ParallelContext, dtype, device):
        super().__init__()
        self.spec, self.eps, self.mult, self.dtype = spec, eps, mult, dtype
        self.norm1, self.rg1_b = _param((1,), ctx, device), _param((width,), ctx, device)
        self.mixer = DualMixer(spec, width, eps, ctx, dtype, device, extra=width)       # + the mixer's residual gate
        self.ff = None
        if spec.ff:
            if spec.ff_kind != "moe":
                raise ValueError(f"gated parallel layers take a routed feed-forward, not {spec.ff_kind!r}")
            self.norm2, self.rg2_b = _param((1,), ctx, device), _param((width,), ctx, device)
            self.ff = RoutedFF(spec, width, ctx, dtype, device, extra=width)             # + the feed-forward's residual gate

    def weights(self, p):
        yield p + "norm1", self.norm1, "ones", None
        yield p + "rg1.b", self.rg1_b, "zeros", None
        yield from self.mixer.weights(p + "mix.", extra_src=(p + "rg1",))
        if self.ff is not None:
            yield p + "norm2", self.norm2, "ones", None
            yield p + "rg2.b", self.rg2_b, "zeros", None
            yield from self.ff.weights(p + "mlp.", extra_src=(p + "rg2",))

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        return self.mixer.cache(num_blocks, num_slots, dtype, device)

    def forward(self, x, restart, meta, cache: LayerCache):
        """``x``: fp32 stream ``[T, W]``, updated in place."""
        assert restart is None, "gated parallel layers are not repeated"
        h1, h2 = seqmix.rms_scale(x, self.norm1.data, self.norm2.data if self.ff is not None else None, self.eps, self.dtype)
        parts, gate1 = self.mixer(h1, meta, cache)
        if self.ff is None:
            seqmix.gated_combine(x, self.mult, parts, list(self.spec.part_scales), gate1, self.rg1_b.data)
            return x
        routed, shared, sgate, gate2 = self.ff(h2)
        seqmix.gated_combine(x, self.mult, parts, list(self.spec.part_scales), gate1, self.rg1_b.data, routed, shared, sgate,
                             gate2, self.rg2_b.data)
        return x


class MixerLayer(nn.Module):
    def __init__(self, spec: MixerSpec, width: int, eps: float, mult: float, ctx: ParallelContext, dtype, device):
        super().__init__()
        self.spec, self.eps, self.mult, self.dtype = spec, eps, mult, dtype
        self.norm1, self.norm1b = Norm(width, ctx, device), Norm(width, ctx, device)
        self.norm2, self.norm2b = Norm(width, ctx, device), Norm(width, ctx, device)
        self.shift = _param((width,), ctx, device)
        self.mixer = MIXERS[spec.kind](spec, width, eps, ctx, dtype, device)
        self.ff = DenseFF(width, spec.ff, ctx, dtype, device) if spec.ff else None

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        c = self.mixer.cache(num_blocks, num_slots, dtype, device)
        c.shift = torch.zeros(num_slots, self.shift.data.shape[0], dtype=torch.float32, device=device)
        return c

    def forward(self, x, restart, meta, cache: LayerCache):
        """``x``: fp32 stream ``[T, W]``, updated in place (a fresh tensor is returned when ``restart`` — the term added in
        front of a repeated pass — is given)."""
        eps, m = self.eps, self.mult
        h, x = seqmix.ln_shift(x, restart, self.norm1.w.data, self.norm1.b.data, eps, self.shift.data, cache.shift, meta, self.dtype)
        y = self.mixer(h, meta, cache)
        if self.ff is None:
            seqmix.add_ln(x, y, self.norm1b.w.data, self.norm1b.b.data, eps, m)
            return x
        h = seqmix.add_ln(x, y, self.norm1b.w.data, self.norm1b.b.data, eps, m, self.norm2.w.data, self.norm2.b.data, self.dtype)
        seqmix.add_ln(x, self.ff(h), self.norm2b.w.data, self.norm2b.b.data, eps, m)
        return x
