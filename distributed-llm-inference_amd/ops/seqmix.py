"""Ops of the heterogeneous decoder stacks (``models/mixers.py``): layer norm with token shift, the
post-norm residual update, token-major paged attention with a sliding window / distance penalty / two-part
scores (latent attention), the decayed linear-attention scan over per-sequence state, and the small
element-wise pieces around them.

Same contract as the rest of ``dli_amd.ops``: GPU tensors go to the gfx950 kernels
(``csrc/kernels/seqmix.hip``, ``torch.ops.dli.sm_*``), CPU tensors to the fp32 torch references below.  The
residual stream, norm statistics, scores, softmax weights, rotation angles and the recurrent state are fp32 in
both; activations between GEMMs are the model dtype (bf16 or fp32).

Cache layout of these mixers: *token-major* pages ``[num_blocks, KV_BLOCK_SIZE, row]`` — one contiguous row per
token (all key heads, or latent | rotated key), addressed by the same slot ids (``page · 32 + offset``) as the
other caches.  State tensors are ``[slots, …]`` fp32 rows addressed by ``AttnMetadata.state_slots``.
"""
from __future__ import annotations

import os
from typing import Optional

import torch

from ..config import KV_BLOCK_SIZE


TILE_ATTENTION = os.environ.get("DLI_TILE_ATTENTION", "1") != "0"     # A/B knob: prefill tiles on the matrix cores (bf16)
HEAD_DECODE = os.environ.get("DLI_HEAD_DECODE", "1") != "0"           # A/B knob: decode rows of head-sharing mixers on the matrix cores
BLOCK_SCAN = os.environ.get("DLI_BLOCK_SCAN", "1") != "0"             # A/B knob: block-parallel lightning prefill
PREFILL_TILE_TOKENS = 64                                                # queries per prefill tile of these stacks


def _hip():
    from . import hip
    return hip()


def _act_ok(x: torch.Tensor) -> bool:
    if not x.is_cuda:
        return False
    if x.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f"the sequence-mixer kernels take bfloat16 or float32 activations, got {x.dtype}")
    return True


def _ln(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return d * torch.rsqrt((d * d).mean(-1, keepdim=True) + eps) * w + b


def rotary_inv_freq(base: float, dims: int, device="cpu") -> torch.Tensor:
    """float64 ``[dims/2]``: ``base**(-2i/dims)`` — the kernels multiply by the position in double and reduce the angle
    before the fp32 sine / cosine, so position 10⁶ is as exact as position 1."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims).to(device)


# ------------------------------------------------------------------------------------ norms
def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """``(x - mean) / sqrt(var + eps) · w + b`` over fp32 rows; ``out_dtype`` result."""
    if x.is_cuda:
        return _hip().sm_layer_norm(x, w, b, eps, out_dtype == torch.bfloat16)
    return _ln(x.float(), w, b, eps).to(out_dtype)


def ln_shift(x: torch.Tensor, add: Optional[torch.Tensor], w: torch.Tensor, b: torch.Tensor, eps: float, mix: torch.Tensor,
             state: torch.Tensor, meta, out_dtype: torch.dtype):
    """Pre-norm of a mixer with token shift.  ``x`` fp32 ``[T, W]`` (``add``: added first — the stream's restart term);
    ``g = layer_norm(x)``; result row ``t`` = ``g[t] + (g[t-1] - g[t]) · mix`` where ``g[t-1]`` is the previous token of the
    same sequence: the row above inside a chunk, the sequence's ``state`` row at a chunk start, zero at position 0.  The
    state row becomes ``g`` of the sequence's last token of this step.  Returns ``(h, x)`` with ``x`` the (new) stream."""
    if x.is_cuda:
        return _hip().sm_ln_shift(x, add, w, b, eps, mix, state, meta.positions, meta.token_seq, meta.query_start_loc,
                                  meta.state_slots, meta.counts, meta.num_seqs, out_dtype == torch.bfloat16)
    if add is not None:
        x = x + add
    g = _ln(x, w, b, eps)
    prev = torch.zeros_like(g)
    prev[1:] = g[:-1]
    B = meta.num_decode + meta.num_prefill
    qsl = meta.query_start_loc[:B + 1].tolist()
    slots = meta.state_slots[:B].tolist()
    for i in range(B):
        t0, t1 = qsl[i], qsl[i + 1]
        if t1 <= t0 or slots[i] < 0:
            continue
        prev[t0] = state[slots[i]] if int(meta.positions[t0]) > 0 else 0.0
        state[slots[i]] = g[t1 - 1]
    return (g + (prev - g) * mix).to(out_dtype), x


def add_ln(x: torch.Tensor, y: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float, mult: float,
           w2: Optional[torch.Tensor] = None, b2: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """In place on the fp32 stream: ``x += mult · layer_norm(y; w, b)``; with ``w2`` / ``b2`` also returns
    ``layer_norm(x; w2, b2)`` (the next sublayer's input) — one pass over the row."""
    if x.is_cuda:
        h = _hip().sm_add_ln(x, y, w, b, eps, mult, w2, b2, out_dtype == torch.bfloat16)
        return None if w2 is None else h
    x.add_(_ln(y.float(), w, b, eps), alpha=mult)
    return None if w2 is None else _ln(x, w2, b2, eps).to(out_dtype)


def rms_gate(o: torch.Tensor, w: Optional[torch.Tensor], eps: float, gate: torch.Tensor, out_dtype: torch.dtype, groups: int = 1,
             gate_act: str = "sigmoid") -> torch.Tensor:
    """``o / rms(o) · w · act(gate)`` per row (``o`` fp32 ``[T, N]``, or — what the GPU scan returns — planes of partial
    sums ``[parts, T, N]`` whose sum is the row; ``gate`` a row-strided view).  ``groups`` > 1: every one of that many equal
    slices of the row is divided by its own root mean square; ``w`` None: no weight; ``gate_act``: ``"sigmoid"`` or ``"silu"``."""
    assert gate_act in ("sigmoid", "silu")
    if o.is_cuda:
        return _hip().sm_rms_gate(o, w, eps, gate, out_dtype == torch.bfloat16, groups, gate_act == "silu")
    if o.dim() == 3:
        o = o.sum(0)
    T, N = o.shape
    g = o.view(T, groups, N // groups)
    y = (g * torch.rsqrt((g * g).mean(-1, keepdim=True) + eps)).reshape(T, N)
    if w is not None:
        y = y * w
    z = gate.float()
    return (y * (torch.sigmoid(z) if gate_act == "sigmoid" else torch.nn.functional.silu(z))).to(out_dtype)


def relu2(x: torch.Tensor) -> torch.Tensor:
    """``max(x, 0)²`` element-wise."""
    if _act_ok(x):
        return _hip().sm_relu2(x)
    z = torch.clamp(x.float(), min=0.0)
    return (z * z).to(x.dtype)


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """fp32 ``cap · tanh(logits / cap)``."""
    if logits.is_cuda:
        return _hip().sm_softcap(logits, cap)
    return cap * torch.tanh(logits.float() / cap)


# ------------------------------------------------------------------------------------ cache writers
def qk_norm_cache(qkv: torch.Tensor, qw: torch.Tensor, kw: torch.Tensor, eps: float, slot_mapping: torch.Tensor,
                  k_cache: torch.Tensor, v_cache: torch.Tensor, H: int, G: int, D: int, Dv: int) -> None:
    """``qkv [T, H·D + G·D + G·Dv]``: every query and key head is divided by its root mean square and multiplied by
    ``qw`` / ``kw`` (fp32 ``[D]``); queries are written back in place, keys and values go to the token-major cache rows
    ``slot_mapping`` (< 0: skipped)."""
    if _act_ok(qkv):
        _hip().sm_qk_norm_cache(qkv, qw, kw, eps, slot_mapping, k_cache, v_cache, H, G, D, Dv)
        return
    T = qkv.shape[0]
    q = qkv[:, :H * D].float().view(T, H, D)
    k = qkv[:, H * D:(H + G) * D].float().view(T, G, D)
    q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps) * qw
    k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps) * kw
    qkv[:, :H * D] = q.reshape(T, H * D).to(qkv.dtype)
    keep = slot_mapping >= 0
    s = slot_mapping[keep].long()
    k_cache.view(-1, G * D)[s] = k.reshape(T, G * D)[keep].to(k_cache.dtype)
    v_cache.view(-1, G * Dv)[s] = qkv[:, (H + G) * D:][keep].to(v_cache.dtype)


def _rotate(v: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, dims: int) -> torch.Tensor:
    """v fp32 ``[T, …, R]``: pairs (2i, 2i+1) of the first ``dims`` entries turned by ``position · inv_freq[i]``."""
    ang = positions.double()[:, None] * inv_freq[None, :]
    cos, sin = ang.cos().float(), ang.sin().float()
    while cos.dim() < v.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out = v.clone()
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


def latent_prep(q: torch.Tensor, dkv: torch.Tensor, cw: torch.Tensor, eps: float, positions: torch.Tensor,
                inv_freq: torch.Tensor, rot_dims: int, slot_mapping: torch.Tensor, cache: torch.Tensor,
                H: int, D: int, R: int, C: int) -> None:
    """Latent attention, per token: the first ``C`` entries of ``dkv [T, C+R]`` divided by their root mean square times
    ``cw`` are the latent, the last ``R`` the shared key part, rotated for the token's position; both go to the cache row
    ``[latent | rotated key]``.  The rotated part (last ``R`` of every ``D+R`` head slice) of ``q`` is rotated in place."""
    if _act_ok(q):
        _hip().sm_latent_prep(q, dkv, cw, eps, positions, inv_freq, rot_dims, slot_mapping, cache, H, D, R, C)
        return
    T = q.shape[0]
    c = dkv[:, :C].float()
    c = c * torch.rsqrt((c * c).mean(-1, keepdim=True) + eps) * cw
    kr = _rotate(dkv[:, C:].float(), positions, inv_freq, rot_dims)
    qv = q.unflatten(1, (H, D + R))
    qv[:, :, D:] = _rotate(qv[:, :, D:].float(), positions, inv_freq, rot_dims).to(q.dtype)
    keep = slot_mapping >= 0
    s = slot_mapping[keep].long()
    cache.view(-1, C + R)[s] = torch.cat([c, kr], dim=-1)[keep].to(cache.dtype)


# ------------------------------------------------------------------------------------ attention over token-major pages
def token_attention(out: torch.Tensor, q1: torch.Tensor, q2: Optional[torch.Tensor], k_cache: torch.Tensor,
                    v_cache: Optional[torch.Tensor], meta, G: int, Dv: int, scale: float, window: int = 0,
                    temp: Optional[torch.Tensor] = None, r1: Optional[torch.Tensor] = None,
                    r2: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                    sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Softmax attention of this step's tokens over their sequences' cached rows (which already hold this step's keys).

    ``q1 [T, H, D1]`` (and ``q2 [T, H, D2]``) against key rows ``[G, D1 + D2]``: ``score = (q1·k[:D1] + q2·k[D1:]) · scale ·
    temp[h] − r1[h] · ln(1 + r2[h] · distance)``; query head ``h`` reads key / value head ``h // (H/G)``.  ``v_cache`` None:
    the values are the first ``Dv`` entries of the key rows (latent attention: the cached latent is key and value).
    ``window`` > 0: a query at position ``p`` sees positions ``p-window+1 … p``; 0: all up to ``p``.  ``gate [T, H]``
    (pre-activation, row-strided view): head ``h``'s result is multiplied by ``sigmoid(gate[t, h])``.  Views may be strided
    (last dim contiguous).  ``sink`` fp32 ``[H]``: the softmax denominator of head ``h`` also holds ``exp(sink[h])`` (a logit
    without key or value, not scaled).  Writes ``out [T, H, Dv]``."""
    if _act_ok(q1):
        lib = _hip()
        rows = -1
        if TILE_ATTENTION and q1.dtype == torch.bfloat16 and meta.num_prefill_tiles > 0:
            # prefill chunks: 64-query tiles on the matrix cores; the per-token kernel keeps the decode rows in front
            if lib.sm_tile_attention(out, q1, q2, k_cache, v_cache, meta.block_tables, meta.seq_lens, meta.query_start_loc,
                                     meta.prefill_tile_seq, meta.prefill_tile_q0, meta.num_prefill_tiles,
                                     meta.counts if meta.counts_on_device else None, G, Dv, scale, window, temp, r1, r2, gate, sink):
                rows = meta.num_decode
        T, H = q1.shape[0], q1.shape[1]
        todo = T if rows < 0 else rows                       # tokens the tile kernel left (all of them in a pure decode step)
        if (HEAD_DECODE and todo > 0 and q1.dtype == torch.bfloat16 and H // G >= 8 and meta.num_prefill_tiles == (0 if rows < 0 else meta.num_prefill_tiles)
                and lib.sm_head_decode_attention(out, q1, q2, k_cache, v_cache, meta.block_tables, meta.positions, meta.token_seq,
                                                 G, Dv, scale, window, temp, r1, r2, todo, gate, sink)):
            rows = 0                                         # done with the heads as matrix-core columns
        if rows != 0:
            lib.sm_token_attention(out, q1, q2, k_cache, v_cache, meta.block_tables, meta.positions, meta.token_seq,
                                   G, Dv, scale, window, temp, r1, r2, rows, gate, sink)
        return out
    T, H, D1 = q1.shape
    rowk = k_cache.shape[-1]
    D2 = 0 if q2 is None else q2.shape[2]
    Dk = D1 + D2
    assert rowk == G * Dk
    B = meta.num_decode + meta.num_prefill
    qsl = meta.query_start_loc[:B + 1].tolist()
    kflat = k_cache.view(-1, rowk)
    vflat = kflat if v_cache is None else v_cache.view(-1, v_cache.shape[-1])
    for i in range(B):
        t0, t1 = qsl[i], qsl[i + 1]
        if t1 <= t0:
            continue
        pos = meta.positions[t0:t1].long()
        L = int(pos[-1]) + 1
        lo = max(int(pos[0]) - window + 1, 0) if window > 0 else 0
        j = torch.arange(lo, L)
        slots = meta.block_tables[i, j // KV_BLOCK_SIZE].long() * KV_BLOCK_SIZE + j % KV_BLOCK_SIZE
        K = kflat[slots].float().view(-1, G, Dk)
        V = (vflat[slots].float().view(-1, G, vflat.shape[-1] // G))[..., :Dv]
        q = q1[t0:t1].float() if q2 is None else torch.cat([q1[t0:t1].float(), q2[t0:t1].float()], dim=-1)
        rep = H // G
        Kh, Vh = K.repeat_interleave(rep, dim=1), V.repeat_interleave(rep, dim=1)      # [L', H, ·]
        s = torch.einsum("nhd,lhd->nhl", q, Kh) * scale
        if temp is not None:
            s = s * temp.view(1, H, 1)
        dist = (pos[:, None] - j[None, :])                                             # [n, L']
        if r1 is not None:
            s = s - r1.view(1, H, 1) * torch.log1p(r2.view(1, H, 1) * dist.clamp(min=0).float().unsqueeze(1))
        hidden = dist < 0
        if window > 0:
            hidden = hidden | (dist >= window)
        s = s.masked_fill(hidden.unsqueeze(1), float("-inf"))
        if sink is not None:
            pw = torch.softmax(torch.cat([s, sink.view(1, H, 1).expand(t1 - t0, H, 1)], dim=-1), dim=-1)[..., :-1]
        else:
            pw = torch.softmax(s, dim=-1)
        o = torch.einsum("nhl,lhd->nhd", pw, Vh)
        if gate is not None:
            o = o * torch.sigmoid(gate[t0:t1].float()).unsqueeze(2)
        out[t0:t1] = o.to(out.dtype)
    return out


# ------------------------------------------------------------------------------------ decayed linear attention
def lightning_scan(qkvg: torch.Tensor, state: torch.Tensor, meta, H: int, D: int, Dv: int, decay: torch.Tensor,
                   activation: str = "silu") -> torch.Tensor:
    """``qkvg [T, 2·H·D + 2·H·Dv]`` = ``[q | k | v | gate]`` (pre-activation; the gate columns are not read and may be
    missing).  Per sequence and head, token by token: ``S ← decay[h] · S + act(k) act(v)ᵀ``, ``o = Sᵀ act(q)`` with ``S`` = the
    sequence's fp32 ``state[slot, h]`` ``[D, Dv]`` (zero at position 0), written back after the step's last token; ``act`` is
    silu, or the identity with ``activation="none"``.  Returns fp32 ``[T, H·Dv]`` (GPU: ``[parts, T, H·Dv]`` partial sums over
    parts of the state rows, for ``rms_gate``)."""
    assert activation in ("silu", "none")
    if _act_ok(qkvg):
        # prefill chunks run block-parallel over the step's 64-token tiles (local states → prefix over blocks → outputs)
        tiles = meta.num_prefill_tiles if BLOCK_SCAN else 0
        return _hip().sm_lightning_scan(qkvg, state, meta.positions, meta.query_start_loc, meta.state_slots, meta.counts,
                                        meta.num_seqs, H, D, Dv, decay, meta.prefill_tile_seq if tiles else None,
                                        meta.prefill_tile_q0 if tiles else None, tiles, activation == "none")
    T = qkvg.shape[0]
    act = qkvg[:, :2 * H * D + H * Dv].float()
    if activation == "silu":
        act = torch.nn.functional.silu(act)
    q, k, v = act[:, :H * D].view(T, H, D), act[:, H * D:2 * H * D].view(T, H, D), act[:, 2 * H * D:].view(T, H, Dv)
    o = torch.zeros(T, H, Dv)
    B = meta.num_decode + meta.num_prefill
    qsl = meta.query_start_loc[:B + 1].tolist()
    slots = meta.state_slots[:B].tolist()
    lam = decay.view(H, 1, 1)
    for i in range(B):
        t0, t1 = qsl[i], qsl[i + 1]
        if t1 <= t0 or slots[i] < 0:
            continue
        S = state[slots[i]].clone() if int(meta.positions[t0]) > 0 else torch.zeros(H, D, Dv)
        for t in range(t0, t1):
            S = lam * S + k[t].unsqueeze(2) * v[t].unsqueeze(1)
            o[t] = torch.einsum("hde,hd->he", S, q[t])
        state[slots[i]] = S
    return o.view(T, H * Dv)


# ====================================================================================== gated parallel layers
# Ops of stacks whose layers run two mixers and a routed feed-forward side by side on scalar-gain RMS norms of the same
# stream (``models/mixers.py``: ``SinkTalkAttention``, ``TimeMix``, ``RoutedFF``, ``GatedParallelLayer``).  GPU kernels:
# ``csrc/kernels/dualmix.hip`` (``torch.ops.dli.dm_*``).
def _seq_rows(meta):
    """(batch row, first token row, end token row, state slot) of the step's sequences that bring tokens (CPU references)."""
    B = meta.num_decode + meta.num_prefill
    qsl = meta.query_start_loc[:B + 1].tolist()
    slots = meta.state_slots[:B].tolist() if meta.state_slots is not None else [-1] * B
    return [(i, qsl[i], qsl[i + 1], slots[i]) for i in range(B) if qsl[i + 1] > qsl[i]]


def rms_scale(x: torch.Tensor, g1: torch.Tensor, g2: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype):
    """Two scalar-gain RMS norms of the same fp32 rows: ``x / sqrt(mean(x²) + eps) · g`` for ``g1`` and (when given) ``g2``
    (one-element fp32 tensors).  Returns ``(h1, h2 or None)`` in ``out_dtype``."""
    if x.is_cuda:
        h1, h2 = _hip().dm_rms_scale(x, g1, g2, eps, out_dtype == torch.bfloat16)
        return h1, (h2 if g2 is not None else None)
    n = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)
    return (n * g1).to(out_dtype), ((n * g2).to(out_dtype) if g2 is not None else None)


def shift_mix(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, meta) -> torch.Tensor:
    """``out[s, t] = h[t] + (h[t-1] - h[t]) · mu[s]`` for every blend ``s`` (``mu`` fp32 ``[S, W]``), ``h[t-1]`` being the
    previous token of the same sequence: the row above inside a chunk, the sequence's fp32 ``state`` row at a chunk start,
    zero at position 0.  The state row becomes ``h`` of the sequence's last token of this step.  Returns ``[S, T, W]``."""
    if _act_ok(h):
        return _hip().dm_shift_mix(h, mu, state, meta.positions, meta.token_seq, meta.query_start_loc, meta.state_slots,
                                   meta.counts, meta.num_seqs)
    hf = h.float()
    prev = torch.zeros_like(hf)
    prev[1:] = hf[:-1]
    for _i, t0, t1, slot in _seq_rows(meta):
        prev[t0] = state[slot] if int(meta.positions[t0]) > 0 else 0.0
        state[slot] = hf[t1 - 1]
    return (hf.unsqueeze(0) + (prev - hf).unsqueeze(0) * mu.unsqueeze(1)).to(h.dtype)


def stretched_inv_freq(base: float, dims: int, scaling: tuple = (), device="cpu"):
    """Rotation frequencies of ``dims`` rotated entries (float64 ``[dims/2]``) and the magnitude applied to cosine and sine.
    ``scaling = (factor, original, fast, slow)``: pairs that turn more than ``fast`` times over ``original`` positions keep
    their frequency, pairs that turn fewer than ``slow`` times have it divided by ``factor``, with a linear blend over the
    pair index between the two corners; the magnitude is ``0.1 · ln(factor) + 1``."""
    import math
    f = rotary_inv_freq(base, dims, "cpu")
    if not scaling:
        return f.to(device), 1.0
    factor, original, fast, slow = scaling

    def corner(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo, hi = max(math.floor(corner(fast)), 0), min(math.ceil(corner(slow)), dims - 1)
    ramp = ((torch.arange(dims // 2, dtype=torch.float64) - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return (f / factor * ramp + f * (1.0 - ramp)).to(device), 0.1 * math.log(factor) + 1.0


def wide_norm_rope_cache(qkv: torch.Tensor, qw: torch.Tensor, kw: torch.Tensor, eps: float, positions: torch.Tensor,
                         inv_freq: Optional[torch.Tensor], mag: float, rot_dims: int, slot_mapping: torch.Tensor,
                         k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], H: int, G: int, D: int, Dv: int) -> None:
    """Leading columns of ``qkv`` rows = ``[q (H·D) | k (G·D) | v (G·Dv)]``.  The whole q row and the whole k row are each
    divided by their root mean square (over all heads at once) and multiplied by ``qw`` / ``kw``; then entries ``i`` and
    ``i + rot_dims/2`` (``i < rot_dims/2``) of every head are turned by ``position · inv_freq[i]`` with cosine and sine
    scaled by ``mag``.  q is written back in place; k and v go to the token-major cache rows ``slot_mapping`` (< 0: skipped).
    ``G = 0`` (no caches, ``kw`` unused): the rows hold queries only — a mixer that reads another layer's keys and values.
    ``inv_freq`` may be None when nothing is rotated."""
    if _act_ok(qkv):
        _hip().dm_wide_norm_rope_cache(qkv, qw, kw if G else None, eps, positions, inv_freq if rot_dims else None, mag, rot_dims,
                                       slot_mapping, k_cache if G else None, v_cache if G else None, H, G, D, Dv)
        return
    T = qkv.shape[0]
    q, k = qkv[:, :H * D].float(), qkv[:, H * D:(H + G) * D].float()
    q = (q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps) * qw).view(T, H, D)
    if G:
        k = (k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps) * kw).view(T, G, D)
    if rot_dims:
        ang = positions.double()[:, None] * inv_freq[None, :]
        cos, sin = (ang.cos() * mag).float().unsqueeze(1), (ang.sin() * mag).float().unsqueeze(1)
        half = rot_dims // 2

        def turn(v):
            a, b = v[..., :half], v[..., half:rot_dims]
            return torch.cat([a * cos - b * sin, b * cos + a * sin, v[..., rot_dims:]], dim=-1)
        q = turn(q)
        k = turn(k) if G else k
    qkv[:, :H * D] = q.reshape(T, H * D).to(qkv.dtype)
    if not G:
        return
    keep = slot_mapping >= 0
    s = slot_mapping[keep].long()
    k_cache.view(-1, G * D)[s] = k.reshape(T, G * D)[keep].to(k_cache.dtype)
    v_cache.view(-1, G * Dv)[s] = qkv[:, (H + G) * D:(H + G) * D + G * Dv][keep].to(v_cache.dtype)


def talk_attention(out: torch.Tensor, q: torch.Tensor, gate: Optional[torch.Tensor], k_cache: torch.Tensor, v_cache: torch.Tensor,
                   meta, G: int, Dv: int, scale: float, sink: Optional[torch.Tensor], talk: Optional[torch.Tensor]) -> torch.Tensor:
    """Causal softmax attention of this step's tokens over their sequences' cached rows with a per-head ``sink`` in the
    denominator (``p = exp(s) / (Σ exp(s) + exp(sink))``) and the normalised weights mixed across heads:
    ``p'_h = Σ_g talk[h, g] · p_g``; head ``h`` applies ``p'_h`` to the values of its own key / value head ``h // (H/G)``.
    ``q [T, H, D]`` (strided view); ``gate [T, H·Dv]`` (pre-activation): the result is multiplied by its sigmoid.
    Writes ``out [T, H·Dv]``."""
    if _act_ok(q):
        lib = _hip()
        rows = -1
        if TILE_ATTENTION and q.dtype == torch.bfloat16 and meta.num_prefill_tiles > 0:
            # prefill chunks: 16-query tiles on the matrix cores; the per-token kernel keeps the decode rows in front
            if lib.dm_talk_tile_attention(out, q, gate, k_cache, v_cache, meta.block_tables, meta.seq_lens, meta.query_start_loc,
                                          meta.prefill_tile_seq, meta.prefill_tile_q0, meta.num_prefill_tiles,
                                          meta.counts if meta.counts_on_device else None, sink, talk, G, Dv, scale):
                rows = meta.num_decode
        if rows != 0:
            lib.dm_talk_attention(out, q, gate, k_cache, v_cache, meta.block_tables, meta.positions, meta.token_seq,
                                  sink, talk, G, Dv, scale, rows)
        return out
    T, H, D = q.shape
    kflat, vflat = k_cache.view(-1, G * D), v_cache.view(-1, G * Dv)
    rep = H // G
    res = torch.zeros(T, H, Dv)
    for i, t0, t1, _slot in _seq_rows(meta):
        pos = meta.positions[t0:t1].long()
        L = int(pos[-1]) + 1
        j = torch.arange(L)
        slots = meta.block_tables[i, j // KV_BLOCK_SIZE].long() * KV_BLOCK_SIZE + j % KV_BLOCK_SIZE
        K = kflat[slots].float().view(L, G, D).repeat_interleave(rep, dim=1)
        V = vflat[slots].float().view(L, G, Dv).repeat_interleave(rep, dim=1)
        s = torch.einsum("nhd,lhd->nhl", q[t0:t1].float(), K) * scale
        s = s.masked_fill((j[None, :] > pos[:, None]).unsqueeze(1), float("-inf"))
        if sink is not None:
            s = torch.cat([s, sink.view(1, H, 1).expand(t1 - t0, H, 1)], dim=-1)
        p = torch.softmax(s, dim=-1)[..., :L]
        if talk is not None:
            p = torch.einsum("hg,ngl->nhl", talk, p)
        res[t0:t1] = torch.einsum("nhl,lhd->nhd", p, V)
    res = res.view(T, H * Dv)
    if gate is not None:
        res = res * torch.sigmoid(gate.float())
    out.copy_(res.to(out.dtype))
    return out


def decay_lora(a: torch.Tensor, w2: torch.Tensor, w0: torch.Tensor) -> torch.Tensor:
    """fp32 ``exp(-exp(w2 · tanh(a) + w0))``: ``a [T, L]`` is the low-rank projection's output, ``w2 [C, L]``, ``w0`` fp32 ``[C]``."""
    if _act_ok(a):
        return _hip().dm_decay(a, w2, w0)
    return torch.exp(-torch.exp(torch.tanh(a.float()) @ w2.float().t() + w0))


def wkv_scan(rkv: torch.Tensor, w: torch.Tensor, u: torch.Tensor, state: torch.Tensor, meta, H: int, D: int) -> torch.Tensor:
    """``rkv [≥3, T, H·D]`` = receptance, key, value; ``w`` fp32 ``[T, H·D]`` decays; ``u`` fp32 ``[H·D]`` bonus.  Per sequence
    and head, token by token, with ``S`` the sequence's fp32 ``state[slot, h]`` ``[D, D]`` (zero at position 0):
    ``o[e] = Σ_d r[d] · (S[d, e] + u[d] k[d] v[e])``, then ``S[d, e] ← w[d] · S[d, e] + k[d] v[e]``.  Returns fp32 ``[T, H·D]``."""
    if _act_ok(rkv):
        return _hip().dm_wkv_scan(rkv, w, u, state, meta.positions, meta.query_start_loc, meta.state_slots, meta.counts,
                                  meta.num_seqs, H, D)
    T = rkv.shape[1]
    r, k, v = (rkv[i].float().view(T, H, D) for i in range(3))
    wv, uv = w.view(T, H, D), u.view(H, D)
    o = torch.zeros(T, H, D)
    for _i, t0, t1, slot in _seq_rows(meta):
        S = state[slot].clone() if int(meta.positions[t0]) > 0 else torch.zeros(H, D, D)
        for t in range(t0, t1):
            kv = k[t].unsqueeze(2) * v[t].unsqueeze(1)
            o[t] = torch.einsum("hde,hd->he", S + uv.unsqueeze(2) * kv, r[t])
            S = wv[t].unsqueeze(2) * S + kv
        state[slot] = S
    return o.view(T, H * D)


def group_rms_gate(o: torch.Tensor, groups: int, w: torch.Tensor, eps: float, gate: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """Every one of the ``groups`` equal slices of an fp32 row is divided by its own root mean square; the row is then
    multiplied by ``w`` and by ``silu(gate)`` (``gate``: pre-activation rows, strided view)."""
    if o.is_cuda:
        return _hip().dm_group_rms_gate(o, groups, w, eps, gate, out_dtype == torch.bfloat16)
    T, C = o.shape
    g = o.view(T, groups, C // groups)
    g = g * torch.rsqrt((g * g).mean(-1, keepdim=True) + eps)
    return (g.reshape(T, C) * w * torch.nn.functional.silu(gate.float())).to(out_dtype)


def sigmoid_route(h: torch.Tensor, router: torch.Tensor, experts: int, top: int, scale: float):
    """fp32 ``s = sigmoid(router · h)`` per token; the ``top`` experts with the largest scores (ties: lowest index) and
    their weights ``s · scale`` (not renormalised).  ``router`` fp32 ``[experts (+1), W]``: a last extra row is a per-token
    gate, returned as its sigmoid.  Returns ``(ids int32 [T, top], weights fp32 [T, top], extra fp32 [T] or None)``."""
    if _act_ok(h):
        ids, wts, extra = _hip().dm_sigmoid_route(h, router, experts, top, scale)
        return ids, wts, (extra if router.shape[0] > experts else None)
    z = h.float() @ router.t()
    val, ids = torch.sort(z[:, :experts], dim=-1, descending=True, stable=True)   # by logit: the same order, no saturated ties
    return ids[:, :top].int(), torch.sigmoid(val[:, :top]) * scale, (torch.sigmoid(z[:, experts]) if router.shape[0] > experts else None)


def relu2_experts(h: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    """``Σ_slots wts[t, s] · down[e] · relu(up[e] · h[t])²`` with ``e = ids[t, s]``; ``up [E, F, W]``, ``down [E, W, F]``."""
    if _act_ok(h):
        return _hip().dm_relu2_experts(h, ids, wts, up, down, False)
    out = torch.zeros(h.shape[0], h.shape[1])
    hf = h.float()
    for e in range(up.shape[0]):
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        if tok.numel():
            a = torch.clamp(hf[tok] @ up[e].float().t(), min=0.0)
            a = (a * a).to(h.dtype).float()
            out.index_add_(0, tok, (a @ down[e].float().t()) * wts[tok, slot].unsqueeze(1))
    return out.to(h.dtype)


def relu2_rows(x: torch.Tensor) -> torch.Tensor:
    """``max(x, 0)²`` of a row-strided 2-D view, as a contiguous tensor."""
    if _act_ok(x):
        return _hip().dm_relu2_rows(x)
    z = torch.clamp(x.float(), min=0.0)
    return (z * z).to(x.dtype)


def gated_combine(x: torch.Tensor, mult: float, parts: list, scales: list, gate1: torch.Tensor, b1: torch.Tensor,
                  ff: Optional[torch.Tensor] = None, shared: Optional[torch.Tensor] = None, shared_gate: Optional[torch.Tensor] = None,
                  gate2: Optional[torch.Tensor] = None, b2: Optional[torch.Tensor] = None) -> None:
    """In place on the fp32 stream: ``x += mult · (sigmoid(gate1 + b1) ⊙ Σ_i scales[i] · parts[i] + sigmoid(gate2 + b2) ⊙
    (ff + shared_gate ⊙ shared))`` — the second term only with ``gate2``; ``shared_gate`` fp32 ``[T]`` (already a sigmoid)."""
    if x.is_cuda:
        assert len(parts) == 2, "the kernel combines two mixers"
        _hip().dm_gated_combine(x, mult, parts[0], parts[1], scales[0], scales[1], gate1, b1, ff, shared, shared_gate, gate2, b2)
        return
    y = sum(s * p.float() for s, p in zip(scales, parts)) * torch.sigmoid(gate1.float() + b1)
    if gate2 is not None:
        f = ff.float() if ff is not None else 0.0
        if shared is not None:
            f = f + shared.float() * (shared_gate.unsqueeze(1) if shared_gate is not None else 1.0)
        y = y + f * torch.sigmoid(gate2.float() + b2)
    x.add_(y, alpha=mult)


# ====================================================================================== hyper-connected stacks
# Ops of stacks that keep several copies of the residual stream, add a short causal convolution to every mixer's input and
# mix gated attention / retention layers with gated dense or softmax-routed feed-forwards (``models/mixers.py``:
# ``GatedAttention``, ``Retention``, ``GatedDenseFF``, ``SoftmaxRoutedFF``, ``HyperLayer``).  GPU kernels:
# ``csrc/kernels/hypermix.hip`` (``torch.ops.dli.hm_*``) beside extensions of the kernels above.
def stream_mix_norm(x: torch.Tensor, y: Optional[torch.Tensor], mix: Optional[torch.Tensor], out_w: Optional[torch.Tensor],
                    in_w: Optional[torch.Tensor], norm_w: Optional[torch.Tensor], eps: float, w_offset: float,
                    out_dtype: torch.dtype, center: bool = False) -> Optional[torch.Tensor]:
    """One pass over the fp32 streams ``x [T, S, W]``.  With ``y [T, W]`` (a sublayer's output): all streams at once from the
    old ones, in place, ``x[:, t] ← Σ_s mix[s, t] · x[:, s] + out_w[t] · y``.  With ``in_w [S]``: returns
    ``rms_norm(Σ_s in_w[s] · x[:, s]) · (w_offset + norm_w)`` in ``out_dtype`` — what the next sublayer (or the LM head)
    reads, computed from the updated streams.  ``center``: a layer norm without bias instead — the mean is taken off first and
    the statistic is the variance."""
    if x.is_cuda:
        h = _hip().hm_stream_mix_norm(x, y, mix, out_w, in_w, norm_w, eps, w_offset, out_dtype == torch.bfloat16, center)
        return h if in_w is not None else None
    if y is not None:
        new = torch.einsum("st,nsw->ntw", mix, x) + out_w.view(1, -1, 1) * y.float().unsqueeze(1)
        x.copy_(new)
    if in_w is None:
        return None
    u = torch.einsum("s,nsw->nw", in_w, x)
    if center:
        u = u - u.mean(-1, keepdim=True)
    return (u * torch.rsqrt((u * u).mean(-1, keepdim=True) + eps) * (w_offset + norm_w)).to(out_dtype)


def causal_conv_add(h: torch.Tensor, w: torch.Tensor, state: torch.Tensor, meta, out_dtype: torch.dtype) -> torch.Tensor:
    """``h [T, W]`` fp32; ``w [taps, W]`` fp32 (tap-major: the last row weighs the token itself).  Row ``t`` of the result is
    ``h[t] + Σ_j w[j] · h[t - taps + 1 + j]`` over the
    rows of the same sequence: rows above inside a chunk, the sequence's ``state`` rows ``[slots, taps-1, W]`` (its last
    ``taps-1`` inputs, oldest first) before a chunk's start, zero before position 0.  The state rows are then moved on to
    the sequence's last ``taps-1`` inputs of this step."""
    if h.is_cuda:
        return _hip().hm_causal_conv_add(h, w, state, meta.positions, meta.token_seq, meta.query_start_loc, meta.state_slots,
                                         meta.counts, meta.num_seqs, out_dtype == torch.bfloat16)
    taps = w.shape[0]
    out = h.clone()
    for _i, t0, t1, slot in _seq_rows(meta):
        p0 = int(meta.positions[t0])
        n = t1 - t0
        hist = state[slot].clone() if taps > 1 else h.new_zeros(0, h.shape[1])          # positions p0-(taps-1) … p0-1
        for r in range(taps - 1):
            if p0 - (taps - 1) + r < 0:
                hist[r] = 0.0
        ext = torch.cat([hist, h[t0:t1]], dim=0)                                         # [taps-1+n, W]
        for j in range(taps):
            out[t0:t1] += w[j] * ext[j:j + n]
        if taps > 1:
            state[slot] = ext[n:]
    return out.to(out_dtype)


def retention_prep(qkvg: torch.Tensor, positions: torch.Tensor, inv_freq: Optional[torch.Tensor], rot_dims: int, H: int, D: int,
                   Dv: int, k_scale: float) -> torch.Tensor:
    """fp32 ``[T, 2·H·D + H·Dv]`` = ``[q' | k' | v]`` from the leading columns ``[q | k | v]`` of ``qkvg``: in every head of q
    and k, entries ``i`` and ``i + rot_dims/2`` (``i < rot_dims/2``) are turned by ``position · inv_freq[i]``; k is then
    multiplied by ``k_scale``."""
    if _act_ok(qkvg):
        return _hip().hm_retention_prep(qkvg, positions, inv_freq if rot_dims else None, rot_dims, H, D, Dv, k_scale)
    T = qkvg.shape[0]
    x = qkvg[:, :2 * H * D + H * Dv].float().clone()
    qk = x[:, :2 * H * D].view(T, 2 * H, D)
    if rot_dims:
        ang = positions.double()[:T, None] * inv_freq[None, :]
        cos, sin = ang.cos().float().unsqueeze(1), ang.sin().float().unsqueeze(1)
        half = rot_dims // 2
        a, b = qk[..., :half].clone(), qk[..., half:rot_dims].clone()
        qk[..., :half] = a * cos - b * sin
        qk[..., half:rot_dims] = b * cos + a * sin
    qk[:, H:] *= k_scale
    return x


def act_mul(x: torch.Tensor, kind: str) -> torch.Tensor:
    """``act(x[:, :F]) · x[:, F:]`` of rows ``[T, 2F]``; ``kind``: ``"gelu_tanh"`` (``0.5 z (1 + tanh(√(2/π) (z + 0.044715 z³)))``)
    or ``"silu"``."""
    assert kind in ("gelu_tanh", "silu")
    if _act_ok(x):
        return _hip().hm_act_mul(x, kind == "silu")
    F = x.shape[1] // 2
    a, b = x[:, :F].float(), x[:, F:].float()
    a = torch.nn.functional.gelu(a, approximate="tanh") if kind == "gelu_tanh" else torch.nn.functional.silu(a)
    return (a * b).to(x.dtype)


def softmax_route(h: torch.Tensor, router: torch.Tensor, bias: Optional[torch.Tensor], top: int):
    """fp32 logits ``router · h + bias`` per token (``router`` fp32 ``[E, W]``); the ``top`` experts with the largest logits
    (ties: lowest index) and the softmax over the chosen logits only.  Returns ``(ids int32 [T, top], weights fp32 [T, top])``."""
    if _act_ok(h):
        return _hip().hm_softmax_route(h, router, bias, top)
    z = h.float() @ router.t()
    if bias is not None:
        z = z + bias
    val, ids = torch.sort(z, dim=-1, descending=True, stable=True)
    return ids[:, :top].int(), torch.softmax(val[:, :top], dim=-1)


def gated_experts(h: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor,
                  limit: float = 0.0) -> torch.Tensor:
    """``Σ_slots wts[t, s] · down[e] · (silu(gate[e] · h[t]) ⊙ up[e] · h[t])`` with ``e = ids[t, s]``; ``gate_up [E, 2F, W]``
    (an expert's gate rows, then its up rows), ``down [E, W, F]``.  ``limit`` > 0: the clamped form instead —
    ``g = min(gate · h, limit)``, ``u = clamp(up · h, ±limit)``, activation ``g · sigmoid(1.702 g) · (u + 1)`` — and an id
    ``e ≥ E`` names an identity expert, whose output is ``h[t]`` itself."""
    if _act_ok(h):
        if limit > 0.0:
            return _hip().rm_clamped_experts(h, ids, wts, gate_up, down, limit)
        return _hip().dm_relu2_experts(h, ids, wts, gate_up, down, True)
    F = gate_up.shape[1] // 2
    out = torch.zeros(h.shape[0], h.shape[1])
    hf = h.float()
    for e in range(gate_up.shape[0]):
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        if tok.numel():
            gu = hf[tok] @ gate_up[e].float().t()
            if limit > 0.0:
                g, u = gu[:, :F].clamp(max=limit), gu[:, F:].clamp(-limit, limit)
                a = (g * torch.sigmoid(1.702 * g) * (u + 1.0)).to(h.dtype).float()
            else:
                a = (torch.nn.functional.silu(gu[:, :F]) * gu[:, F:]).to(h.dtype).float()
            out.index_add_(0, tok, (a @ down[e].float().t()) * wts[tok, slot].unsqueeze(1))
    if limit > 0.0:
        out += hf * (wts * (ids >= gate_up.shape[0])).sum(-1, keepdim=True)
    return out.to(h.dtype)


# ====================================================================================== gated recurrences, gated latent attention
# Ops of stacks that alternate a gated linear recurrence per channel with latent attention behind a normed query latent
# (``models/mixers.py``: ``GatedLinearRecurrence``, ``GatedLatentAttention``, ``ScoreRoutedFF``).  GPU kernels:
# ``csrc/kernels/recurmix.hip`` (``torch.ops.dli.rm_*``) beside extensions of the kernels above.
def causal_conv(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor, meta,
                out_dtype: torch.dtype) -> torch.Tensor:
    """``x [T, C]`` (a row-strided view); ``w [taps, C]`` fp32 (tap-major: the last row weighs the token itself).  Row ``t`` of
    the result is ``bias + Σ_j w[j] · x[t - taps + 1 + j]`` over the rows of the same sequence: rows above inside a chunk, the
    sequence's ``state`` rows ``[slots, taps-1, C]`` (its last ``taps-1`` inputs, oldest first) before a chunk's start, zero
    before position 0.  The state rows are then moved on to the sequence's last ``taps-1`` inputs of this step."""
    if _act_ok(x):
        return _hip().rm_causal_conv(x, w, bias, state, meta.positions, meta.token_seq, meta.query_start_loc, meta.state_slots,
                                     meta.counts, meta.num_seqs, out_dtype == torch.bfloat16)
    taps, C = w.shape
    xf = x.float()
    out = torch.zeros(x.shape[0], C)
    for _i, t0, t1, slot in _seq_rows(meta):
        p0, n = int(meta.positions[t0]), t1 - t0
        hist = state[slot].clone() if taps > 1 else xf.new_zeros(0, C)
        for r in range(taps - 1):
            if p0 - (taps - 1) + r < 0:
                hist[r] = 0.0
        ext = torch.cat([hist, xf[t0:t1]], dim=0)
        for j in range(taps):
            out[t0:t1] += w[j] * ext[j:j + n]
        if taps > 1:
            state[slot] = ext[n:]
    if bias is not None:
        out = out + bias
    return out.to(out_dtype)


def rglru_scan(z: torch.Tensor, u: torch.Tensor, y: torch.Tensor, gate_bias: torch.Tensor, rate: torch.Tensor, state: torch.Tensor,
               meta, out_dtype: torch.dtype) -> torch.Tensor:
    """The gated linear recurrence per channel.  ``z [B, T, 2·n]``: pre-activations of the recurrence gate (first ``n`` of a
    block's row) and the input gate (last ``n``) of the ``B`` blocks of ``n`` channels, before their biases ``gate_bias`` fp32
    ``[2, B·n]``; ``u [T, B·n]`` the recurrence's input; ``y [T, B·n]`` (row-strided view) the other branch before its
    tanh-GELU; ``rate`` fp32 ``[B·n]`` = ``8 · softplus(λ)``.  Per sequence and channel, in fp32, token by token:
    ``a = exp(-rate · sigmoid(z_r + b_r))``, ``S ← a · S + sqrt(1 - a²) · sigmoid(z_i + b_i) · u`` with ``S`` the sequence's
    ``state[slot]`` row (zero at position 0), written back after the step's last token.  Returns ``S · gelu_tanh(y)``."""
    if _act_ok(u):
        # chunks run block-parallel over the step's 64-token tiles (local states → prefix over blocks → outputs)
        tiles = meta.num_prefill_tiles if BLOCK_SCAN else 0
        return _hip().rm_rglru_scan(z, u, y, gate_bias, rate, state, meta.positions, meta.query_start_loc, meta.state_slots,
                                    meta.counts, meta.num_seqs, out_dtype == torch.bfloat16, meta.prefill_tile_seq if tiles else None,
                                    meta.prefill_tile_q0 if tiles else None, tiles)
    B, T, n2 = z.shape
    n = n2 // 2
    zf = z.float().view(B, T, 2, n).permute(2, 1, 0, 3).reshape(2, T, B * n)
    r, i = torch.sigmoid(zf[0] + gate_bias[0]), torch.sigmoid(zf[1] + gate_bias[1])
    a = torch.exp(-rate * r)
    b = torch.sqrt(1.0 - a * a) * i * u.float()
    out = torch.zeros(T, B * n)
    for _i, t0, t1, slot in _seq_rows(meta):
        S = state[slot].clone() if int(meta.positions[t0]) > 0 else torch.zeros(B * n)
        for t in range(t0, t1):
            S = a[t] * S + b[t]
            out[t] = S
        state[slot] = S
    return (out * torch.nn.functional.gelu(y.float(), approximate="tanh")).to(out_dtype)


def _turn_half(v: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, mag: float, dims: int) -> torch.Tensor:
    """fp32 ``[T, …, R]``: entries ``i`` and ``i + dims/2`` turned by ``position · inv_freq[i]``, cosine and sine times ``mag``."""
    ang = positions.double()[:, None] * inv_freq[None, :]
    cos, sin = (ang.cos() * mag).float(), (ang.sin() * mag).float()
    while cos.dim() < v.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    half = dims // 2
    a, b = v[..., :half], v[..., half:dims]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, v[..., dims:]], dim=-1)


def latent_norm_cache(proj: torch.Tensor, Q: int, qw: torch.Tensor, cw: Optional[torch.Tensor], eps: float, positions: torch.Tensor,
                      inv_freq: torch.Tensor, mag: float, rot_dims: int, slot_mapping: torch.Tensor, cache: Optional[torch.Tensor],
                      C: int, R: int) -> torch.Tensor:
    """Leading columns of ``proj`` rows = ``[query latent (Q) | key / value latent (C) | shared key part (R)]``.  Returns the
    query latent divided by its root mean square times ``qw`` (contiguous ``[T, Q]``).  With ``cache`` (token-major rows
    ``[latent | rotated key]``): the key / value latent, divided by its root mean square times ``cw``, and the shared key
    part, entries ``i`` and ``i + rot_dims/2`` turned by ``position · inv_freq[i]`` with cosine and sine times ``mag``, go to
    the rows ``slot_mapping`` (< 0: skipped).  Without: the rows hold the query latent only."""
    if _act_ok(proj):
        return _hip().rm_latent_norm_cache(proj, Q, qw, cw, eps, positions, inv_freq, mag, rot_dims, slot_mapping, cache, C, R)
    T = proj.shape[0]
    cq = proj[:, :Q].float()
    cq = (cq * torch.rsqrt((cq * cq).mean(-1, keepdim=True) + eps) * qw).to(proj.dtype)
    if cache is not None:
        c = proj[:, Q:Q + C].float()
        c = c * torch.rsqrt((c * c).mean(-1, keepdim=True) + eps) * cw
        kr = _turn_half(proj[:, Q + C:Q + C + R].float(), positions[:T], inv_freq, mag, rot_dims)
        keep = slot_mapping[:T] >= 0
        cache.view(-1, C + R)[slot_mapping[:T][keep].long()] = torch.cat([c, kr], dim=-1)[keep].to(cache.dtype)
    return cq


def rotate_heads(q: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, mag: float, rot_dims: int, H: int, D: int,
                 R: int) -> None:
    """In place on ``q [T, H·(D+R)]``: in the last ``R`` entries of every head, entries ``i`` and ``i + rot_dims/2`` are
    turned by ``position · inv_freq[i]`` with cosine and sine times ``mag`` (fp32 arithmetic)."""
    if _act_ok(q):
        _hip().rm_rotate_heads(q, positions, inv_freq, mag, rot_dims, H, D, R)
        return
    T = q.shape[0]
    qv = q.view(T, H, D + R)
    qv[:, :, D:] = _turn_half(qv[:, :, D:].float(), positions[:T], inv_freq, mag, rot_dims).to(q.dtype)


def gate_heads(o: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """``o [H, T, Dv]`` (head-major) times ``sigmoid(gate [T, H·Dv])`` (pre-activation, row-strided view), as token-major
    contiguous rows ``[T, H·Dv]``."""
    if _act_ok(o):
        return _hip().rm_gate_heads(o, gate)
    H, T, Dv = o.shape
    return (o.float().transpose(0, 1).reshape(T, H * Dv) * torch.sigmoid(gate.float())).to(o.dtype)


def softmax_all_route(h: torch.Tensor, router: torch.Tensor, choice_bias: Optional[torch.Tensor], top: int):
    """fp32 scores ``s = softmax(router · h)`` over ALL router outputs (``router`` fp32 ``[E, W]``); the ``top`` outputs with
    the largest ``s + choice_bias`` are chosen (ties: lowest index) and weigh ``s / (Σ_chosen s + 1e-20)`` — the bias moves the
    choice, not the weights.  Returns ``(ids int32 [T, top], weights fp32 [T, top])``."""
    if _act_ok(h):
        return _hip().hm_softmax_route(h, router, choice_bias, top, True)
    sc = torch.softmax(h.float() @ router.t(), dim=-1)
    ch = sc if choice_bias is None else sc + choice_bias
    _val, ids = torch.sort(ch, dim=-1, descending=True, stable=True)
    ids = ids[:, :top]
    w = torch.gather(sc, 1, ids)
    return ids.int(), w / (w.sum(-1, keepdim=True) + 1e-20)
