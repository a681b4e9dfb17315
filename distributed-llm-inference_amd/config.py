"""Configuration dataclasses for the serving stack.

The reference has no server-side configuration at all (its only config is the harness dict at
`/root/reference/traffic_generator/main.py:302-313`); SURVEY.md §5.6 asks for a dataclass config
for the new server.  Model shapes are the public ones listed in SURVEY.md §2.5.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass, field
from typing import Optional

KV_BLOCK_SIZE = 32          # tokens per KV page: one MFMA k-step (16x16x32) of the P·V product


@dataclass(frozen=True)
class MixerSpec:
    """One layer of a heterogeneous stack (``ModelConfig.layer_specs``): which sequence mixer it has, the mixer's sizes and
    constants, and its feed-forward.  Fields a mixer kind does not use stay at their defaults.

    ``kind``: ``"attention"`` (grouped-query softmax attention over a sliding window, unit-RMS queries / keys, per-head
    temperature and logarithmic distance penalty), ``"latent_attention"`` (keys / values expanded from a cached low-rank
    latent + one shared rotated key part), ``"lightning"`` (linear attention with a per-head decay and a recurrent state),
    ``"sink_attention"`` (causal grouped-query attention: q / k normalised over the whole projection, half-split rotation of
    the leading ``rot_dims`` entries of every head with optionally stretched frequencies, a per-head sink in the softmax
    denominator, softmax weights mixed across heads, sigmoid output gate), ``"time_mix"`` (recurrence with a per-token,
    per-channel decay from a low-rank projection, a bonus for the current token and a ``[D, D]`` state per head; all five
    projections read their own blend of the token's and the previous token's input), ``"parallel"`` (the mixers in
    ``parts`` read the same input; their outputs are summed with the weights ``part_scales``), ``"gated_attention"`` (causal
    grouped-query softmax attention without positions: q / k normalised over the whole projection, one sigmoid output gate
    per head; ``kv_from`` ≥ 0: the layer has no key / value projections and reads that layer's cache) or ``"retention"``
    (linear attention with a per-head decay and no activation or denominator: half-split rotation of the leading
    ``rot_dims`` entries of q and k, keys scaled by ``dim**-0.5``, a ``[D, Dv]`` state per head, per-head unit RMS and a
    silu gate behind it), ``"rglru"`` (a gated linear recurrence per channel, ``heads`` blocks of ``dim`` channels: a causal
    convolution over ``conv_taps`` inputs, block-diagonal recurrence and input gates, decay ``exp(-8 · r · softplus(λ))``,
    the state multiplied by a tanh-GELU branch) or ``"gated_latent_attention"`` (latent attention whose queries come from a
    normed latent of size ``q_rank``: half-split rotation with optionally stretched frequencies, sliding ``window``, a
    per-head ``sink`` in the softmax denominator, an element-wise sigmoid output gate; ``kv_from`` ≥ 0: the layer reads that
    layer's cached latents and rotated keys and expands them with its own matrices)."""
    kind: str
    heads: int
    dim: int                            # per-head query / key size (latent attention: the unrotated part)
    vdim: int
    kv_heads: int = 0                   # attention: key / value heads
    scale: float = 1.0                  # multiplies q·k
    window: int = 0                     # attention, gated latent attention: a query sees itself and the window-1 tokens before it (0: all)
    kv_rank: int = 0                    # latent attention: size of the cached latent
    rot_dim: int = 0                    # latent attention: size of the rotated query / key part
    rot_base: float = 10000.0
    rot_dims: int = 0                   # leading entries of the rotated part that are actually rotated
    decay: tuple = ()                   # lightning: per-head state decay
    rot_scaling: tuple = ()             # sink / gated latent attention: (factor, original length, fast turns, slow turns) or ()
    lora: int = 0                       # time mix: rank of the decay projection
    parts: tuple = ()                   # parallel: the mixers run side by side (MixerSpec each)
    part_scales: tuple = ()             # parallel: weight of every part's output
    ff: int = 0                         # feed-forward inner width (0: the layer has none); routed: of ONE expert
    ff_kind: str = "dense"              # "dense" | "moe" (sigmoid-routed squared-ReLU experts + optional gated shared expert)
    experts: int = 0                    # moe: number of routed experts
    top: int = 0                        # moe: experts per token
    router_scale: float = 1.0           # moe: multiplies the chosen experts' scores
    shared_ff: int = 0                  # moe: inner width of the expert every token takes (0: none)
    kv_from: int = -1                   # gated (latent) attention: index of the layer whose cached rows this layer reads (-1: its own)
    ff_act: str = "relu2"               # feed-forward activation: "relu2" | "gelu_tanh" / "silu" (gated) | "clamped" (gated experts)
    router: str = "sigmoid"             # moe: "sigmoid" (scores, not renormalised) | "softmax" (biased logits, softmax over the chosen)
                                        # | "softmax_all" (softmax over all logits, a choice bias, renormalised over the chosen)
    q_rank: int = 0                     # gated latent attention: size of the normed query latent
    sink: bool = False                  # gated latent attention: a learned per-head logit in the softmax denominator
    conv_taps: int = 0                  # rglru: taps of the causal convolution in front of the recurrence
    identity_experts: int = 0           # moe ("softmax_all"): trailing router outputs whose expert returns its input
    ff_limit: float = 0.0               # moe ("clamped" experts): bound of the gate (above) and of the up projection (both sides)
    ff_bias: bool = False               # dense feed-forward: the three projections have biases

    @property
    def stateful(self) -> bool:
        return self.kind in ("lightning", "time_mix", "retention", "rglru") or any(p.stateful for p in self.parts)

    @property
    def cache_row(self) -> tuple:
        """Widths of the per-token rows this mixer keeps in the paged cache: ``(key row, value row)``; a latent mixer keeps
        one row (latent | rotated key) that serves as both; a recurrent one keeps none."""
        if self.kind in ("attention", "sink_attention") or (self.kind == "gated_attention" and self.kv_from < 0):
            return self.kv_heads * self.dim, self.kv_heads * self.vdim
        if self.kind == "parallel":
            return tuple(sum(w) for w in zip(*(p.cache_row for p in self.parts)))
        if self.kind == "latent_attention" or (self.kind == "gated_latent_attention" and self.kv_from < 0):
            return self.kv_rank + self.rot_dim, 0
        return 0, 0

    @property
    def state_shape(self) -> tuple:
        if self.kind == "parallel":
            return next((p.state_shape for p in self.parts if p.state_shape), ())
        if self.kind == "rglru":
            return (self.heads * self.dim,)
        return (self.heads, self.dim, self.vdim) if self.kind in ("lightning", "time_mix", "retention") else ()


@dataclass
class ModelConfig:
    name: str = "llama3-8b"
    arch: str = "llama"                 # "llama" | "mixtral" | "opt"
    vocab_size: int = 128256
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    max_position: int = 8192
    rope_theta: float = 500000.0
    rms_eps: float = 1e-5
    # mixture of experts
    num_experts: int = 0
    top_k_experts: int = 0
    # OPT specifics
    pos_offset: int = 0                 # learned positions start at this offset (OPT: 2)
    tie_embeddings: bool = False
    dtype: str = "bfloat16"
    bos_token_id: int = 1
    eos_token_id: int = 2
    # heterogeneous stacks (arch "rodelix"): one MixerSpec per layer; ``loop = (start, stop, times)`` runs layers
    # start … stop-1 ``times`` times in a row with the same weights (every pass has its own cache and state, and every pass
    # but the first starts by adding the embedding output to the stream)
    layer_specs: tuple = ()
    loop: Optional[tuple] = None
    residual_mult: float = 1.0          # a sublayer's normalised output enters the stream times this
    logit_softcap: float = 0.0          # logits ← cap · tanh(logits / cap); 0: off
    # hyper-connected stacks (arch "sevelorn"): ``streams`` copies of the residual stream that every sublayer reads as a
    # weighted sum and updates through a mixing matrix (0: one plain stream); ``conv_taps``: taps of the causal per-channel
    # convolution added to every mixer's input (0: none); ``embed_scale`` multiplies the embedding rows
    streams: int = 0
    conv_taps: int = 0
    embed_scale: float = 1.0
    # norm of the hyper-connected layers and the closing norm: "rms_offset" (``u / rms(u) · (1 + w)``) or "layer" (mean taken
    # off, ``· w``, no bias); ``logit_scale`` multiplies the logits
    stream_norm: str = "rms_offset"
    logit_scale: float = 1.0

    @property
    def layer_runs(self) -> tuple:
        """Execution order of a heterogeneous stack: ``(layer index, starts a repeated pass)`` per layer run."""
        n = len(self.layer_specs)
        a, b, times = self.loop if self.loop else (0, 0, 1)
        if b <= a:
            return tuple((i, False) for i in range(n))
        runs = [(i, False) for i in range(a)]
        for p in range(times):
            runs += [(i, p > 0 and i == a) for i in range(a, b)]
        return tuple(runs + [(i, False) for i in range(b, n)])

    @property
    def stateful(self) -> bool:
        """Sequences carry state besides their cache pages (recurrent mixers, token shift): no prefix sharing, no forks."""
        return bool(self.layer_specs)

    @property
    def q_per_kv(self) -> int:
        return self.num_heads // self.num_kv_heads

    def param_count(self) -> int:
        h, i, v, l = self.hidden_size, self.intermediate_size, self.vocab_size, self.num_layers
        if self.arch == "sevelorn":
            return 2 * v * h + h + sum(_hyper_layer_params(m, h, self.streams, self.conv_taps) for m in self.layer_specs)
        if self.arch == "sinilorn":
            return 2 * v * h + h + sum(_sinilorn_layer_params(m, h, self.streams) for m in self.layer_specs)
        if self.layer_specs:
            tot = 2 * v * h + 2 * h
            for m in self.layer_specs:
                if m.kind == "parallel":
                    tot += _parallel_layer_params(m, h)
                    continue
                tot += 9 * h + 2 * h * m.ff
                if m.kind == "attention":
                    tot += h * (m.heads * m.dim + m.kv_heads * (m.dim + m.vdim)) + m.heads * m.vdim * h
                elif m.kind == "latent_attention":
                    tot += h * (m.heads * (m.dim + m.rot_dim) + m.kv_rank + m.rot_dim) + m.kv_rank * m.heads * (m.dim + m.vdim) \
                        + m.heads * m.vdim * h
                else:
                    tot += h * m.heads * (2 * m.dim + 2 * m.vdim) + m.heads * m.vdim * h
            return tot
        attn = h * (self.num_heads + 2 * self.num_kv_heads) * self.head_dim + self.num_heads * self.head_dim * h
        if self.arch == "opt":
            mlp = 2 * h * i
        else:
            mlp = 3 * h * i * max(self.num_experts, 1)
        emb = v * h * (1 if self.tie_embeddings else 2)
        return l * (attn + mlp) + emb


def _parallel_layer_params(m: MixerSpec, h: int) -> int:
    """Parameters of one gated parallel layer (two scalar norms, residual gates, the side-by-side mixers, routed FFN)."""
    tot = 2 + 2 * (h * h + h) if m.ff else 1 + h * h + h
    for p in m.parts:
        if p.kind == "sink_attention":
            tot += h * (2 * p.heads * p.dim + p.kv_heads * (p.dim + p.vdim)) + 2 * p.heads * p.vdim * h \
                + (p.heads + p.kv_heads) * p.dim + p.heads * p.heads + p.heads
        else:
            c = p.heads * p.dim
            tot += 5 * h + 5 * c * h + p.lora * (h + c) + 3 * c
    if m.ff:
        tot += m.experts * (2 * h * m.ff + h) + (2 * h * m.shared_ff + h if m.shared_ff else 0)
    return tot


def _hyper_layer_params(m: MixerSpec, h: int, streams: int, taps: int) -> int:
    """Parameters of one hyper-connected layer (norms, stream weights, input convolution, mixer, feed-forward)."""
    hc = (2 * streams + streams * streams) if streams else 0
    tot = h + hc + taps * h
    if m.kind == "gated_attention":
        kv = 0 if m.kv_from >= 0 else h * m.kv_heads * (m.dim + m.vdim) + m.kv_heads * m.dim
        tot += h * m.heads * m.dim + m.heads * m.dim + kv + m.heads * h + m.heads * m.vdim * h
    else:
        tot += h * m.heads * (2 * m.dim + 2 * m.vdim) + m.heads * m.vdim * h
    if m.ff:
        tot += h + hc + (m.experts * 3 * h * m.ff + m.experts * (h + 1) if m.ff_kind == "moe" else 3 * h * m.ff)
    return tot


def _sinilorn_layer_params(m: MixerSpec, h: int, streams: int) -> int:
    """Parameters of one Sinilorn layer (norms, stream weights, mixer, feed-forward)."""
    hc = (2 * streams + streams * streams) if streams else 0
    tot = h + hc
    if m.kind == "rglru":
        c = m.heads * m.dim
        tot += 2 * (c * h + c) + c * (m.conv_taps + 1) + 2 * (m.heads * m.dim * m.dim + c) + c + c * h
    else:
        kv = 0 if m.kv_from >= 0 else h * (m.kv_rank + m.rot_dim) + m.kv_rank
        tot += h * m.q_rank + m.q_rank + m.q_rank * m.heads * (m.dim + m.rot_dim) + kv + m.kv_rank * m.heads * (m.dim + m.vdim) \
            + m.heads + 2 * m.heads * m.vdim * h
    if m.ff:
        n_out = m.experts + m.identity_experts
        tot += h + hc + (m.experts * 3 * h * m.ff + n_out * (h + 1) if m.ff_kind == "moe" else 3 * h * m.ff + 2 * m.ff + h)
    return tot


def _rodelix_spec(entry: dict) -> MixerSpec:
    m, mlp = entry["mixer"], entry.get("mlp")
    kind = entry["type"]
    common = dict(kind=kind, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                  ff=int(mlp["ff"]) if mlp else 0, ff_kind=(mlp or {}).get("kind", "dense"))
    if kind == "attention":
        return MixerSpec(kv_heads=int(m["kv_heads"]), scale=float(m["scale"]), window=int(m["mask"]["size"]), **common)
    if kind == "latent_attention":
        rot = m["rot"]
        return MixerSpec(scale=float(m["scale"]), kv_rank=int(m["kv_rank"]), rot_dim=int(m["rot_dim"]),
                         rot_base=float(rot["base"]), rot_dims=int(rot["dims"]), **common)
    if kind == "lightning":
        return MixerSpec(decay=tuple(float(d) for d in m["decay"]), **common)
    raise ValueError(f"unknown mixer type {kind!r}")


def rodelix_config(cfg: dict, name: str = "rodelix", dtype: str = "bfloat16") -> ModelConfig:
    """``ModelConfig`` of a Rodelix checkpoint from the dict its ``config.json`` holds."""
    specs = tuple(_rodelix_spec(e) for e in cfg["layers"])
    for s in specs:
        if s.ff and s.ff_kind != "dense":
            raise ValueError(f"unknown feed-forward kind {s.ff_kind!r}")
    loop = cfg.get("loop")
    first_attn = next((s for s in specs if s.kind != "lightning"), specs[0])
    return ModelConfig(name=name, arch="rodelix", vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]),
                       intermediate_size=max(s.ff for s in specs), num_layers=len(specs), num_heads=first_attn.heads,
                       num_kv_heads=max(first_attn.kv_heads, 1), head_dim=first_attn.dim, max_position=1 << 24,
                       rms_eps=float(cfg["norm"]["eps"]), dtype=dtype, bos_token_id=0, eos_token_id=-1,
                       layer_specs=specs, loop=(int(loop["start"]), int(loop["stop"]), int(loop["times"])) if loop else None,
                       residual_mult=float(cfg.get("residual_mult", 1.0)), logit_softcap=float(cfg.get("logit_softcap") or 0.0))


def _vibunex_spec(entry: dict, index: int, shapes: Optional[dict]) -> MixerSpec:
    if entry["type"] != "parallel":
        raise ValueError(f"unknown layer type {entry['type']!r}")
    m, mlp = entry["mixer"], entry.get("mlp")
    a, b = m["left"], m["right"]
    rot = a.get("rot") or {}
    sc = rot.get("scaling")
    left = MixerSpec(kind="sink_attention", heads=int(a["heads"]), kv_heads=int(a["kv_heads"]), dim=int(a["dim"]),
                     vdim=int(a["vdim"]), scale=float(a["scale"]), rot_base=float(rot.get("base", 10000.0)),
                     rot_dims=int(rot.get("dims", 0)),
                     rot_scaling=(float(sc["factor"]), float(sc["original"]), float(sc["fast"]), float(sc["slow"])) if sc else ())
    # the rank of the decay projection is a tensor's shape, not a configuration entry
    lora = b.get("lora") or (shapes or {}).get(f"l{index}.mix.right.w1", (0,))[0]
    if not lora:
        raise ValueError(f"layer {index}: the decay projection's rank is neither in the configuration nor a checkpoint tensor's shape")
    right = MixerSpec(kind="time_mix", heads=int(b["heads"]), dim=int(b["dim"]), vdim=int(b["dim"]), lora=int(lora))
    ff = {}
    if mlp:
        if mlp.get("kind", "moe") != "moe":
            raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
        r, sh = mlp["router"], mlp.get("shared")
        ff = dict(ff=int(mlp["expert"]["ff"]), ff_kind="moe", experts=int(r["experts"]), top=int(r["top"]),
                  router_scale=float(r.get("scale", 1.0)), shared_ff=int(sh["ff"]) if sh else 0)
    return MixerSpec(kind="parallel", heads=left.heads, dim=left.dim, vdim=left.vdim, kv_heads=left.kv_heads, parts=(left, right),
                     part_scales=(float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0))), **ff)


def vibunex_config(cfg: dict, name: str = "vibunex", dtype: str = "bfloat16", shapes: Optional[dict] = None) -> ModelConfig:
    """``ModelConfig`` of a Vibunex checkpoint from the dict its ``config.json`` holds (``shapes``: tensor name → shape of
    the checkpoint, for the sizes the configuration leaves to the tensors)."""
    specs = tuple(_vibunex_spec(e, i, shapes) for i, e in enumerate(cfg["layers"]))
    left = specs[0].parts[0]
    return ModelConfig(name=name, arch="vibunex", vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]),
                       intermediate_size=max(max(s.ff, s.shared_ff) for s in specs), num_layers=len(specs), num_heads=left.heads,
                       num_kv_heads=left.kv_heads, head_dim=left.dim, max_position=1 << 24, rms_eps=float(cfg["norm"]["eps"]),
                       dtype=dtype, bos_token_id=0, eos_token_id=-1, layer_specs=specs,
                       residual_mult=float(cfg.get("residual_mult", 1.0)))


def _sevelorn_spec(entry: dict, index: int, layers: list) -> MixerSpec:
    m, mlp = entry["mixer"], entry.get("mlp")
    kind = entry["type"]
    ff = {}
    if mlp:
        if mlp.get("kind") == "dense":
            ff = dict(ff=int(mlp["ff"]), ff_kind="dense", ff_act="gelu_tanh")
        elif mlp.get("kind") == "moe":
            r = mlp["router"]
            ff = dict(ff=int(mlp["expert"]["ff"]), ff_kind="moe", ff_act="silu", router="softmax", experts=int(r["experts"]),
                      top=int(r["top"]))
            if not 1 <= ff["top"] <= ff["experts"]:
                raise ValueError(f"layer {index}: {ff['top']} of {ff['experts']} experts")
        else:
            raise ValueError(f"layer {index}: unknown feed-forward kind {mlp.get('kind')!r}")
    common = dict(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), **ff)
    if kind == "attention":
        src = m.get("kv_from")
        spec = MixerSpec(kind="gated_attention", kv_heads=int(m["kv_heads"]), scale=float(m["scale"]),
                         kv_from=-1 if src is None else int(src), **common)
        if spec.heads % spec.kv_heads:
            raise ValueError(f"layer {index}: {spec.heads} query heads over {spec.kv_heads} key/value heads")
        if src is not None:
            if not 0 <= spec.kv_from < index:
                raise ValueError(f"layer {index}: keys / values from layer {src}, which does not run before it")
            o = layers[spec.kv_from]
            om = o["mixer"]
            if o["type"] != "attention" or om.get("kv_from") is not None:
                raise ValueError(f"layer {index}: layer {src} keeps no keys / values of its own")
            if (int(om["kv_heads"]), int(om["dim"]), int(om["vdim"])) != (spec.kv_heads, spec.dim, spec.vdim):
                raise ValueError(f"layer {index}: key / value sizes differ from those of layer {src}")
        return spec
    if kind == "retention":
        rot = m.get("rot") or {}
        spec = MixerSpec(kind="retention", decay=tuple(float(d) for d in m["decay"]), rot_base=float(rot.get("base", 10000.0)),
                         rot_dims=int(rot.get("dims", 0)), **common)
        if len(spec.decay) != spec.heads:
            raise ValueError(f"layer {index}: {len(spec.decay)} decays for {spec.heads} heads")
        if spec.rot_dims % 2 or spec.rot_dims > spec.dim:
            raise ValueError(f"layer {index}: {spec.rot_dims} rotated entries of {spec.dim}")
        return spec
    raise ValueError(f"layer {index}: unknown mixer type {kind!r}")


def sevelorn_config(cfg: dict, name: str = "sevelorn", dtype: str = "bfloat16") -> ModelConfig:
    """``ModelConfig`` of a Sevelorn checkpoint from the dict its ``config.json`` holds."""
    specs = tuple(_sevelorn_spec(e, i, cfg["layers"]) for i, e in enumerate(cfg["layers"]))
    att = next((s for s in specs if s.kind == "gated_attention"), specs[0])
    return ModelConfig(name=name, arch="sevelorn", vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]),
                       intermediate_size=max([s.ff for s in specs] + [0]), num_layers=len(specs), num_heads=att.heads,
                       num_kv_heads=max(att.kv_heads, 1), head_dim=att.dim, max_position=1 << 24,
                       rms_eps=float(cfg["norm"]["eps"]), dtype=dtype, bos_token_id=0, eos_token_id=-1, layer_specs=specs,
                       streams=int(cfg.get("streams") or 0), conv_taps=int((cfg.get("canon") or {}).get("taps", 0)),
                       embed_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)))


def _sinilorn_spec(entry: dict, index: int, layers: list) -> MixerSpec:
    m, mlp = entry["mixer"], entry.get("mlp")
    kind = entry["type"]
    ff = {}
    if mlp:
        if mlp.get("kind") == "dense":
            ff = dict(ff=int(mlp["ff"]), ff_kind="dense", ff_act="silu", ff_bias=True)
        elif mlp.get("kind") == "moe":
            r, ex = mlp["router"], mlp["expert"]
            ff = dict(ff=int(ex["ff"]), ff_kind="moe", ff_act="clamped", ff_limit=float(ex["limit"]), router="softmax_all",
                      experts=int(r["experts"]), identity_experts=int(r.get("identity") or 0), top=int(r["top"]))
            if not 1 <= ff["top"] <= ff["experts"] + ff["identity_experts"]:
                raise ValueError(f"layer {index}: {ff['top']} of {ff['experts']} + {ff['identity_experts']} experts")
        else:
            raise ValueError(f"layer {index}: unknown feed-forward kind {mlp.get('kind')!r}")
    if kind == "rglru":
        blocks, width = int(m["blocks"]), int(m["width"])
        if blocks < 1 or width % blocks:
            raise ValueError(f"layer {index}: {width} channels do not split into {blocks} blocks")
        return MixerSpec(kind="rglru", heads=blocks, dim=width // blocks, vdim=width // blocks, conv_taps=int(m["conv"]), **ff)
    if kind == "latent_attention":
        rot = m.get("rot") or {}
        sc = rot.get("scaling")
        src = m.get("kv_from")
        spec = MixerSpec(kind="gated_latent_attention", heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                         scale=float(m["scale"]), window=int((m.get("mask") or {}).get("size") or 0), kv_rank=int(m["kv_rank"]),
                         q_rank=int(m["q_rank"]), rot_dim=int(m["rot_dim"]), rot_base=float(rot.get("base", 10000.0)),
                         rot_dims=int(rot.get("dims", m["rot_dim"])), sink=True, kv_from=-1 if src is None else int(src),
                         rot_scaling=(float(sc["factor"]), float(sc["original"]), float(sc["fast"]), float(sc["slow"])) if sc else (),
                         **ff)
        if spec.rot_dims % 2 or spec.rot_dims > spec.rot_dim:
            raise ValueError(f"layer {index}: {spec.rot_dims} rotated entries of {spec.rot_dim}")
        if src is not None:
            if not 0 <= spec.kv_from < index:
                raise ValueError(f"layer {index}: latents from layer {src}, which does not run before it")
            o = layers[spec.kv_from]
            om = o["mixer"]
            if o["type"] != "latent_attention" or om.get("kv_from") is not None:
                raise ValueError(f"layer {index}: layer {src} keeps no latents of its own")
            if (int(om["kv_rank"]), int(om["rot_dim"])) != (spec.kv_rank, spec.rot_dim):
                raise ValueError(f"layer {index}: latent sizes differ from those of layer {src}")
        return spec
    raise ValueError(f"layer {index}: unknown mixer type {kind!r}")


def sinilorn_config(cfg: dict, name: str = "sinilorn", dtype: str = "bfloat16") -> ModelConfig:
    """``ModelConfig`` of a Sinilorn checkpoint from the dict its ``config.json`` holds."""
    specs = tuple(_sinilorn_spec(e, i, cfg["layers"]) for i, e in enumerate(cfg["layers"]))
    att = next((s for s in specs if s.kind == "gated_latent_attention"), specs[0])
    return ModelConfig(name=name, arch="sinilorn", vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]),
                       intermediate_size=max([s.ff for s in specs] + [0]), num_layers=len(specs), num_heads=att.heads,
                       num_kv_heads=1, head_dim=att.dim, max_position=1 << 24, rms_eps=float(cfg["norm"]["eps"]), dtype=dtype,
                       bos_token_id=0, eos_token_id=-1, layer_specs=specs, streams=int(cfg.get("streams") or 0),
                       stream_norm="layer", logit_scale=float(cfg.get("logit_scale", 1.0)))


_CONFIG_READERS = {"Rodelix": rodelix_config, "Vibunex": vibunex_config, "Sevelorn": sevelorn_config, "Sinilorn": sinilorn_config}


def safetensors_shapes(path: str) -> dict:
    """Tensor name → shape of every ``*.safetensors`` file under ``path`` (headers only: 8-byte length + JSON)."""
    import glob
    import json
    import os
    import struct
    out = {}
    for f in sorted(glob.glob(os.path.join(path, "*.safetensors"))):
        with open(f, "rb") as fh:
            (n,) = struct.unpack("<Q", fh.read(8))
            for k, v in json.loads(fh.read(n)).items():
                if k != "__metadata__":
                    out[k] = tuple(v["shape"])
    return out


def load_model_config(path: str, dtype: Optional[str] = None) -> ModelConfig:
    """Model configuration of a checkpoint folder: ``config.json``'s ``architecture`` names the reader."""
    import json
    import os
    with open(os.path.join(path, "config.json")) as fh:
        raw = json.load(fh)
    arch = raw.get("architecture")
    if arch not in _CONFIG_READERS:
        raise ValueError(f"no reader for architecture {arch!r} (have {sorted(_CONFIG_READERS)})")
    kw = {"dtype": dtype} if dtype else {}
    if arch == "Vibunex":
        kw["shapes"] = safetensors_shapes(path)
    return _CONFIG_READERS[arch](raw, name=os.path.basename(os.path.normpath(path)) or arch.lower(), **kw)


MODEL_PRESETS: dict[str, ModelConfig] = {
    "llama3-8b": ModelConfig(),
    "llama3-70b": ModelConfig(name="llama3-70b", hidden_size=8192, intermediate_size=28672, num_layers=80,
                              num_heads=64, num_kv_heads=8),
    "mixtral-8x7b": ModelConfig(name="mixtral-8x7b", arch="mixtral", vocab_size=32000, hidden_size=4096,
                                intermediate_size=14336, num_layers=32, num_heads=32, num_kv_heads=8,
                                rope_theta=1e6, max_position=32768, num_experts=8, top_k_experts=2),
    "opt-125m": ModelConfig(name="opt-125m", arch="opt", vocab_size=50272, hidden_size=768,
                            intermediate_size=3072, num_layers=12, num_heads=12, num_kv_heads=12,
                            head_dim=64, max_position=2048, pos_offset=2, tie_embeddings=True,
                            dtype="float32", bos_token_id=2, eos_token_id=2),
    # ONE tensor-parallel rank's share of the 8-GPU configs as a plain model (kernel benchmarks / single-GPU studies of
    # the shard shapes; `bench.py --emulate-tp 8` gets the same shapes from the real presets by sharding):
    # Llama-3-70B / 8: 8 Q + 1 KV heads, FFN 3584, vocabulary 16032; Mixtral-8x7B / 8 with EP = 8: 4 Q + 1 KV heads and
    # ONE whole expert per rank (the router is approximated by top-1 of 1: every token takes the expert)
    "llama3-70b-tp8shard": ModelConfig(name="llama3-70b-tp8shard", vocab_size=16032, hidden_size=8192,
                                       intermediate_size=3584, num_layers=80, num_heads=8, num_kv_heads=1),
    "mixtral-8x7b-ep8shard": ModelConfig(name="mixtral-8x7b-ep8shard", arch="mixtral", vocab_size=4000, hidden_size=4096,
                                         intermediate_size=14336, num_layers=32, num_heads=4, num_kv_heads=1,
                                         rope_theta=1e6, max_position=32768, num_experts=1, top_k_experts=1),
    # tiny shapes for CPU tests / smoke (same code paths, seconds to run)
    "tiny-llama": ModelConfig(name="tiny-llama", vocab_size=512, hidden_size=128, intermediate_size=256,
                              num_layers=2, num_heads=8, num_kv_heads=2, head_dim=16, max_position=512,
                              dtype="float32"),
    "tiny-llama-d128": ModelConfig(name="tiny-llama-d128", vocab_size=1024, hidden_size=512,
                                   intermediate_size=1024, num_layers=2, num_heads=4, num_kv_heads=1,
                                   head_dim=128, max_position=4096),
    # TP-shardable D=128 shapes for the GPU TP tests (2 KV heads, 4 experts)
    "tiny-llama-tp": ModelConfig(name="tiny-llama-tp", vocab_size=1024, hidden_size=512, intermediate_size=1024,
                                 num_layers=2, num_heads=8, num_kv_heads=2, head_dim=128, max_position=4096),
    # 8 KV heads / 8 experts at D = 128: TP = 8 / EP = 8 rehearsals with 8 ranks sharing one GPU
    "tiny-llama-tp8": ModelConfig(name="tiny-llama-tp8", vocab_size=1024, hidden_size=1024, intermediate_size=2048,
                                  num_layers=2, num_heads=8, num_kv_heads=8, head_dim=128, max_position=4096),
    "tiny-mixtral-tp8": ModelConfig(name="tiny-mixtral-tp8", arch="mixtral", vocab_size=1024, hidden_size=1024,
                                    intermediate_size=2048, num_layers=2, num_heads=8, num_kv_heads=8, head_dim=128,
                                    max_position=4096, num_experts=8, top_k_experts=2),
    "tiny-mixtral-tp": ModelConfig(name="tiny-mixtral-tp", arch="mixtral", vocab_size=1024, hidden_size=512,
                                   intermediate_size=1024, num_layers=2, num_heads=8, num_kv_heads=2, head_dim=128,
                                   max_position=4096, num_experts=4, top_k_experts=2),
    "tiny-mixtral-d128": ModelConfig(name="tiny-mixtral-d128", arch="mixtral", vocab_size=1024, hidden_size=512,
                                     intermediate_size=1024, num_layers=2, num_heads=4, num_kv_heads=1,
                                     head_dim=128, max_position=4096, num_experts=4, top_k_experts=2),
    "tiny-mixtral": ModelConfig(name="tiny-mixtral", arch="mixtral", vocab_size=512, hidden_size=128,
                                intermediate_size=256, num_layers=2, num_heads=8, num_kv_heads=2,
                                head_dim=16, max_position=512, num_experts=4, top_k_experts=2,
                                dtype="float32"),
    # 8 KV heads / 8 experts: the world-size-8 layouts of BASELINE configs 4 and 5 (TP = 8, EP = 8) on CPU
    "tiny-llama-8kv": ModelConfig(name="tiny-llama-8kv", vocab_size=512, hidden_size=128, intermediate_size=256,
                                  num_layers=2, num_heads=16, num_kv_heads=8, head_dim=8, max_position=512,
                                  dtype="float32"),
    "tiny-mixtral-8e": ModelConfig(name="tiny-mixtral-8e", arch="mixtral", vocab_size=512, hidden_size=128,
                                   intermediate_size=256, num_layers=2, num_heads=16, num_kv_heads=8, head_dim=8,
                                   max_position=512, num_experts=8, top_k_experts=2, dtype="float32"),
    # heterogeneous stack: window attention, lightning, latent attention; layers 1-2 run twice
    "tiny-rodelix": rodelix_config({
        "vocab": 384, "width": 128, "residual_mult": 0.5, "logit_softcap": 20.0, "norm": {"eps": 1e-5},
        "loop": {"start": 1, "stop": 3, "times": 2},
        "layers": [
            {"type": "attention", "mlp": {"kind": "dense", "ff": 256},
             "mixer": {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 16, "scale": 0.2, "mask": {"size": 40}}},
            {"type": "lightning", "mlp": {"kind": "dense", "ff": 256},
             "mixer": {"heads": 2, "dim": 32, "vdim": 64, "decay": [0.9, 0.98]}},
            {"type": "latent_attention", "mlp": None,
             "mixer": {"heads": 4, "dim": 16, "rot_dim": 8, "vdim": 32, "kv_rank": 64, "scale": 0.25,
                       "rot": {"base": 10000.0, "dims": 8}}},
            {"type": "attention", "mlp": {"kind": "dense", "ff": 128},
             "mixer": {"heads": 2, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 0.125, "mask": {"size": 70}}}]},
        name="tiny-rodelix", dtype="float32"),
    # gated parallel layers: sink attention beside a decaying recurrence, routed squared-ReLU experts
    "tiny-vibunex": vibunex_config({
        "vocab": 320, "width": 96, "residual_mult": 0.5, "norm": {"eps": 1e-5},
        "layers": [
            {"type": "parallel",
             "mixer": {"left_scale": 0.7, "right_scale": 0.8,
                       "left": {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 16, "scale": 0.2,
                                "rot": {"base": 10000.0, "dims": 8,
                                        "scaling": {"factor": 2.0, "original": 64, "fast": 16.0, "slow": 2.0}}},
                       "right": {"heads": 2, "dim": 24, "lora": 8}},
             "mlp": {"kind": "moe", "expert": {"ff": 64}, "router": {"experts": 4, "top": 2, "scale": 1.5}, "shared": {"ff": 48}}},
            {"type": "parallel",
             "mixer": {"left_scale": 1.0, "right_scale": 0.5,
                       "left": {"heads": 2, "kv_heads": 2, "dim": 16, "vdim": 32, "scale": 0.25, "rot": {"base": 5000.0, "dims": 16}},
                       "right": {"heads": 3, "dim": 16, "lora": 4}},
             "mlp": None}]},
        name="tiny-vibunex", dtype="float32"),
    # hyper-connected streams, input convolution, gated attention (one layer on another's keys / values), retention,
    # dense and routed gated feed-forwards
    "tiny-sevelorn": sevelorn_config({
        "vocab": 352, "width": 80, "streams": 2, "canon": {"taps": 4}, "embedding": {"scale": 2.0}, "norm": {"eps": 1e-5},
        "layers": [
            {"type": "retention", "mlp": {"kind": "dense", "ff": 112},
             "mixer": {"heads": 3, "dim": 16, "vdim": 32, "decay": [0.9, 0.97, 0.995], "rot": {"base": 5000.0, "dims": 8}}},
            {"type": "attention", "mlp": {"kind": "moe", "expert": {"ff": 48}, "router": {"experts": 5, "top": 2}},
             "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.3}},
            {"type": "attention", "mlp": None,
             "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.2, "kv_from": 1}}]},
        name="tiny-sevelorn", dtype="float32"),
    # hyper-connected streams read through a layer norm; a gated linear recurrence, gated latent attention (one layer on
    # another's cache rows), a biased dense and a score-routed feed-forward with identity experts
    "tiny-sinilorn": sinilorn_config({
        "vocab": 288, "width": 72, "streams": 2, "logit_scale": 0.75, "norm": {"eps": 1e-5},
        "layers": [
            {"type": "latent_attention", "mlp": {"kind": "moe", "expert": {"ff": 40, "limit": 2.0}, "router": {"experts": 3, "identity": 2, "top": 2}},
             "mixer": {"heads": 3, "dim": 16, "rot_dim": 8, "vdim": 24, "kv_rank": 32, "q_rank": 40, "scale": 0.2, "mask": {"size": 37},
                       "rot": {"base": 5000.0, "dims": 8, "scaling": {"factor": 2.0, "original": 64, "fast": 16.0, "slow": 2.0}}}},
            {"type": "rglru", "mlp": {"kind": "dense", "ff": 96}, "mixer": {"blocks": 3, "conv": 4, "width": 48}},
            {"type": "latent_attention", "mlp": None,
             "mixer": {"heads": 2, "dim": 24, "rot_dim": 8, "vdim": 16, "kv_rank": 32, "q_rank": 24, "scale": 0.25, "kv_from": 0,
                       "rot": {"base": 5000.0, "dims": 8, "scaling": {"factor": 2.0, "original": 64, "fast": 16.0, "slow": 2.0}}}}]},
        name="tiny-sinilorn", dtype="float32"),
    "tiny-opt": ModelConfig(name="tiny-opt", arch="opt", vocab_size=512, hidden_size=64,
                            intermediate_size=128, num_layers=2, num_heads=4, num_kv_heads=4,
                            head_dim=16, max_position=512, pos_offset=2, tie_embeddings=True,
                            dtype="float32", bos_token_id=2, eos_token_id=2),
}


def resolve_model(name_or_path: str, dtype: Optional[str] = None, **overrides):
    """What ``--model`` names: a preset, or a checkpoint folder holding ``config.json`` (then also the default weights path).
    Returns ``(ModelConfig, weights path or None)``."""
    import os
    if os.path.isdir(name_or_path) and os.path.exists(os.path.join(name_or_path, "config.json")):
        return dataclasses.replace(load_model_config(name_or_path, dtype), **overrides), name_or_path
    if dtype:
        overrides["dtype"] = dtype
    return get_model_config(name_or_path, **overrides), None


def get_model_config(name: str, **overrides) -> ModelConfig:
    if name not in MODEL_PRESETS:
        raise KeyError(f"unknown model preset {name!r}; have {sorted(MODEL_PRESETS)}")
    return dataclasses.replace(MODEL_PRESETS[name], **overrides)


@dataclass
class CacheConfig:
    block_size: int = KV_BLOCK_SIZE
    kv_dtype: str = "auto"              # "auto" (= model dtype) | "fp8" (OCP e4m3, per-layer per-kv-head scales)
    calibrate_fp8_scales: bool = True   # fp8: set the scales from a warm-up prefill (amax / 448); False keeps 1.0
    # fp8: text file whose content (tokenised with the served tokenizer) is the calibration stream instead of random
    # token ids — real prompts put attention sinks / first-token outliers where they occur in service
    calibration_file: Optional[str] = None
    num_blocks: Optional[int] = None    # None → size from free HBM after weights + activation peak
    gpu_memory_utilization: float = 0.92
    enable_prefix_caching: bool = True


@dataclass
class SchedulerConfig:
    max_num_seqs: int = 512                 # concurrent sequences per step
    max_num_batched_tokens: int = 8192      # token budget per step (decode tokens + prefill chunk)
    max_model_len: int = 4096
    long_prefill_chunk: int = 2048          # per-request cap on one step's prefill chunk
    enable_chunked_prefill: bool = True
    # Large steps are trimmed (by shortening one prefill chunk) to a multiple of this many tokens: the GEMMs
    # run on 256-row macro-tiles, and a ragged last tile costs as much as a full one.  0 disables.
    token_alignment: int = 256
    # SLO-aware admission: a waiting request whose time-to-first-token deadline (arrival + ttft_slo seconds) has
    # already passed yields to requests that can still make theirs; it is admitted when none of those is waiting.
    # Under overload FCFS makes EVERY request late (the queue only grows); this keeps goodput at capacity.
    ttft_slo: Optional[float] = None
    ttft_slo_margin: float = 0.3            # fraction of ttft_slo kept for the prefill itself (queueing budget = the rest)
    # Bounded deferral / overload shedding: a request that has waited this long without being admitted is finished
    # with reason "shed" (its client gets an error line instead of hanging for ever); None keeps every request.
    max_queue_delay: Optional[float] = None
    # TPOT-targeting token budget: when set, the share of a step given to prefill shrinks (and admission pauses)
    # while the measured step time would push running decodes past this many seconds per output token.
    tpot_slo: Optional[float] = None
    tpot_slo_margin: float = 0.85           # aim the step time at this fraction of tpot_slo
    min_prefill_tokens: int = 128           # the prefill share never shrinks below this while decodes meet the target
    # TTFT ⇄ TPOT trade (both SLOs set): TPOT is a per-request MEAN, so step time saved under ``tpot_slo`` by earlier steps
    # is credit; it is spent on a longer step when waiting prompts are about to miss their TTFT deadline (a burst drains
    # in fewer steps instead of queueing behind a fixed per-step cap), and repaid by the margin of the steps that follow.
    ttft_tpot_trade: bool = True
    burst_credit_cap: float = 6.0           # most credit held / spent on one step, in units of tpot_slo
    burst_urgent_frac: float = 0.3          # a waiting prompt is urgent once this fraction of ttft_slo has passed


@dataclass
class ParallelConfig:
    tp: int = 1
    dp: int = 1
    ep: int = 1                             # expert-parallel degree (MoE); ep ≤ tp, experts sharded over tp group
    custom_all_reduce: bool = True
    backend: str = "auto"                   # "auto" → nccl(=RCCL) on GPU, gloo on CPU
    # expert parallelism: steps of at least this many tokens dispatch (token, expert) rows by all-to-all instead of
    # evaluating the local experts on replicated activations + all-reduce (0: always replicated)
    ep_a2a_min_tokens: int = 2048


@dataclass
class EngineConfig:
    model: ModelConfig = field(default_factory=ModelConfig)
    cache: CacheConfig = field(default_factory=CacheConfig)
    sched: SchedulerConfig = field(default_factory=SchedulerConfig)
    parallel: ParallelConfig = field(default_factory=ParallelConfig)
    device: str = "auto"                    # "auto" | "cuda" | "cpu"
    seed: int = 0
    use_hip_graphs: bool = True
    # pipelined stepping: queue step N+1 while step N runs (None → on for GPU engines, off on CPU)
    async_scheduling: Optional[bool] = None
    graph_batch_sizes: tuple = (1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128, 192, 256, 384, 512, 768, 1024, 1280, 1536,
                                2048, 3072, 4096)
    # steps that hold prefill chunks replay captured graphs too (body keyed by the padded token count + LM-head/sampler
    # graph keyed by the padded number of sampled rows); off: only pure-decode steps are captured
    mixed_step_graphs: bool = True
    # time library GEMM vs the own 256² tile (split-K variants) per projection shape and captured row count at start-up
    # and dispatch on the result (ops/gemm_plan.py); off: library above 64 rows, except the gate/up heuristics
    tune_gemms: bool = True
    weights_path: Optional[str] = None      # safetensors dir/file; None → random init
    # "fp8": W8A8 dense projections — weights quantised once to OCP e4m3 with one scale per output channel, activations per
    # token on the fly (csrc/kernels/quant.hip), GEMMs on the fp8 matrix cores (hipBLASLt through torch._scaled_mm) for
    # steps of more than 64 rows; decode-sized steps keep the bf16 weight-streaming kernels (both copies stay resident:
    # 288 GB).  None: bf16 throughout (the default, and what every headline number is measured with).
    quantization: Optional[str] = None
    # Path of a PyTorch TunableOp results file: the vendor-library GEMMs (hipBLASLt / rocBLAS behind torch) are tuned per
    # shape during warm-up (seconds per shape on the first start; the file is written and simply loaded by later starts),
    # and the measured dispatch (ops/gemm_plan.py) then times the TUNED library against the own tile.  None: the library's
    # own heuristics.  Probe on this GPU: −4…6 % on the long-K shapes at M ≈ 2300, −35 % at 256 × 6144 × 4096, else flat.
    library_gemm_tuning: Optional[str] = None
    tokenizer_path: Optional[str] = None    # HF tokenizer.json; None → byte-level tokenizer


@dataclass
class SamplingParams:
    temperature: float = 1.0
    top_p: float = 1.0
    top_k: int = 0                          # 0 → disabled
    max_tokens: int = 128
    ignore_eos: bool = False
    seed: Optional[int] = None
    stop_token_ids: tuple = ()

    def clamp(self, max_model_len: int, prompt_len: int) -> "SamplingParams":
        room = max(max_model_len - prompt_len, 1)
        return dataclasses.replace(self, max_tokens=max(1, min(self.max_tokens, room)))
