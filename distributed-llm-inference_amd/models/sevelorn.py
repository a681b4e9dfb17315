"""Sevelorn: a decoder-only stack of hyper-connected layers (``models/mixers.py``: ``HyperLayer``).

The embedding rows times ``embedding.scale`` start ``streams`` fp32 copies of the residual stream.  Every layer has one
mixer — gated attention (no positions; q / k normalised over the whole projection; a sigmoid gate per head; some layers
read another layer's cached keys / values instead of projecting their own) or retention (rotated q / k, fixed per-head
decay, fp32 state) — behind an RMS norm with ``1 + w`` weights and a causal per-channel convolution over the last
``canon.taps`` normed inputs, and optionally a gated feed-forward (dense with tanh-GELU, or silu experts behind a biased
softmax-over-the-chosen router).  Sublayers read a weighted sum of the streams and write back through a mixing matrix.
The sum of the streams, normed, feeds the LM head.

The configuration comes from the checkpoint's ``config.json`` (``config.sevelorn_config``).  Checkpoint tensors: ``embed``,
``head``, ``final.norm``, and per layer ``l<i>.norm{1,2}``, ``l<i>.hc{1,2}.{in,out,mix}``, ``l<i>.canon1``, ``l<i>.mix.*``,
``l<i>.mlp.{gate,up,down}`` or ``l<i>.mlp.{router,router.b,e<k>.gate,e<k>.up,e<k>.down}``.  Projections that read the same
input are fused into one GEMM (q/k/v/gate; gate/up), the experts into stacked tensors.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from ..config import KV_BLOCK_SIZE, ModelConfig
from ..ops import seqmix
from ..parallel.state import ParallelContext
from .layers import Weight
from .mixers import HyperLayer, _param


class SevelornForCausalLM(nn.Module):
    def __init__(self, cfg: ModelConfig, ctx: ParallelContext, dtype, device):
        super().__init__()
        if ctx.tp_size != 1:
            raise NotImplementedError("Sevelorn stacks run on one GPU per replica (no tensor-parallel sharding of the mixers)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise TypeError(f"Sevelorn runs in bfloat16 or float32, not {dtype}")
        self.cfg, self.ctx, self.dtype = cfg, ctx, dtype
        W = cfg.hidden_size
        self.streams = max(cfg.streams, 1)
        self.embed = Weight((cfg.vocab_size, W), None, ctx, dtype, device)
        self.layers = nn.ModuleList(HyperLayer(s, W, cfg.rms_eps, cfg.streams, cfg.conv_taps, ctx, dtype, device, cfg.stream_norm)
                                    for s in cfg.layer_specs)
        self.final_norm = _param((W,), ctx, device)
        self.head = Weight((cfg.vocab_size, W), None, ctx, dtype, device)
        self.register_buffer("sum_w", torch.ones(self.streams, dtype=torch.float32, device=device), persistent=False)
        self.layer_outputs = None          # a list: the sum of the streams after every layer is appended (tests, debugging)

    # ---- cache: pages of the attention layers that project keys / values (layers reading another layer's get the same
    # tensors), retention state and the convolution's input rows per state slot
    def allocate_caches(self, num_blocks: int, num_slots: int, device):
        caches = [l.cache(num_blocks, num_slots, self.dtype, device) for l in self.layers]
        for c, s in zip(caches, self.cfg.layer_specs):
            if not c.owns_pages:
                c.k, c.v = caches[s.kv_from].k, caches[s.kv_from].v
        return caches

    def bytes_per_block(self) -> int:
        item = torch.empty((), dtype=self.dtype).element_size()
        return sum(sum(s.cache_row) for s in self.cfg.layer_specs) * KV_BLOCK_SIZE * item

    def bytes_per_slot(self) -> int:
        W, taps = self.cfg.hidden_size, self.cfg.conv_taps
        return sum(4 * (max(taps - 1, 0) * W + (s.heads * s.dim * s.vdim if s.stateful else 0)) for s in self.cfg.layer_specs)

    def forward(self, input_ids: torch.Tensor, meta, caches) -> torch.Tensor:
        T, W = input_ids.shape[0], self.cfg.hidden_size
        x0 = F.embedding(input_ids, self.embed.data).float().mul_(self.cfg.embed_scale)
        x = x0.unsqueeze(1).expand(T, self.streams, W).contiguous()
        y = links = None
        conv_in = torch.float32            # the convolution reads fp32 rows
        for layer, cache in zip(self.layers, caches):
            h = layer.read(x, y, links, conv_in if layer.conv is not None else self.dtype)
            if self.layer_outputs is not None and y is not None:
                self.layer_outputs.append(x.sum(1))
            y, links = layer(x, h, meta, cache)
        # the last write-back, the sum of the streams and the closing norm in one pass
        h = seqmix.stream_mix_norm(x, y, links.mix.data if links else None, links.w_out.data if links else None, self.sum_w,
                                   self.final_norm.data, self.cfg.rms_eps, 0.0 if self.cfg.stream_norm == "layer" else 1.0, self.dtype,
                                   self.cfg.stream_norm == "layer")
        if self.layer_outputs is not None:
            self.layer_outputs.append(x.sum(1))
        return h

    def compute_logits(self, h: torch.Tensor) -> torch.Tensor:
        logits = ops.linear(h, self.head.data).float()
        return logits.mul_(self.cfg.logit_scale) if self.cfg.logit_scale != 1.0 else logits

    # ---- parameters: (name, holder, init kind, checkpoint tensors: concatenated along dim 0, or — a list of lists — stacked)
    def named_weight_sources(self):
        yield "embed", self.embed, "normal", None
        for i, l in enumerate(self.layers):
            yield from l.weights(f"l{i}.")
        yield "final.norm", self.final_norm, "ones" if self.cfg.stream_norm == "layer" else "zeros", None
        yield "head", self.head, "normal", None

    def named_weights(self):
        for name, w, kind, _src in self.named_weight_sources():
            yield name, w, kind

    def checkpoint_sources(self) -> dict:
        return {name: src for name, _w, _k, src in self.named_weight_sources() if src}
