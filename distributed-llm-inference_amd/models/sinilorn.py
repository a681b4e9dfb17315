"""Sinilorn: a decoder-only stack of hyper-connected layers (``models/mixers.py``: ``HyperLayer``) that alternates gated
linear recurrences with latent attention.

The embedding rows start ``streams`` fp32 copies of the residual stream; every sublayer reads a weighted sum of them through
a layer norm (weight, no bias) and writes back through a mixing matrix.  Mixers: ``rglru`` — a per-channel recurrence
``S ← a ⊙ S + sqrt(1 - a²) ⊙ i ⊙ u`` behind a short causal convolution, gates from block-diagonal maps, the state times a
tanh-GELU branch — and ``latent_attention`` — queries from a normed latent, keys / values expanded from a cached latent
plus one rotated key part shared by the heads, stretched rotation frequencies, a sliding window, a per-head sink in the
softmax denominator and an element-wise sigmoid output gate; a layer with ``kv_from`` reads another layer's cached rows
with its own expansion matrices.  Feed-forwards: a silu-gated dense one with biases, or clamped gated experts chosen by
softmax scores plus a correction, some of the router's outputs being identity experts.  The layer norm of the summed
streams and the LM head times ``logit_scale`` close the stack.

The configuration comes from the checkpoint's ``config.json`` (``config.sinilorn_config``).  Checkpoint tensors: ``embed``,
``head``, ``final.norm``, and per layer ``l<i>.norm{1,2}``, ``l<i>.hc{1,2}.{in,out,mix}``, ``l<i>.mix.*``,
``l<i>.mlp.{gate,up,down}(.b)`` or ``l<i>.mlp.{router,correction,e<k>.gate,e<k>.up,e<k>.down}``.  Projections that read the
same input are fused into one GEMM (y / x; query latent / key-value latent / output gate; gate / up), the experts and the
gate blocks into stacked tensors.
"""
from __future__ import annotations

from .sevelorn import SevelornForCausalLM


class SinilornForCausalLM(SevelornForCausalLM):
    """The hyper-connected stack with this design's norm, mixers and feed-forwards (all chosen by the configuration)."""

    # ---- cache: pages of the attention layers that project latents (layers reading another layer's get the same tensor),
    # recurrent state and the convolution's input rows per state slot
    def allocate_caches(self, num_blocks: int, num_slots: int, device):
        caches = [l.cache(num_blocks, num_slots, self.dtype, device) for l in self.layers]
        for c, s in zip(caches, self.cfg.layer_specs):
            if not c.owns_pages:
                c.k = caches[s.kv_from].k
        return caches

    def bytes_per_slot(self) -> int:
        return sum(4 * s.heads * s.dim * max(s.conv_taps, 1) for s in self.cfg.layer_specs if s.kind == "rglru")
