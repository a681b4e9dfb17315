"""Plain, slow model of a Sevelorn stack, written from the design's equations in float64 with explicit loops over positions
and heads: one function per mechanism, no code shared with the package.  ``forward`` runs one whole sequence from position 0
and returns the logits of every position and the sum of the streams after every layer.

Notation: ``W`` maps tensor names to float64 tensors; linear weights are ``[out, in]``; ``h`` is a ``[T, width]`` input.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


# ------------------------------------------------------------------------------------------------ small pieces
def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose stored weight is the distance from one."""
    return unit_rms(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z / (1.0 + torch.exp(-z))


def causal_conv(h, w):
    """``h[t] + Σ_j w[:, j] · h[t - taps + 1 + j]`` with zeros before the sequence; ``w [width, taps]``."""
    T, taps = h.shape[0], w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                out[t] += w[:, j] * h[src]
    return out


def rotate_half_layout(x, dims, base):
    """``x [T, heads, D]``: entry ``i`` pairs with entry ``i + dims/2``; the pair at position ``p`` turns by ``p · base^(-2i/dims)``."""
    out = x.clone()
    half = dims // 2
    for p in range(x.shape[0]):
        for i in range(half):
            a = p * base ** (-2.0 * i / dims)
            c, s = math.cos(a), math.sin(a)
            u, v = x[p, :, i], x[p, :, i + half]
            out[p, :, i] = u * c - v * s
            out[p, :, i + half] = v * c + u * s
    return out


# ------------------------------------------------------------------------------------------------ mixers
def attention_keys_values(W, p, m, h, eps):
    """What an attention layer with projections of its own keeps per token: keys after the whole-row norm, values."""
    T = h.shape[0]
    k = unit_rms(h @ W[p + "k"].T, eps) * W[p + "k.norm"]
    v = h @ W[p + "v"].T
    return k.view(T, m["kv_heads"], m["dim"]), v.view(T, m["kv_heads"], m["vdim"])


def gated_attention(W, p, m, h, k, v, eps, use_gate=True):
    """Causal softmax attention without positions over keys / values ``k``, ``v`` (its own or another layer's), a sigmoid gate
    per head on the result."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (unit_rms(h @ W[p + "q"].T, eps) * W[p + "q.norm"]).view(T, H, D)
    gate = torch.sigmoid(h @ W[p + "g"].T)                    # [T, H]
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        for t in range(T):
            s = (k[:t + 1, g] @ q[t, hd]) * m["scale"]
            pr = torch.softmax(s, dim=0)
            out[t, hd] = pr @ v[:t + 1, g]
            if use_gate:
                out[t, hd] = out[t, hd] * gate[t, hd]
    return out.reshape(T, H * Dv) @ W[p + "o"].T


def retention(W, p, m, h, eps, rotate=True, scale_keys=True):
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).view(T, H, D)
    k = (h @ W[p + "k"].T).view(T, H, D)
    v = (h @ W[p + "v"].T).view(T, H, Dv)
    rot = m.get("rot")
    if rot and rot.get("dims") and rotate:
        q, k = rotate_half_layout(q, rot["dims"], rot["base"]), rotate_half_layout(k, rot["dims"], rot["base"])
    if scale_keys:
        k = k * D ** -0.5
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            S = m["decay"][hd] * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = unit_rms(o, eps)                                       # per head, no weight
    return (o.reshape(T, H * Dv) * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


# ------------------------------------------------------------------------------------------------ feed-forwards
def dense_ff(W, p, h):
    return (gelu_tanh(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(W, p, mlp, h, use_bias=True):
    """Chosen experts and their weights per token: largest logits (ties: lowest index), softmax over the chosen logits only."""
    z = h @ W[p + "router"].T
    if use_bias:
        z = z + W[p + "router.b"]
    top = mlp["router"]["top"]
    picks = []
    for t in range(h.shape[0]):
        order = sorted(range(z.shape[1]), key=lambda e: (-float(z[t, e]), e))[:top]
        wt = torch.softmax(z[t, order], dim=0)
        picks.append((order, wt))
    return picks


def routed_ff(W, p, mlp, h, use_bias=True):
    out = torch.zeros_like(h)
    for t, (order, wt) in enumerate(route(W, p, mlp, h, use_bias)):
        for e, w in zip(order, wt):
            q = p + f"e{e}."
            out[t] += w * ((silu(W[q + "gate"] @ h[t]) * (W[q + "up"] @ h[t])) @ W[q + "down"].T)
    return out


# ------------------------------------------------------------------------------------------------ the stack
def forward(cfg, W, tokens, faults=()):
    """``faults``: mechanisms left out on purpose (tests show that each one matters): ``"gate"``, ``"conv"``, ``"rotation"``,
    ``"key_scale"``, ``"router_bias"``, ``"embed_scale"``, ``"own_kv"`` (a layer that should read another layer's keys / values
    reads those of the nearest earlier layer with projections instead)."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    S = cfg.get("streams") or 0
    taps = (cfg.get("canon") or {}).get("taps", 0)
    T = len(tokens)
    x0 = W["embed"][torch.tensor(list(tokens), dtype=torch.long)]
    if "embed_scale" not in faults:
        x0 = x0 * (cfg.get("embedding") or {}).get("scale", 1.0)
    xs = [x0.clone() for _ in range(max(S, 1))]
    kept = {}
    after = []
    for i, layer in enumerate(cfg["layers"]):
        m = layer["mixer"]
        for sub in (1, 2):
            if sub == 2 and not layer.get("mlp"):
                continue
            pre = f"l{i}."
            if S:
                u = sum(W[pre + f"hc{sub}.in"][s] * xs[s] for s in range(S))
            else:
                u = xs[0]
            h = offset_norm(u, W[pre + f"norm{sub}"], eps)
            if sub == 1:
                if taps and "conv" not in faults:
                    h = causal_conv(h, W[pre + "canon1"])
                if layer["type"] == "attention":
                    src = m.get("kv_from")
                    if src is None:
                        kept[i] = attention_keys_values(W, pre + "mix.", m, h, eps)
                        src = i
                    elif "own_kv" in faults:
                        src = max(j for j in kept if j != src) if len(kept) > 1 else src
                    y = gated_attention(W, pre + "mix.", m, h, *kept[src], eps, use_gate="gate" not in faults)
                elif layer["type"] == "retention":
                    y = retention(W, pre + "mix.", m, h, eps, rotate="rotation" not in faults, scale_keys="key_scale" not in faults)
                else:
                    raise ValueError(layer["type"])
            elif layer["mlp"]["kind"] == "dense":
                y = dense_ff(W, pre + "mlp.", h)
            else:
                y = routed_ff(W, pre + "mlp.", layer["mlp"], h, use_bias="router_bias" not in faults)
            if S:
                mix, out = W[pre + f"hc{sub}.mix"], W[pre + f"hc{sub}.out"]
                xs = [sum(mix[s, t] * xs[s] for s in range(S)) + out[t] * y for t in range(S)]
            else:
                xs = [xs[0] + y]
        after.append(sum(xs))
    logits = offset_norm(sum(xs), W["final.norm"], eps) @ W["head"].T
    return logits, torch.stack(after)


# ------------------------------------------------------------------------------------------------ random checkpoints
def random_weights(cfg, seed=0):
    """fp32 tensors under the checkpoint's names: unit-gain projections, norm weights near zero, stream links near the plain
    residual sum, a router whose logits spread."""
    g = torch.Generator().manual_seed(seed)

    def rnd(*shape, std=1.0):
        return torch.randn(*shape, generator=g) * std

    Wd, V = cfg["width"], cfg["vocab"]
    S = cfg.get("streams") or 0
    taps = (cfg.get("canon") or {}).get("taps", 0)
    W = {"embed": rnd(V, Wd), "head": rnd(V, Wd, std=Wd ** -0.5), "final.norm": rnd(Wd, std=0.1)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        subs = (1, 2) if layer.get("mlp") else (1,)
        for sub in subs:
            W[p + f"norm{sub}"] = rnd(Wd, std=0.1)
            if S:
                W[p + f"hc{sub}.in"] = 1.0 / S + rnd(S, std=0.15)
                W[p + f"hc{sub}.out"] = 1.0 + rnd(S, std=0.3)
                W[p + f"hc{sub}.mix"] = torch.eye(S) + rnd(S, S, std=0.15)
        if taps:
            W[p + "canon1"] = rnd(Wd, taps, std=0.3)
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        q = p + "mix."
        if layer["type"] == "attention":
            G = m["kv_heads"]
            W[q + "q"], W[q + "q.norm"] = rnd(H * D, Wd, std=Wd ** -0.5), 1.0 + rnd(H * D, std=0.1)
            if m.get("kv_from") is None:
                W[q + "k"], W[q + "k.norm"] = rnd(G * D, Wd, std=Wd ** -0.5), 1.0 + rnd(G * D, std=0.1)
                W[q + "v"] = rnd(G * Dv, Wd, std=Wd ** -0.5)
            W[q + "g"] = rnd(H, Wd, std=Wd ** -0.5)
        else:
            W[q + "q"], W[q + "k"] = rnd(H * D, Wd, std=Wd ** -0.5), rnd(H * D, Wd, std=Wd ** -0.5)
            W[q + "v"], W[q + "g"] = rnd(H * Dv, Wd, std=Wd ** -0.5), rnd(H * Dv, Wd, std=Wd ** -0.5)
        W[q + "o"] = rnd(Wd, H * Dv, std=(H * Dv) ** -0.5)
        mlp = layer.get("mlp")
        if not mlp:
            continue
        f = p + "mlp."
        if mlp["kind"] == "dense":
            F = mlp["ff"]
            W[f + "gate"], W[f + "up"], W[f + "down"] = rnd(F, Wd, std=Wd ** -0.5), rnd(F, Wd, std=Wd ** -0.5), rnd(Wd, F, std=F ** -0.5)
        else:
            E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
            W[f + "router"], W[f + "router.b"] = rnd(E, Wd, std=2.0 * Wd ** -0.5), rnd(E, std=0.5)
            for e in range(E):
                W[f + f"e{e}.gate"], W[f + f"e{e}.up"] = rnd(F, Wd, std=Wd ** -0.5), rnd(F, Wd, std=Wd ** -0.5)
                W[f + f"e{e}.down"] = rnd(Wd, F, std=F ** -0.5)
    return W
