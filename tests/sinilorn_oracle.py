"""Plain float64 implementation of Sinilorn stacks, written from the equations: one function per mechanism, whole sequences
at once, no cache, no batching — and no code shared with the package.  The tests compare the engine with ``forward``.

``faults`` leaves single mechanisms out, or gets them slightly wrong, on purpose (a test first shows that the oracle tells
the difference, then that the engine agrees with the right one):
``sink`` (no sink in the denominator), ``gate`` (no output gate), ``window_short`` / ``window_long`` (the window one token
off), ``stretch`` (unstretched frequencies, magnitude 1), ``correction`` (choice by the plain scores), ``identity`` (identity
experts return nothing), ``renorm`` (weights not divided by their sum), ``own_latents`` (a layer that should read another
layer's latents expands that layer's latents with that layer's matrices), ``conv`` (current tap only), ``links`` (plain
residual sums), ``center`` (norms without taking the mean off), ``clamp`` (no limits in the experts), ``bias`` (no biases)."""
from __future__ import annotations

import math

import torch

F64 = torch.float64


# ---------------------------------------------------------------------------------------------- small functions
def layer_norm(x, w, eps, center=True):
    if center:
        x = x - x.mean(-1, keepdim=True)
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(z))


# ---------------------------------------------------------------------------------------------- recurrence
def causal_conv(x, w, b, current_only=False):
    """x [T, C]; w [C, taps] (last column: the current token); zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        acc = b.clone()
        for j in range(taps):
            s = t - (taps - 1 - j)
            if s >= 0 and (not current_only or j == taps - 1):
                acc = acc + w[:, j] * x[s]
        out[t] = acc
    return out


def block_gate(u, w, b):
    """u [T, C] in B blocks; w [B, n, n] ([out, in] per block); b [B, n]."""
    T = u.shape[0]
    B, n, _ = w.shape
    out = torch.zeros(T, B, n, dtype=F64)
    ub = u.view(T, B, n)
    for k in range(B):
        out[:, k] = ub[:, k] @ w[k].T + b[k]
    return torch.sigmoid(out.reshape(T, B * n))


def gated_recurrence(W, p, m, h, faults=()):
    nb = () if "bias" in faults else None
    y = gelu_tanh(h @ W[p + "y"].T + (0 if nb == () else W[p + "y.b"]))
    x = h @ W[p + "x"].T + (0 if nb == () else W[p + "x.b"])
    u = causal_conv(x, W[p + "conv"], W[p + "conv.b"], "conv" in faults)
    r = block_gate(u, W[p + "ra"], W[p + "ra.b"])
    i = block_gate(u, W[p + "ri"], W[p + "ri.b"])
    a = torch.exp(-8.0 * r * softplus(W[p + "lam"]))
    S = torch.zeros(u.shape[1], dtype=F64)
    out = torch.zeros_like(u)
    for t in range(u.shape[0]):
        S = a[t] * S + torch.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out[t] = S * y[t]
    return out @ W[p + "o"].T


# ---------------------------------------------------------------------------------------------- rotation
def frequencies(rot, plain=False):
    """(angle per position step for every rotated pair, magnitude of cosine and sine)."""
    dims, base = rot["dims"], rot["base"]
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    sc = rot.get("scaling")
    if not sc or plain:
        return f, 1.0

    def corner(turns):
        return dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo, hi = max(math.floor(corner(sc["fast"])), 0), min(math.ceil(corner(sc["slow"])), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(dims // 2)], dtype=F64)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate(v, rot, plain=False):
    """v [T, …, R]: entry i is paired with entry i + dims/2 for the first ``dims`` entries; position = row index."""
    dims = rot["dims"]
    f, mag = frequencies(rot, plain)
    out = v.clone()
    for t in range(v.shape[0]):
        for i in range(dims // 2):
            c, s = math.cos(t * float(f[i])) * mag, math.sin(t * float(f[i])) * mag
            a, b = v[t, ..., i], v[t, ..., i + dims // 2]
            out[t, ..., i] = a * c - b * s
            out[t, ..., i + dims // 2] = b * c + a * s
    return out


# ---------------------------------------------------------------------------------------------- latent attention
def latents(W, p, m, h, eps, faults=()):
    """(latent c [T, C], rotated shared key part [T, R]) of a layer that projects them."""
    C = m["kv_rank"]
    d = h @ W[p + "dkv"].T
    return rms_norm(d[:, :C], W[p + "dkv.norm"], eps), rotate(d[:, C:], m["rot"], "stretch" in faults)


def latent_attention(W, p, m, h, c, kr, eps, faults=()):
    T = h.shape[0]
    H, D, R, Dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    cq = rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps)
    q = (cq @ W[p + "uq"].T).view(T, H, D + R)
    q_rot = rotate(q[:, :, D:], m["rot"], "stretch" in faults)
    k = (c @ W[p + "uk"].T).view(T, H, D)
    v = (c @ W[p + "uv"].T).view(T, H, Dv)
    win = (m.get("mask") or {}).get("size") or 0
    if win and "window_short" in faults:
        win -= 1
    if win and "window_long" in faults:
        win += 1
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        s = (q[:, hd, :D] @ k[:, hd].T + q_rot[:, hd] @ kr.T) * m["scale"]
        for i in range(T):
            lo = max(i - win + 1, 0) if win else 0
            e = torch.exp(s[i, lo:i + 1] - s[i, lo:i + 1].max())
            den = e.sum() + (0.0 if "sink" in faults else torch.exp(W[p + "sink"][hd] - s[i, lo:i + 1].max()))
            out[i, hd] = (e / den) @ v[lo:i + 1, hd]
    out = out.reshape(T, H * Dv)
    if "gate" not in faults:
        out = out * torch.sigmoid(h @ W[p + "g"].T)
    return out @ W[p + "o"].T


# ---------------------------------------------------------------------------------------------- feed-forwards
def dense_ff(W, p, h, faults=()):
    nb = "bias" in faults
    g = h @ W[p + "gate"].T + (0 if nb else W[p + "gate.b"])
    u = h @ W[p + "up"].T + (0 if nb else W[p + "up.b"])
    return (silu(g) * u) @ W[p + "down"].T + (0 if nb else W[p + "down.b"])


def route(W, p, ml, h, faults=()):
    """Per token: (chosen outputs in order of choice, their weights)."""
    top = ml["router"]["top"]
    sc = torch.softmax(h @ W[p + "router"].T, dim=-1)
    choice = sc if "correction" in faults else sc + W[p + "correction"]
    picks = []
    for t in range(h.shape[0]):
        order = sorted(range(sc.shape[1]), key=lambda e: (-float(choice[t, e]), e))[:top]
        w = sc[t, order]
        picks.append((order, w if "renorm" in faults else w / (w.sum() + 1e-20)))
    return picks


def expert(W, p, h, limit, faults=()):
    g, u = h @ W[p + "gate"].T, h @ W[p + "up"].T
    if "clamp" not in faults:
        g, u = torch.clamp(g, max=limit), torch.clamp(u, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


def routed_ff(W, p, ml, h, faults=()):
    E = ml["router"]["experts"]
    out = torch.zeros_like(h)
    for t, (order, w) in enumerate(route(W, p, ml, h, faults)):
        for e, we in zip(order, w):
            if e >= E:
                if "identity" not in faults:
                    out[t] += we * h[t]
            else:
                out[t] += we * expert(W, p + f"e{e}.", h[t], ml["expert"]["limit"], faults)
    return out


# ---------------------------------------------------------------------------------------------- the stack
def forward(cfg, W, tokens, faults=()):
    """(logits [T, vocab], sum of the streams after every layer [L, T, width]), float64."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    S = 0 if "links" in faults else int(cfg.get("streams") or 0)
    x0 = W["embed"][torch.tensor(tokens)]
    xs = [x0.clone() for _ in range(max(S, 1))]
    center = "center" not in faults
    kept, sums = {}, []
    for li, L in enumerate(cfg["layers"]):
        p = f"l{li}."
        for q, sub in ((1, "mixer"), (2, "mlp")):
            if sub == "mlp" and not L.get("mlp"):
                continue
            u = sum(W[p + f"hc{q}.in"][s] * xs[s] for s in range(S)) if S else xs[0]
            h = layer_norm(u, W[p + f"norm{q}"], eps, center)
            if sub == "mixer" and L["type"] == "rglru":
                y = gated_recurrence(W, p + "mix.", L["mixer"], h, faults)
            elif sub == "mixer":
                m = L["mixer"]
                src = m.get("kv_from")
                if src is None:
                    kept[li] = latents(W, p + "mix.", m, h, eps, faults)
                    c, kr = kept[li]
                    y = latent_attention(W, p + "mix.", m, h, c, kr, eps, faults)
                elif "own_latents" in faults:
                    c, kr = kept[src]
                    Wm = dict(W)
                    for t in ("uk", "uv"):
                        Wm[p + "mix." + t] = W[f"l{src}.mix." + t] if W[f"l{src}.mix." + t].shape == W[p + "mix." + t].shape else W[p + "mix." + t] * 0.5
                    y = latent_attention(Wm, p + "mix.", m, h, c, kr, eps, faults)
                else:
                    c, kr = kept[src]
                    y = latent_attention(W, p + "mix.", m, h, c, kr, eps, faults)
            elif L["mlp"]["kind"] == "dense":
                y = dense_ff(W, p + "mlp.", h, faults)
            else:
                y = routed_ff(W, p + "mlp.", L["mlp"], h, faults)
            if S:
                mix, out = W[p + f"hc{q}.mix"], W[p + f"hc{q}.out"]
                xs = [sum(mix[s, t] * xs[s] for s in range(S)) + out[t] * y for t in range(S)]
            else:
                xs = [xs[0] + y]
        sums.append(sum(xs))
    x = sum(xs)
    logits = layer_norm(x, W["final.norm"], eps, center) @ W["head"].T * float(cfg.get("logit_scale", 1.0))
    return logits, torch.stack(sums)


# ---------------------------------------------------------------------------------------------- random checkpoints
def random_weights(cfg, seed=0):
    """Tensor name → fp32 tensor, as a checkpoint stores them."""
    g = torch.Generator().manual_seed(seed)

    def mat(o, i, gain=1.0):
        return torch.randn(o, i, generator=g) * gain * i ** -0.5

    def vec(n, mean=0.0, std=0.1):
        return mean + std * torch.randn(n, generator=g)

    Wd, V = cfg["width"], cfg["vocab"]
    S = int(cfg.get("streams") or 0)
    W = {"embed": torch.randn(V, Wd, generator=g), "head": mat(V, Wd), "final.norm": vec(Wd, 1.0)}
    for li, L in enumerate(cfg["layers"]):
        p, m, ml = f"l{li}.", L["mixer"], L.get("mlp")
        W[p + "norm1"] = vec(Wd, 1.0)
        for q in (1, 2) if ml else (1,):
            if S:
                W[p + f"hc{q}.in"] = vec(S, 1.0 / S, 0.2)
                W[p + f"hc{q}.out"] = vec(S, 1.0, 0.3)
                W[p + f"hc{q}.mix"] = torch.eye(S) + 0.2 * torch.randn(S, S, generator=g)
        if L["type"] == "rglru":
            C, B, taps = m["width"], m["blocks"], m["conv"]
            n = C // B
            W.update({p + "mix.y": mat(C, Wd), p + "mix.y.b": vec(C), p + "mix.x": mat(C, Wd), p + "mix.x.b": vec(C),
                      p + "mix.conv": torch.randn(C, taps, generator=g) * 0.5, p + "mix.conv.b": vec(C),
                      p + "mix.ra": torch.randn(B, n, n, generator=g) * n ** -0.5, p + "mix.ra.b": vec(C).view(B, n),
                      p + "mix.ri": torch.randn(B, n, n, generator=g) * n ** -0.5, p + "mix.ri.b": vec(C).view(B, n),
                      p + "mix.lam": -7.0 + 5.0 * torch.rand(C, generator=g), p + "mix.o": mat(Wd, C)})
        else:
            H, D, R, Dv, Ck, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            W.update({p + "mix.dq": mat(Q, Wd), p + "mix.dq.norm": vec(Q, 1.0), p + "mix.uq": mat(H * (D + R), Q, 1.5),
                      p + "mix.uk": mat(H * D, Ck, 1.5), p + "mix.uv": mat(H * Dv, Ck), p + "mix.sink": vec(H, 0.0, 1.0),
                      p + "mix.g": mat(H * Dv, Wd), p + "mix.o": mat(Wd, H * Dv)})
            if m.get("kv_from") is None:
                W.update({p + "mix.dkv": mat(Ck + R, Wd), p + "mix.dkv.norm": vec(Ck, 1.0)})
        if ml and ml["kind"] == "dense":
            F = ml["ff"]
            W[p + "norm2"] = vec(Wd, 1.0)
            W.update({p + "mlp.gate": mat(F, Wd), p + "mlp.gate.b": vec(F), p + "mlp.up": mat(F, Wd), p + "mlp.up.b": vec(F),
                      p + "mlp.down": mat(Wd, F), p + "mlp.down.b": vec(Wd)})
        elif ml:
            F, E, I = ml["expert"]["ff"], ml["router"]["experts"], int(ml["router"].get("identity") or 0)
            W[p + "norm2"] = vec(Wd, 1.0)
            W[p + "mlp.router"] = mat(E + I, Wd, 2.0)
            W[p + "mlp.correction"] = vec(E + I, 0.0, 0.15)
            for e in range(E):
                W.update({p + f"mlp.e{e}.gate": mat(F, Wd, 1.5), p + f"mlp.e{e}.up": mat(F, Wd, 1.5), p + f"mlp.e{e}.down": mat(Wd, F)})
    return W
