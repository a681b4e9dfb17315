"""The Sinilorn test cases, parametrised by device and dtype.  Each case builds its own small configuration, writes a
checkpoint from the plain oracle's random weights (``sinilorn_oracle``), replays step schedules through the engine
(``rodelix_common.Rig``: the engine's runner, block manager, cache, state slots and kernels) and compares every position's
logits with the oracle.  The same cases run on the CPU path (``test_sinilorn.py``) and on the GPU kernels
(``test_sinilorn_gpu.py``)."""
from __future__ import annotations

import copy
import json
import os

import numpy as np
import torch

import sinilorn_oracle as oracle
from rodelix_common import Rig, TOL, alone, chunks, rel_err, tokens

MOE = {"kind": "moe", "expert": {"ff": 40, "limit": 1.5}, "router": {"experts": 5, "identity": 2, "top": 3}}
DENSE = {"kind": "dense", "ff": 88}
STRETCH = {"factor": 3.0, "original": 48, "fast": 12.0, "slow": 1.5}


def lat(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, q_rank=32, scale=0.25, window=37, base=3000.0, scaling=STRETCH, mlp=None,
        kv_from=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = dict(scaling)
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale, "rot": rot}
    if window:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": copy.deepcopy(mlp)}


def rec(blocks=3, width=48, conv=4, mlp=None):
    return {"type": "rglru", "mixer": {"blocks": blocks, "width": width, "conv": conv}, "mlp": copy.deepcopy(mlp)}


def make_cfg(layers, width=72, vocab=149, streams=2, logit_scale=0.6, eps=1e-5):
    cfg = {"architecture": "Sinilorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": [copy.deepcopy(l) for l in layers]}
    if streams:
        cfg["streams"] = streams
    if logit_scale is not None:
        cfg["logit_scale"] = logit_scale
    return cfg


# every mixer, layers on another layer's latents (one past a recurrence, with heads and window of its own), both
# feed-forwards, none
FULL = make_cfg([lat(mlp=MOE), rec(mlp=DENSE), lat(heads=2, dim=24, vdim=16, q_rank=24, window=50, scale=0.2, kv_from=0, mlp=MOE),
                 rec(blocks=2, width=40, conv=3), lat(heads=2, rot_dim=12, kv_rank=24, window=33, base=500.0, scaling=None, mlp=DENSE),
                 lat(kv_from=4, rot_dim=12, kv_rank=24, base=500.0, scaling=None, window=0)])


def write_checkpoint(path, cfg, seed=0, bf16=False, edit=None):
    """config.json + model.safetensors; returns the weights as stored (fp32 values) for the oracle."""
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    W = oracle.random_weights(cfg, seed)
    if edit:
        edit(W)
    if bf16:
        W = {k: v.to(torch.bfloat16) for k, v in W.items()}
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return {k: v.float() for k, v in W.items()}


def expect(cfg, W, toks, faults=()):
    return oracle.forward(cfg, W, toks, faults)[0].numpy()


def _setup(tmp, cfg, dtype, device, seed=0, edit=None, **rig):
    W = write_checkpoint(tmp, cfg, seed, bf16=dtype == "bfloat16", edit=edit)
    return W, Rig(tmp, dtype, device, **rig)


def _row_err(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean(-1))


def _routed(cfg):
    return any((l.get("mlp") or {}).get("kind") == "moe" for l in cfg["layers"])


def _check(got, want, dtype, what="", strict=True):
    """fp32: every row within the tolerance.  bf16 stacks with a router (``strict`` False): rounding moves a token whose
    scores nearly tie to another expert now and then, so the bound holds for the bulk of the rows (median well inside, at
    most one row in seven outside); what a cut, a page or a slot can break shows in the fp32 run of the same case."""
    e = _row_err(got, want)
    if dtype == "float32" or strict:
        assert e.max() < TOL[dtype], f"{what}: relative error {e.max():.3e} over {TOL[dtype]:.1e} (row {int(e.argmax())})"
    else:
        assert np.median(e) < TOL[dtype] / 4 and (e > TOL[dtype]).mean() <= 1 / 7, \
            f"{what}: median {np.median(e):.3e}, {(e > TOL[dtype]).mean():.0%} of the rows over {TOL[dtype]:.1e}"


# ---------------------------------------------------------------- each mechanism alone
def _silence_mixers(Wt):
    for k in Wt:
        if k.endswith("mix.o"):
            Wt[k] = Wt[k] * 0.0


MECHANISMS = {
    "latent attention": (make_cfg([lat(), lat(heads=2, dim=8, vdim=32, window=20)], streams=0, logit_scale=None), None),
    "latent attention without window or stretching": (make_cfg([lat(window=0, scaling=None)], streams=0), None),
    "latent attention on another layer's latents": (make_cfg([lat(), lat(kv_from=0, scale=0.5, heads=2, window=12), lat(kv_from=0)], streams=0), None),
    "gated recurrence": (make_cfg([rec(), rec(blocks=1, width=24, conv=2)], streams=0), None),
    "stream links": (make_cfg([lat(mlp=DENSE), rec()], streams=3), None),
    "dense feed-forward": (make_cfg([lat(mlp=DENSE), rec(mlp=DENSE)], streams=0), _silence_mixers),
    "routed feed-forward": (make_cfg([lat(mlp=MOE), rec(mlp=MOE)], streams=0), _silence_mixers),
}


def case_mechanism(tmp, device, dtype, kind):
    cfg, edit = MECHANISMS[kind]
    W, rig = _setup(tmp, cfg, dtype, device, seed=3, edit=edit)
    toks = tokens(110, cfg["vocab"], 1)
    want = expect(cfg, W, toks)
    strict = not _routed(cfg)
    _check(rig.run({"a": toks}, alone("a", len(toks), [len(toks)]))["a"], want, dtype, f"{kind} whole prompt", strict)
    _check(rig.run({"b": toks}, alone("b", len(toks), [31, 2, 1, 40, 1, 1, 7]))["b"], want, dtype, f"{kind} in portions", strict)


# ---------------------------------------------------------------- leaving a mechanism out must show
FAULTS = ("sink", "gate", "window_short", "window_long", "stretch", "correction", "identity", "renorm", "own_latents", "conv", "links",
          "center", "clamp", "bias")


def case_each_piece_matters(tmp, device, dtype):
    W, rig = _setup(tmp, FULL, dtype, device, seed=4)
    toks = tokens(70, FULL["vocab"], 2)
    want = expect(FULL, W, toks)
    for fault in FAULTS:
        # the oracle itself must tell these faults, or the comparison below shows nothing
        assert rel_err(expect(FULL, W, toks, (fault,))[40:], want[40:]) > 3 * TOL[dtype], fault
    _check(rig.run({"p": toks}, alone("p", 70, [70]))["p"], want, dtype, "prompt", strict=False)
    _check(rig.run({"d": toks}, alone("d", 70, [20, 2, 3] + [1] * 45))["d"], want, dtype, "portions and decoding", strict=False)


# ---------------------------------------------------------------- prefill against token-by-token, portions down to two
def case_prefill_decode_portions(tmp, device, dtype):
    W, rig = _setup(tmp, FULL, dtype, device, seed=5)
    toks = tokens(100, FULL["vocab"], 2)
    want = expect(FULL, W, toks)
    for name, sizes in (("whole", [100]), ("one by one", [1]), ("portions", [2, 3, 64, 5, 2, 17]), ("page edges", [32, 32, 1, 31, 4]),
                        ("shorter than the convolution", [2, 1, 2, 2, 1, 1, 3, 88])):
        _check(rig.run({name: toks}, alone(name, len(toks), sizes))[name], want, dtype, name, strict=False)


# ---------------------------------------------------------------- unequal requests in one batch against each alone
def case_mixed_batch(tmp, device, dtype):
    W, rig = _setup(tmp, FULL, dtype, device, seed=7, max_tokens=512)
    reqs = {"s1": tokens(1, FULL["vocab"], 10), "s23": tokens(23, FULL["vocab"], 11), "m70": tokens(70, FULL["vocab"], 12),
            "l130": tokens(130, FULL["vocab"], 13)}
    want = {i: expect(FULL, W, t) for i, t in reqs.items()}
    plan = {"s1": [1], "s23": [2, 1, 1, 16, 1, 1, 1], "m70": chunks(70, [33, 1, 1, 2, 1]), "l130": chunks(130, [40, 3, 1, 1, 64, 1])}
    sched, k = [], 0
    while any(plan.values()):
        step = [(i, plan[i].pop(0)) for i in ("l130", "s23", "m70", "s1") if plan[i] and (k % 3 != 2 or i != "s23")]
        k += 1
        if step:
            sched.append(step)
    got = rig.run(reqs, sched)
    for i in reqs:
        _check(got[i], want[i], dtype, f"request {i} in mixed batches", strict=False)


def case_mixed_batch_on_tiles(tmp, device, dtype):
    """Chunks of two sequences beside single tokens of others in one step, with sizes the matrix-core kernels take (on the
    GPU in bf16: chunks on the tile kernel, single tokens on the heads-as-columns kernel, experts as grouped products)."""
    cfg = other_size_configs()["matrix-core shapes, eight heads, wide experts"]
    W, rig = _setup(tmp, cfg, dtype, device, seed=21, max_tokens=640)
    reqs = {"a": tokens(150, cfg["vocab"], 50), "b": tokens(97, cfg["vocab"], 51), "c": tokens(40, cfg["vocab"], 52),
            "d": tokens(3, cfg["vocab"], 53)}
    want = {i: expect(cfg, W, t) for i, t in reqs.items()}
    sched = [[("a", 70), ("c", 33)], [("a", 1), ("b", 64), ("c", 1), ("d", 1)], [("a", 50), ("b", 1), ("c", 1), ("d", 2)],
             [("a", 1), ("b", 32), ("c", 5)], [("a", 28)]]
    got = rig.run(reqs, sched)
    for i in reqs:
        _check(got[i], want[i], dtype, f"request {i} beside the others", strict=False)


# ---------------------------------------------------------------- pages and state slots freed and used again
def case_reuse(tmp, device, dtype):
    W, rig = _setup(tmp, FULL, dtype, device, seed=9, max_tokens=160, max_seqs=2)      # five pages, two slots
    reqs = {f"r{j}": tokens(n, FULL["vocab"], 20 + j) for j, n in enumerate([70, 45, 64, 33, 80, 5])}
    want = {i: expect(FULL, W, t) for i, t in reqs.items()}
    sched = ([[("r0", 40), ("r1", 45)], [("r0", 30)]] +
             [[("r2", 30), ("r3", 2)], [("r3", 31), ("r2", 1)], [("r2", 33)]] +
             [[("r4", 64)], [("r4", 1), ("r5", 5)], [("r4", 15)]])
    got = rig.run(reqs, sched)
    for i in reqs:
        _check(got[i], want[i], dtype, f"request {i} after reuse", strict=False)
    bm = rig.rep.bm
    assert bm.num_free == bm.num_blocks and bm.num_free_state_slots == 2


# ---------------------------------------------------------------- a key far back among hundreds; memory of the recurrence
def _sharpen(Wt):
    for k in list(Wt):
        if k.endswith("mix.dq.norm") or k.endswith("mix.dkv.norm"):
            Wt[k] = Wt[k] * 2.5                               # peaked softmax: single keys carry weight
        if k.endswith("mix.sink"):
            Wt[k] = Wt[k] - 2.0
        if k.endswith("mix.lam"):
            Wt[k] = Wt[k] - 4.0                               # decays close to one: the state remembers hundreds of tokens


FAR = {
    "latent attention": make_cfg([lat(window=0, scale=0.5), lat(window=0, scale=0.5)], width=64),
    "another layer's latents": make_cfg([lat(window=0, scale=0.5), lat(window=0, scale=0.5, kv_from=0)], width=64),
    "gated recurrence": make_cfg([rec(), rec(blocks=2, width=32)], width=64),
}


def case_far_key(tmp, device, dtype, which):
    cfg = FAR[which]
    W, rig = _setup(tmp, cfg, dtype, device, seed=13, edit=_sharpen)
    toks = tokens(330, cfg["vocab"], 4)
    want = expect(cfg, W, toks)
    changed = list(toks)
    changed[1] = (toks[1] + 17) % cfg["vocab"]                # position 1 must reach the last rows
    assert rel_err(expect(cfg, W, changed)[-20:], want[-20:]) > 5 * TOL[dtype], which
    _check(rig.run({"p": toks}, alone("p", 330, [300] + [1] * 30))["p"], want, dtype, f"far keys ({which}), prompt then decoding")
    _check(rig.run({"c": toks}, alone("c", 330, [64, 63, 2, 129]))["c"], want, dtype, f"far keys ({which}), portions")


# ---------------------------------------------------------------- window edges: the last key inside, the first outside
def _one_key_stands_out(Wt):
    """One attention layer whose rows depend on the tokens inside the window only; flat scores and a low sink, so that every
    key of the window — the one at its edge too — carries about 1 / window of the weight."""
    for k in list(Wt):
        if k.endswith("mix.dq.norm"):
            Wt[k] = Wt[k] * 0.5
        if k.endswith("mix.sink"):
            Wt[k] = Wt[k] - 3.0


def case_window_edges(tmp, device, dtype, window):
    cfg = make_cfg([lat(window=window, scale=0.6)], width=64, streams=0)
    W, rig = _setup(tmp, cfg, dtype, device, seed=29, edit=_one_key_stands_out)
    n = 3 * window + 9
    toks = tokens(n, cfg["vocab"], 14)
    want = expect(cfg, W, toks)
    # a window one token off shows in the rows past the first window; the row where it shows most is the one whose edge key
    # carries most weight
    off = {f: _row_err(expect(cfg, W, toks, (f,)), want) for f in ("window_short", "window_long")}
    for f, e in off.items():
        assert np.median(e[window + 1:]) > 5 * TOL["float32"] and e.max() > TOL[dtype], f
    row = window + 1 + int(off["window_short"][window + 1:n - 2].argmax())
    j = row - window + 1
    # in the oracle: a changed token moves exactly the rows whose window holds it
    changed = list(toks)
    changed[j] = (toks[j] + 5) % cfg["vocab"]
    moved = _row_err(expect(cfg, W, changed), want)
    assert moved[row] > TOL[dtype] and moved[row + 1] == 0.0 and moved[j - 1] == 0.0
    # prompts cut at and beside the edge (pages of 32 tokens fall elsewhere), then decoding across several windows
    _check(rig.run({"w": toks}, alone("w", n, [n]))["w"], want, dtype, f"window {window}: whole prompt")
    _check(rig.run({"e": toks}, alone("e", n, [window, 1, window - 1, 2, window + 1, 5]))["e"], want, dtype, f"window {window}: cut at the edge")
    _check(rig.run({"d": toks}, alone("d", n, [window - 2] + [1] * (n - window + 2)))["d"], want, dtype, f"window {window}: decoding across")
    got = rig.run({"x": changed}, alone("x", n, [j + 1] + [1] * (n - j - 1)))["x"]
    _check(got, expect(cfg, W, changed), dtype, f"window {window}: changed token")


# ---------------------------------------------------------------- first tokens, very short requests, long decoding
def case_first_tokens_and_long_decode(tmp, device, dtype):
    W, rig = _setup(tmp, FULL, dtype, device, seed=15)
    for n in (1, 2, 3, 5):
        toks = tokens(n, FULL["vocab"], 30 + n)
        _check(rig.run({"x": toks}, alone("x", n, [1]))["x"], expect(FULL, W, toks), dtype, f"{n}-token request", strict=False)
        _check(rig.run({"y": toks}, alone("y", n, [n]))["y"], expect(FULL, W, toks), dtype, f"{n}-token prompt", strict=False)
    toks = tokens(190, FULL["vocab"], 5)
    _check(rig.run({"long": toks}, alone("long", 190, [20] + [1] * 170))["long"], expect(FULL, W, toks), dtype, "170 decoded tokens",
           strict=False)


# ---------------------------------------------------------------- other sizes
def other_size_configs():
    wide_moe = {"kind": "moe", "expert": {"ff": 128, "limit": 2.0}, "router": {"experts": 6, "identity": 2, "top": 3}}
    return {
        # latent and rotated parts in multiples of 16 and 8, eight heads (decode rows with the heads as matrix-core columns),
        # expert and model widths the grouped products and the weight-streaming kernels take
        "matrix-core shapes, eight heads, wide experts":
            make_cfg([lat(8, 32, 16, 32, 64, 48, 0.2, 45, mlp=wide_moe), rec(2, 128, 4, mlp=DENSE),
                      lat(8, 16, 16, 16, 64, 32, 0.25, 0, kv_from=0, mlp=wide_moe)], width=128, vocab=90, streams=4),
        "sixteen heads, latent of 128, no identity experts":
            make_cfg([lat(16, 16, 32, 16, 128, 64, 0.2, 100, base=1e5,
                          mlp={"kind": "moe", "expert": {"ff": 64, "limit": 1.0}, "router": {"experts": 4, "top": 2}}),
                      lat(16, 16, 32, 16, 128, 64, 0.2, 70, base=1e5, kv_from=0)], width=128, vocab=70, streams=1),
        "one head, one block, one tap, every output chosen": make_cfg(
            [lat(1, 16, 4, 64, 12, 8, 1.0, 3, mlp={"kind": "moe", "expert": {"ff": 8, "limit": 0.5}, "router": {"experts": 3, "identity": 3, "top": 6}}),
             rec(1, 40, 1, mlp={"kind": "moe", "expert": {"ff": 24, "limit": 4.0}, "router": {"experts": 3, "identity": 1, "top": 1}})],
            width=50, vocab=130, streams=1, eps=1e-3, logit_scale=None),    # a width that rules out 16-byte accesses
        "odd sizes, part of the key part rotated, six taps": make_cfg(
            [lat(3, 12, 10, 20, 22, 14, 0.4, 41, mlp=DENSE), rec(5, 35, 6), lat(2, 6, 10, 9, 22, 30, 0.4, 2, kv_from=0)],
            width=40, vocab=50, streams=3),
        "window of one, eight streams, blocks of two channels": make_cfg(
            [rec(12, 24, 7, mlp=MOE), lat(6, 8, 2, 8, 16, 16, 0.5, 1), lat(4, 8, 6, 8, 24, 16, 0.5, 64, scaling={"factor": 8.0, "original": 16, "fast": 4.0, "slow": 1.0})],
            width=88, vocab=97, streams=8, logit_scale=2.0),
    }


def _partly_rotated(cfg):
    """``rot.dims`` below ``rot_dim``: the tail of the shared key part passes unrotated."""
    cfg = copy.deepcopy(cfg)
    for l in cfg["layers"]:
        if l["type"] == "latent_attention":
            l["mixer"]["rot"]["dims"] = 6
    return cfg


def case_other_sizes(tmp, device, dtype, name):
    cfg = other_size_configs()[name]
    if name.startswith("odd sizes"):
        cfg = _partly_rotated(cfg)
    W, rig = _setup(tmp, cfg, dtype, device, seed=17)
    toks = tokens(75, cfg["vocab"], 6)
    want = expect(cfg, W, toks)
    strict = not _routed(cfg)
    _check(rig.run({"w": toks}, alone("w", 75, [75]))["w"], want, dtype, name + " whole", strict)
    _check(rig.run({"c": toks}, alone("c", 75, [2, 30, 1, 1, 33, 1]))["c"], want, dtype, name + " portions", strict)
    if "heads" in name:                                       # tiles that start inside a page, with hundreds of keys behind them
        toks = tokens(300, cfg["vocab"], 8)
        want = expect(cfg, W, toks)
        _check(rig.run({"l": toks}, alone("l", 300, [45, 130, 17, 64, 43, 1]))["l"], want, dtype, name + " long portions", strict)


# ---------------------------------------------------------------- greedy generation through the engine's own entry point
def case_generate(tmp, device, dtype, graphs=False):
    from dli_amd.config import CacheConfig, EngineConfig, SamplingParams, SchedulerConfig, resolve_model
    from dli_amd.engine.engine import LLMEngine
    W = write_checkpoint(tmp, FULL, 19, bf16=dtype == "bfloat16")
    mcfg, wpath = resolve_model(str(tmp), dtype)
    seqs, lens = (8, (5, 61, 30, 90, 2, 17, 33, 64, 1, 45, 8)) if graphs else (3, (5, 61, 30, 90, 2))
    eng = LLMEngine(EngineConfig(model=mcfg, weights_path=wpath, device=device, cache=CacheConfig(num_blocks=8 * seqs),
                                 sched=SchedulerConfig(max_num_seqs=seqs, max_num_batched_tokens=64, max_model_len=256,
                                                       long_prefill_chunk=40, token_alignment=0),
                                 use_hip_graphs=graphs, graph_batch_sizes=(1, 2, 4, 8), tune_gemms=False))
    if graphs:
        eng.warmup()
    prompts = [tokens(n, FULL["vocab"], 40 + n) for n in lens]                     # more requests than slots: some wait
    n_new = 10
    outs = eng.generate(None, SamplingParams(temperature=0.0, max_tokens=n_new, ignore_eos=True), prompt_ids=prompts)
    for p, o in zip(prompts, outs):
        assert len(o) == n_new
        seq = list(p)
        for tok in o:                                             # teacher-forced: every generated token is the oracle's argmax
            logits = oracle.forward(FULL, W, seq)[0][-1]
            top2 = torch.topk(logits, 2).values
            if float(top2[0] - top2[1]) > (1e-3 if dtype == "float32" else 0.3):   # skip near-ties
                assert int(torch.argmax(logits)) == tok
            seq.append(tok)
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == seqs
    if graphs:
        assert eng.runner.stats["graph_steps"] > 0, eng.runner.selftest
    return eng
