"""The Sevelorn test cases, parametrised by device and dtype.  Each case builds its own small configuration, writes a
checkpoint from the plain oracle's random weights (``sevelorn_oracle``), replays step schedules through the engine
(``rodelix_common.Rig``: the engine's runner, block manager, cache, state slots and kernels) and compares every position's
logits with the oracle.  The same cases run on the CPU path (``test_sevelorn.py``) and on the GPU kernels
(``test_sevelorn_gpu.py``)."""
from __future__ import annotations

import copy
import json
import os

import numpy as np
import torch

import sevelorn_oracle as oracle
from rodelix_common import Rig, TOL, alone, chunks, rel_err, tokens

MOE = {"kind": "moe", "expert": {"ff": 40}, "router": {"experts": 5, "top": 2}}
DENSE = {"kind": "dense", "ff": 88}


def attn(heads=4, kv_heads=2, dim=24, vdim=16, scale=0.3, mlp=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": copy.deepcopy(mlp)}


def ret(heads=3, dim=16, vdim=24, decay=(0.8, 0.96, 0.999), rot=(8, 5000.0), mlp=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
    return {"type": "retention", "mixer": m, "mlp": copy.deepcopy(mlp)}


def make_cfg(layers, width=72, vocab=149, streams=2, taps=4, scale=1.7, eps=1e-5):
    cfg = {"architecture": "Sevelorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": [copy.deepcopy(l) for l in layers]}
    if streams:
        cfg["streams"] = streams
    if taps:
        cfg["canon"] = {"taps": taps}
    if scale is not None:
        cfg["embedding"] = {"scale": scale}
    return cfg


# every mixer, a layer on another layer's keys / values (twice, past a retention layer), both feed-forwards, none
FULL = make_cfg([attn(mlp=MOE), ret(mlp=DENSE), attn(kv_from=0, scale=0.2, mlp=MOE), ret(heads=2, dim=20, vdim=12, decay=(0.9, 1.0), rot=(20, 300.0)),
                 attn(heads=2, kv_heads=2, dim=24, vdim=16, mlp=DENSE), attn(kv_from=0, mlp=None)])


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
    logits nearly tie to another expert now and then, so the bound holds for the bulk of the rows (median well inside, at
    most one row in seven outside); what a cut, a page or a slot can break shows in the fp32 run of the same case."""
    e = _row_err(got, want)
    if dtype == "float32" or strict:
        assert e.max() < TOL[dtype], f"{what}: relative error {e.max():.3e} over {TOL[dtype]:.1e}"
    else:
        assert np.median(e) < TOL[dtype] / 4 and (e > TOL[dtype]).mean() <= 1 / 7, \
            f"{what}: median {np.median(e):.3e}, {(e > TOL[dtype]).mean():.0%} of the rows over {TOL[dtype]:.1e}"


# ---------------------------------------------------------------- each mechanism alone
def _silence_mixers(Wt):
    for k in Wt:
        if k.endswith("mix.o"):
            Wt[k] = Wt[k] * 0.0


MECHANISMS = {
    "attention": (make_cfg([attn(), attn(heads=3, kv_heads=3, dim=8, vdim=32)], streams=0, taps=0), None),
    "attention on another layer's keys and values": (make_cfg([attn(), attn(kv_from=0, scale=0.5), attn(kv_from=0)], streams=0, taps=0), None),
    "retention": (make_cfg([ret(), ret(heads=2, dim=24, vdim=8, decay=(0.5, 0.99), rot=(24, 100.0))], streams=0, taps=0), None),
    "input convolution": (make_cfg([attn(), ret()], streams=0, taps=5), None),
    "stream links": (make_cfg([attn(mlp=DENSE), ret()], streams=3, taps=0), None),
    "dense feed-forward": (make_cfg([attn(mlp=DENSE), attn(mlp=DENSE)], streams=0, taps=0), _silence_mixers),
    "routed feed-forward": (make_cfg([attn(mlp=MOE), attn(mlp=MOE)], streams=0, taps=0), _silence_mixers),
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
def case_each_piece_matters(tmp, device, dtype):
    W, rig = _setup(tmp, FULL, dtype, device, seed=4)
    toks = tokens(60, FULL["vocab"], 2)
    want = expect(FULL, W, toks)
    # (the key scale of retention is not among them: the unit norm behind the state takes a constant factor out again, up
    # to eps; the op-level test of the rotation kernel covers it)
    for fault in ("gate", "conv", "rotation", "router_bias", "embed_scale", "own_kv"):
        # the oracle itself must tell these faults, or the comparison below shows nothing
        assert rel_err(expect(FULL, W, toks, (fault,))[6:], want[6:]) > 3 * TOL[dtype], fault
    _check(rig.run({"p": toks}, alone("p", 60, [60]))["p"], want, dtype, "prompt", strict=False)
    _check(rig.run({"d": toks}, alone("d", 60, [20, 2, 3] + [1] * 35))["d"], want, dtype, "portions and decoding", strict=False)


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
    """Chunks of two sequences beside single tokens of others in one step, with heads of 64 (on the GPU in bf16: the chunks
    take the matrix-core tile kernel, the single tokens the per-token kernels)."""
    cfg = other_size_configs()["matrix-core tiles, heads of 64, shared keys, no feed-forward"]
    W, rig = _setup(tmp, cfg, dtype, device, seed=21, max_tokens=640)
    reqs = {"a": tokens(150, cfg["vocab"], 50), "b": tokens(97, cfg["vocab"], 51), "c": tokens(40, cfg["vocab"], 52),
            "d": tokens(3, cfg["vocab"], 53)}
    want = {i: expect(cfg, W, t) for i, t in reqs.items()}
    sched = [[("a", 70), ("c", 33)], [("a", 1), ("b", 64), ("c", 1), ("d", 1)], [("a", 50), ("b", 1), ("c", 1), ("d", 2)],
             [("a", 1), ("b", 32), ("c", 5)], [("a", 28)]]
    got = rig.run(reqs, sched)
    for i in reqs:
        _check(got[i], want[i], dtype, f"request {i} beside the others")


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
        if k.endswith("mix.q.norm") or k.endswith("mix.k.norm"):
            Wt[k] = Wt[k] * 3.0                               # peaked softmax: single keys carry weight


FAR = {
    "attention": make_cfg([attn(scale=1.0), attn(scale=1.0)], width=64, taps=2),
    "another layer's keys": make_cfg([attn(scale=1.0), attn(scale=1.0, kv_from=0)], width=64, taps=2),
    "retention": make_cfg([ret(decay=(0.9995, 0.999, 1.0)), ret(decay=(0.9995, 0.999, 1.0))], width=64, taps=2),
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
    big_moe = {"kind": "moe", "expert": {"ff": 64}, "router": {"experts": 6, "top": 3}}
    wide_moe = {"kind": "moe", "expert": {"ff": 128}, "router": {"experts": 4, "top": 2}}
    return {
        "matrix-core tiles, heads of 64, shared keys, no feed-forward":
            make_cfg([attn(8, 2, 64, 64, 0.15), ret(2, 64, 64, (0.97, 0.999), (32, 1e4)), attn(8, 2, 64, 64, 0.1, kv_from=0)], width=96, vocab=80),
        "matrix-core tiles, heads of 128, one query head per key head":
            make_cfg([attn(2, 2, 128, 128, 0.1), attn(2, 2, 128, 128, 0.1, kv_from=0)], width=64, vocab=70, streams=1, taps=1),
        # (an expert width of 128 also takes the weight-streaming kernels at decode size)
        "experts as grouped products": make_cfg([attn(2, 1, 64, 64, 0.15, mlp=big_moe), ret(2, 32, 64, (0.9, 0.99), (16, 1e4), mlp=wide_moe)],
                                                width=128, vocab=90, streams=4, taps=2),
        "eight query heads per key head": make_cfg([attn(16, 2, 16, 32, 0.35, mlp=DENSE), attn(8, 1, 32, 16, 0.2)], width=56, vocab=64, streams=5),
        "single heads, every expert chosen, one tap": make_cfg(
            [attn(1, 1, 16, 64, 1.0, mlp={"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 7, "top": 7}}),
             ret(1, 40, 8, (0.93,), (2, 1e6), mlp={"kind": "moe", "expert": {"ff": 24}, "router": {"experts": 3, "top": 1}})],
            width=50, vocab=130, streams=1, taps=1, eps=1e-3, scale=None),      # a width that rules out 16-byte accesses
        "odd head sizes, no rotation, wide state": make_cfg([attn(3, 3, 12, 20, 0.4, mlp=DENSE), ret(2, 100, 70, (0.9, 0.99), None)],
                                                            width=40, vocab=50, streams=3, taps=6),
        "partly rotated heads, seven taps, eight streams": make_cfg([ret(4, 32, 16, (0.5, 0.9, 0.99, 0.999), (6, 50.0)), attn(6, 3, 8, 8, 0.5)],
                                                                    width=88, vocab=97, streams=8, taps=7, scale=0.5),
    }


def case_other_sizes(tmp, device, dtype, name):
    cfg = other_size_configs()[name]
    W, rig = _setup(tmp, cfg, dtype, device, seed=17)
    toks = tokens(75, cfg["vocab"], 6)
    want = expect(cfg, W, toks)
    strict = not _routed(cfg)
    _check(rig.run({"w": toks}, alone("w", 75, [75]))["w"], want, dtype, name + " whole", strict)
    _check(rig.run({"c": toks}, alone("c", 75, [2, 30, 1, 1, 33, 1]))["c"], want, dtype, name + " portions", strict)
    if "matrix-core" in name:                                 # tiles that start inside a page, with hundreds of keys behind them
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
