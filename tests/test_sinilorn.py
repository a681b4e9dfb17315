"""Sinilorn stacks on the CPU path of the ops (fp32 torch references behind the same model, runner, block manager and
engine code as on the GPU) against the plain oracle ``sinilorn_oracle``; plus the configuration reader and single ops
against the oracle's functions.  The GPU kernels run the same cases in ``test_sinilorn_gpu.py``."""
import types

import pytest
import torch

import sinilorn_cases as cases
import sinilorn_oracle as oracle


@pytest.mark.parametrize("kind", sorted(cases.MECHANISMS))
def test_each_mechanism_alone(tmp_path, kind):
    cases.case_mechanism(tmp_path, "cpu", "float32", kind)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_piece_shows_when_left_out(tmp_path, dtype):
    cases.case_each_piece_matters(tmp_path, "cpu", dtype)


def test_prefill_decode_and_portions(tmp_path):
    cases.case_prefill_decode_portions(tmp_path, "cpu", "float32")


def test_unequal_requests_in_one_batch(tmp_path):
    cases.case_mixed_batch(tmp_path, "cpu", "float32")


def test_chunks_beside_single_tokens_at_matrix_core_sizes(tmp_path):
    cases.case_mixed_batch_on_tiles(tmp_path, "cpu", "float32")


def test_pages_and_slots_used_again(tmp_path):
    cases.case_reuse(tmp_path, "cpu", "float32")


@pytest.mark.parametrize("which", sorted(cases.FAR))
def test_far_keys(tmp_path, which):
    cases.case_far_key(tmp_path, "cpu", "float32", which)


@pytest.mark.parametrize("window", [5, 32, 45])
def test_window_edges(tmp_path, window):
    cases.case_window_edges(tmp_path, "cpu", "float32", window)


def test_first_tokens_and_long_decoding(tmp_path):
    cases.case_first_tokens_and_long_decode(tmp_path, "cpu", "float32")


@pytest.mark.parametrize("name", sorted(cases.other_size_configs()))
def test_other_sizes(tmp_path, name):
    cases.case_other_sizes(tmp_path, "cpu", "float32", name)


def test_greedy_generation_through_the_engine(tmp_path):
    cases.case_generate(tmp_path, "cpu", "float32")


def test_layer_outputs_against_the_oracle(tmp_path):
    """The sum of the streams after every layer, not only the logits."""
    from dli_amd.engine.trace import TraceReplayer
    W = cases.write_checkpoint(tmp_path, cases.FULL, 23)
    toks = cases.tokens(40, cases.FULL["vocab"], 9)
    want = oracle.forward(cases.FULL, W, toks)[1]
    rep = TraceReplayer(str(tmp_path), "float32", 64, 2, "cpu")
    rep.runner.model.layer_outputs = got = []
    rep.step([{"id": "a", "tokens": toks, "want": []}], ["a"])
    assert len(got) == len(cases.FULL["layers"])
    for i, (g, w) in enumerate(zip(got, want)):
        assert torch.allclose(g.double(), w, rtol=2e-4, atol=2e-4 * float(w.abs().max())), f"after layer {i}"


def load_model_config_from(cfg, path):
    import json
    import os
    from dli_amd.config import load_model_config
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    return load_model_config(str(path), "float32")


def test_config_reader(tmp_path):
    from dli_amd.config import get_model_config, load_model_config, resolve_model
    cases.write_checkpoint(tmp_path, cases.FULL, 1)
    cfg = load_model_config(str(tmp_path), "float32")
    assert cfg.arch == "sinilorn" and cfg.stateful and len(cfg.layer_specs) == 6
    assert (cfg.streams, cfg.stream_norm, cfg.logit_scale, cfg.conv_taps) == (2, "layer", 0.6, 0)
    a, r, shared = cfg.layer_specs[0], cfg.layer_specs[1], cfg.layer_specs[2]
    assert a.kind == "gated_latent_attention" and a.kv_from == -1 and a.sink
    assert (a.heads, a.dim, a.rot_dim, a.vdim, a.kv_rank, a.q_rank, a.scale, a.window) == (3, 16, 8, 24, 40, 32, 0.25, 37)
    assert (a.rot_dims, a.rot_base, a.rot_scaling) == (8, 3000.0, (3.0, 48.0, 12.0, 1.5))
    assert (a.ff_kind, a.router, a.ff_act, a.experts, a.identity_experts, a.top, a.ff, a.ff_limit) == ("moe", "softmax_all", "clamped", 5, 2, 3, 40, 1.5)
    assert r.kind == "rglru" and (r.heads, r.dim, r.conv_taps) == (3, 16, 4) and r.state_shape == (48,)
    assert (r.ff_kind, r.ff_act, r.ff, r.ff_bias) == ("dense", "silu", 88, True)
    assert shared.kv_from == 0 and shared.cache_row == (0, 0) and a.cache_row == (48, 0) and shared.window == 50
    assert cfg.layer_specs[5].window == 0 and cfg.layer_specs[5].ff == 0 and cfg.layer_specs[4].rot_scaling == ()
    assert resolve_model(str(tmp_path))[1] == str(tmp_path)
    assert get_model_config("tiny-sinilorn").arch == "sinilorn"
    plain = load_model_config_from(cases.make_cfg([cases.rec()], streams=0, logit_scale=None), tmp_path / "plain")
    assert (plain.streams, plain.logit_scale) == (0, 1.0)
    for bad in ([cases.lat(kv_from=0)], [cases.rec(), cases.lat(kv_from=0)], [cases.lat(), cases.lat(kv_rank=8, kv_from=0)],
                [cases.lat(), cases.lat(kv_from=0), cases.lat(kv_from=1)], [cases.rec(blocks=5)],
                [cases.lat(mlp={"kind": "moe", "expert": {"ff": 8, "limit": 1.0}, "router": {"experts": 2, "identity": 1, "top": 4}})]):
        with pytest.raises(ValueError):
            load_model_config_from(cases.make_cfg(bad), tmp_path / "bad")


def test_shared_pages_are_one_tensor_and_counted_once():
    from dli_amd.config import get_model_config
    from dli_amd.models import build_model
    m = build_model(get_model_config("tiny-sinilorn"))
    caches = m.allocate_caches(3, 2, "cpu")
    assert caches[2].k is caches[0].k and caches[0].v is None and caches[1].k is None
    assert m.bytes_per_block() == 32 * 4 * (32 + 8)
    assert caches[1].shift.shape == (2, 3, 48) and caches[1].state.shape == (2, 48)
    assert m.bytes_per_slot() == 4 * 48 * 4


def test_router_picks_and_weights_against_the_oracle():
    from dli_amd.ops import seqmix
    torch.manual_seed(0)
    h, R, b = torch.randn(40, 24), torch.randn(9, 24), torch.randn(9) * 0.2
    R[3], b[3] = R[1], b[1]                                    # a tie: the lower index wins
    b[5] = 5.0                                                 # always chosen, whatever its score: the weight stays the score
    ids, wts = seqmix.softmax_all_route(h, R, b, 4)
    picks = oracle.route({"router": R.double(), "correction": b.double()}, "", {"router": {"top": 4}}, h.double())
    for t, (order, w) in enumerate(picks):
        assert ids[t].tolist() == order and ids[t, 0] == 5
        assert torch.allclose(wts[t].double(), w, atol=1e-6)
    assert torch.allclose(wts.sum(-1), torch.ones(40), atol=1e-6)


def _one_chunk(n, pos0=0):
    """Step metadata of one sequence bringing ``n`` tokens from position ``pos0`` (what the CPU references read)."""
    return types.SimpleNamespace(num_decode=0, num_prefill=1, query_start_loc=torch.tensor([0, n], dtype=torch.int32),
                                 state_slots=torch.tensor([0], dtype=torch.int32), positions=torch.arange(pos0, pos0 + n, dtype=torch.int32))


def test_small_ops_against_the_oracle():
    from dli_amd.ops import seqmix
    torch.manual_seed(1)
    # convolution: whole, and in two portions through the state rows
    x, w, b = torch.randn(9, 6), torch.randn(6, 4), torch.randn(6)
    want = oracle.causal_conv(x.double(), w.double(), b.double())
    st = torch.zeros(1, 3, 6)
    assert torch.allclose(seqmix.causal_conv(x, w.t().contiguous(), b, st, _one_chunk(9), torch.float32).double(), want, atol=1e-5)
    st = torch.full((1, 3, 6), 7.0)                            # a reused slot: nothing before position 0 is read
    a = seqmix.causal_conv(x[:2], w.t().contiguous(), b, st, _one_chunk(2), torch.float32)
    c = seqmix.causal_conv(x[2:], w.t().contiguous(), b, st, _one_chunk(7, 2), torch.float32)
    assert torch.allclose(torch.cat([a, c]).double(), want, atol=1e-5)
    # rotation of the query heads' last entries, stretched frequencies
    rot = {"base": 77.0, "dims": 6, "scaling": {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}}
    q = torch.randn(11, 3 * (5 + 8))
    f, mag = seqmix.stretched_inv_freq(77.0, 6, (4.0, 32.0, 8.0, 1.0))
    fo, mo = oracle.frequencies(rot)
    assert torch.allclose(f, fo) and abs(mag - mo) < 1e-12 and not torch.allclose(f, oracle.frequencies(rot, plain=True)[0])
    got = q.clone()
    seqmix.rotate_heads(got, torch.arange(11, dtype=torch.int32), f, mag, 6, 3, 5, 8)
    want = q.double().view(11, 3, 13).clone()
    want[:, :, 5:] = oracle.rotate(want[:, :, 5:], rot)
    assert torch.allclose(got.double().view(11, 3, 13), want, atol=1e-5)
    # clamped experts with an identity expert
    h, gu, dn = torch.randn(7, 10), torch.randn(2, 12, 10), torch.randn(2, 10, 6)
    ids, wts = torch.tensor([[0, 2], [1, 0], [2, 1], [2, 2], [0, 1], [1, 2], [0, 0]], dtype=torch.int32), torch.rand(7, 2)
    got = seqmix.gated_experts(h, ids, wts, gu, dn, limit=0.7)
    for t in range(7):
        want = torch.zeros(10, dtype=torch.float64)
        for e, we in zip(ids[t].tolist(), wts[t].double()):
            Wt = {"gate": gu[e, :6].double(), "up": gu[e, 6:].double(), "down": dn[e].double()} if e < 2 else None
            want += we * (oracle.expert(Wt, "", h[t].double(), 0.7) if e < 2 else h[t].double())
        assert torch.allclose(got[t].double(), want, atol=1e-5)
