"""Sinilorn stacks on the gfx950 kernels (``csrc/kernels/recurmix.hip`` and the extended attention / stream / routing / expert
kernels), fp32 and bf16, against the plain oracle: the cases of ``sinilorn_cases`` on ``cuda``, plus generation with captured
decode / mixed-step hipGraphs and kernel-against-kernel comparisons of the fast paths."""
import pytest
import torch

import sinilorn_cases as cases

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(autouse=True)
def _needs_gpu():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from dli_amd import ops
    ops.hip()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", sorted(cases.MECHANISMS))
def test_each_mechanism_alone(tmp_path, kind, dtype):
    cases.case_mechanism(tmp_path, "cuda", dtype, kind)


@pytest.mark.parametrize("dtype", DTYPES)
def test_every_piece_shows_when_left_out(tmp_path, dtype):
    cases.case_each_piece_matters(tmp_path, "cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_prefill_decode_and_portions(tmp_path, dtype):
    cases.case_prefill_decode_portions(tmp_path, "cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_unequal_requests_in_one_batch(tmp_path, dtype):
    cases.case_mixed_batch(tmp_path, "cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_chunks_beside_single_tokens_at_matrix_core_sizes(tmp_path, dtype):
    cases.case_mixed_batch_on_tiles(tmp_path, "cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_pages_and_slots_used_again(tmp_path, dtype):
    cases.case_reuse(tmp_path, "cuda", dtype)


@pytest.mark.parametrize("which", sorted(cases.FAR))
def test_far_keys(tmp_path, which):
    cases.case_far_key(tmp_path, "cuda", "float32", which)     # the effect of one far token is below bf16 rounding


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [5, 32, 45])
def test_window_edges(tmp_path, window, dtype):
    cases.case_window_edges(tmp_path, "cuda", dtype, window)


def test_first_tokens_and_long_decoding(tmp_path):
    cases.case_first_tokens_and_long_decode(tmp_path, "cuda", "float32")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(cases.other_size_configs()))
def test_other_sizes(tmp_path, name, dtype):
    cases.case_other_sizes(tmp_path, "cuda", dtype, name)


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_eager(tmp_path, dtype):
    cases.case_generate(tmp_path, "cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_with_hip_graphs(tmp_path, dtype):
    eng = cases.case_generate(tmp_path, "cuda", dtype, graphs=True)
    st = eng.runner.selftest
    assert st.get("graph_vs_eager", {}).get("ok", True) and st.get("mixed_graph_vs_eager", {}).get("ok", True), st


def test_tiles_against_the_per_token_kernel(tmp_path, monkeypatch):
    """bf16 prompts through the matrix-core tile kernel and through the per-token kernel (both with window and sink) give the
    same logits up to rounding."""
    import numpy as np
    from dli_amd.ops import seqmix
    from rodelix_common import alone, tokens
    cfg = cases.other_size_configs()["sixteen heads, latent of 128, no identity experts"]
    W, rig = cases._setup(tmp_path, cfg, "bfloat16", "cuda", seed=23)
    toks = tokens(260, cfg["vocab"], 9)
    tiled = rig.run({"a": toks}, alone("a", 260, [70, 190]))["a"]
    monkeypatch.setattr(seqmix, "TILE_ATTENTION", False)
    plain = rig.run({"b": toks}, alone("b", 260, [70, 190]))["b"]
    assert not np.array_equal(tiled, plain), "both runs took the same kernel"
    cases._check(tiled, plain, "bfloat16", "tile kernel against the per-token kernel", strict=False)
    cases._check(tiled, cases.expect(cfg, W, toks), "bfloat16", "tile kernel against the oracle", strict=False)


def test_head_columns_against_the_per_token_kernel(tmp_path, monkeypatch):
    """bf16 decode rows: the heads of a token as matrix-core columns against the per-token kernel, window and sink included,
    decoding across the window."""
    import numpy as np
    from dli_amd.ops import seqmix
    from rodelix_common import alone, tokens
    cfg = cases.other_size_configs()["sixteen heads, latent of 128, no identity experts"]
    W, rig = cases._setup(tmp_path, cfg, "bfloat16", "cuda", seed=25)
    toks = tokens(160, cfg["vocab"], 10)
    fast = rig.run({"a": toks}, alone("a", 160, [80] + [1] * 80))["a"]
    monkeypatch.setattr(seqmix, "HEAD_DECODE", False)
    plain = rig.run({"b": toks}, alone("b", 160, [80] + [1] * 80))["b"]
    assert not np.array_equal(fast[80:], plain[80:]), "both runs took the same kernel"
    cases._check(fast, plain, "bfloat16", "heads as columns against the per-token kernel", strict=False)
    cases._check(fast, cases.expect(cfg, W, toks), "bfloat16", "heads as columns against the oracle", strict=False)


def test_block_scan_against_the_sequential_scan(tmp_path, monkeypatch):
    """The gated recurrence over a long prompt: the block-parallel prefill against the token-by-token walk."""
    from dli_amd.ops import seqmix
    from rodelix_common import alone, tokens
    cfg = cases.FAR["gated recurrence"]
    W, rig = cases._setup(tmp_path, cfg, "float32", "cuda", seed=27, edit=cases._sharpen)
    toks = tokens(400, cfg["vocab"], 11)
    blocks = rig.run({"a": toks}, alone("a", 400, [333, 67]))["a"]
    monkeypatch.setattr(seqmix, "BLOCK_SCAN", False)
    walk = rig.run({"b": toks}, alone("b", 400, [333, 67]))["b"]
    cases._check(blocks, walk, "float32", "block scan against the walk")
    cases._check(blocks, cases.expect(cfg, W, toks), "float32", "block scan against the oracle")


@pytest.mark.parametrize("T", [300, 100, 9])
def test_grouped_clamped_experts_against_the_row_kernels(T):
    """The clamped experts as grouped GEMMs (or, at decode size, weight streams) against the any-shape row kernels, same
    routing, identity experts among the picks."""
    from dli_amd import ops
    from dli_amd.ops import seqmix
    lib = ops.hip()
    torch.manual_seed(1)
    W, F, E, K, limit = 256, 128, 6, 3, 0.8
    h = torch.randn(T, W, device="cuda").bfloat16()
    gate_up = (torch.randn(E, 2 * F, W, device="cuda") / W ** 0.5).bfloat16()
    down = (torch.randn(E, W, F, device="cuda") / F ** 0.5).bfloat16()
    ids = torch.stack([torch.randperm(E + 2, device="cuda")[:K] for _ in range(T)]).int()      # ids E, E+1: identity experts
    wts = torch.softmax(torch.randn(T, K, device="cuda"), -1)
    try:
        grouped = seqmix.gated_experts(h, ids, wts, gate_up, down, limit=limit).float()
        lib.dm_set_grouped_experts(False)
        rows = seqmix.gated_experts(h, ids, wts, gate_up, down, limit=limit).float()
    finally:
        lib.dm_set_grouped_experts(True)
    want = seqmix.gated_experts(h.cpu(), ids.cpu(), wts.cpu(), gate_up.cpu(), down.cpu(), limit=limit).float().cuda()
    for got, name in ((grouped, "grouped"), (rows, "rows")):
        err = ((got - want).norm() / want.norm()).item()
        assert err < 1e-2, f"{name}: {err}"
    assert not torch.equal(grouped, rows), "both calls took the same kernels"


def test_router_kernel_against_the_reference_op():
    from dli_amd.ops import seqmix
    torch.manual_seed(2)
    for E, K, W in ((8, 3, 96), (64, 64, 40), (12, 4, 200), (1, 1, 16)):
        h, R, b = torch.randn(70, W), torch.randn(E, W) * 0.3, torch.randn(E) * 0.1
        if E > 3:
            R[3], b[3] = R[1], b[1]                            # a tie: the lower index wins
        ids, wts = seqmix.softmax_all_route(h, R, b, K)
        gi, gw = seqmix.softmax_all_route(h.cuda(), R.cuda(), b.cuda(), K)
        ch = torch.softmax(h @ R.t(), -1) + b
        gap = torch.sort(ch, -1, descending=True).values.diff(dim=-1).abs()
        clear = ((gap > 1e-5) | (gap == 0)).all(-1) | (E <= 3)  # rows whose order rounding cannot move (exact ties go by index)
        assert clear.sum() > 20 or E == 64
        assert torch.equal(gi.cpu()[clear], ids[clear]) and torch.allclose(gw.cpu()[clear], wts[clear], atol=1e-5)
    nan = torch.full((4, 32), float("nan")).cuda()             # rows of padding: picks stay inside the router's outputs
    gi, gw = seqmix.softmax_all_route(nan, torch.randn(6, 32).cuda(), torch.zeros(6).cuda(), 3)
    assert int(gi.min()) >= 0 and int(gi.max()) < 6 and bool(torch.isfinite(gw).all())
