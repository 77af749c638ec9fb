"""Safilorn on the CPU: configuration, spec and tensor names, the torch stand-ins of its kernels against the plain
implementation mechanism by mechanism (each mixer in pieces on scattered pages and on a slot that held something,
inputs made so that one far key or the sink decides), and the engine's host side (cache and state manager, step
function, the stream formed out of all layers' results, slots and pages used again) against the plain model
under every cut."""
import copy
import math

import pytest
import torch

from tests import trace_tools as tt
from tests.plain import safilorn_plain as plain
from tests.safilorn_cases import (CASES, SAFI_A, SAFI_B, build_gla, build_latent, gla_tensors, latent_tensors, make_folder,
                                  random_case, run_mixer_in_pieces)
from tests.torch_ops import TorchOps

RANDOM_SEEDS = [101, 102, 103, 104, 105, 106]


@pytest.fixture(scope="module", params=sorted(CASES) + RANDOM_SEEDS, ids=str)
def model(request, tmp_path_factory):
    folder = make_folder(tmp_path_factory, request.param)
    cfg, w = plain.read_folder(folder)
    return folder, cfg, w


def runner_for(folder, max_tokens, page=16, max_live=4, **kw):
    from return_amd.config import EngineConfig
    from return_amd.engine import ModelRunner
    ec = EngineConfig(dtype="float32", device="cpu", page_size=page, max_token=max_tokens, max_reside=max_live,
                      max_step_tokens=max(max_tokens, 4), prefill_chunk=max_tokens, use_graphs=False,
                      tune_products=False, **kw)
    return ModelRunner(folder, engine_config=ec, ops=TorchOps("cpu"))


# ------------------------------------------------------------------ configuration and spec
def test_config_reads_every_layer_and_refuses_what_it_cannot_run():
    from return_amd.config.base import ConfigError
    from return_amd.config.safilorn import SafilornConfig
    cfg = SafilornConfig.from_dict(SAFI_A)
    assert [layer["type"] for layer in cfg.layers] == ["gla", "latent_attention", "gla", "latent_attention"]
    assert SafilornConfig.from_dict(cfg.to_dict()) == cfg
    for change in (lambda c: c["layers"][0].update(type="attention"),
                   lambda c: c["layers"][1]["mixer"].update(kv_rank=0),
                   lambda c: c["layers"][1]["mixer"].pop("scale"),
                   lambda c: c["layers"][1]["mixer"]["rot"].update(dims=3),
                   lambda c: c["layers"][1]["mixer"]["rot"].update(dims=6),
                   lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].pop("fast"),
                   lambda c: c["layers"][0]["mixer"].update(tau=0.0),
                   lambda c: c["layers"][0]["mlp"].update(kind="routed"),
                   lambda c: c["layers"][0]["mlp"]["router"].update(top=7),
                   lambda c: c["layers"][1]["mlp"].pop("ff"),
                   lambda c: c.update(layers=[]),
                   lambda c: c.pop("norm")):
        bad = copy.deepcopy(SAFI_A)
        change(bad)
        with pytest.raises(ConfigError):
            SafilornConfig.from_dict(bad)


def test_spec_names_the_tensors_and_gives_every_layer_its_own_cache(model):
    from return_amd.config import load_config, lookup_architecture
    folder, cfg, w = model
    config = load_config(folder)
    spec = lookup_architecture(config.architecture)[1](config)
    assert set(spec.expected_tensors()) == set(w)
    assert [call.cache for call in spec.schedule] == list(range(len(cfg["layers"])))
    assert [call.stream_mix for call in spec.schedule] == list(range(len(cfg["layers"])))
    for i, layer in enumerate(cfg["layers"]):
        assert tuple(w[f"l{i}.dwa"].shape) == (i + 2,)
        assert (f"l{i}.norm2" in w) == (layer["mlp"] is not None)


def test_a_stored_model_gives_the_sizes_that_config_leaves_out(tmp_path_factory):
    """config.json need not name the decay's rank nor the query latent's size: the shapes in the file do. A file
    may also hold the second pair of norms of a layer without feed-forward."""
    import json
    import os
    from safetensors.torch import load_file, save_file
    folder = make_folder(tmp_path_factory, "a")
    path = os.path.join(folder, "config.json")
    with open(path) as f:
        raw = json.load(f)
    for layer in raw["layers"]:
        layer["mixer"].pop("rank", None)
        layer["mixer"].pop("q_rank", None)
    with open(path, "w") as f:
        json.dump(raw, f)
    st = os.path.join(folder, "model.safetensors")
    tensors = load_file(st)
    tensors["l2.norm2"] = torch.zeros(raw["width"], dtype=torch.bfloat16)
    tensors["l2.norm2b"] = torch.zeros(raw["width"], dtype=torch.bfloat16)
    save_file(tensors, st)
    cfg, w = plain.read_folder(folder)
    toks = tt.random_tokens(cfg["vocab"], 12, seed=3)
    got = tt.run_in_process(runner_for(folder, 64), tt.whole({"r": toks}))
    torch.testing.assert_close(torch.stack([got[("r", p)] for p in range(12)]).double(), plain.logits(cfg, w, toks),
                               atol=2e-4, rtol=1e-4)


# ------------------------------------------------------------------ the stand-ins, mechanism by mechanism
def test_stretched_rotary_tables_are_the_rule_in_64_bit():
    from return_amd.parts.position import RotaryPosition
    from return_amd.parts.runtime import Runtime
    rt = Runtime("cpu", "float32", ops=TorchOps("cpu"))
    for base, dims, stretch in ((100.0, 4, (4.0, 16, 8.0, 1.0)), (200000.0, 32, (40.0, 256, 24.0, 0.5)),
                                (10000.0, 16, (2.0, 64, 4.0, 1.0)), (10.0, 2, (8.0, 8, 4.0, 1.0)), (500.0, 6, None)):
        rot = {"base": base, "dims": dims}
        if stretch:
            rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), stretch))
        part = RotaryPosition({"head_dim": dims, "rotary_dim": dims, "theta": base, "max_position": 300,
                               "exact_tables": True, "scaling": rot.get("scaling")}, {}, rt)
        cos, sin, n = part.tables()
        f, m = plain.yarn_frequencies(rot)
        a = torch.arange(300, dtype=torch.float64)[:, None] * f[None, :]
        assert n == dims
        torch.testing.assert_close(cos.double(), a.cos() * m, atol=1e-6, rtol=0)
        torch.testing.assert_close(sin.double(), a.sin() * m, atol=1e-6, rtol=0)
        if stretch and dims > 2:                                  # the blend does something: some pair turns slower
            assert bool((f < base ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / dims) * 0.999).any())


LATENTS = [
    dict(heads=3, dim=8, rot_dim=4, vdim=6, q_rank=10, kv_rank=12, scale=0.4, rot={"base": 100.0, "dims": 4}),
    dict(heads=1, dim=5, rot_dim=6, vdim=9, q_rank=7, kv_rank=5, scale=0.3,
         rot={"base": 1000.0, "dims": 6, "scaling": {"factor": 4.0, "original": 16, "fast": 8.0, "slow": 1.0}}),
    dict(heads=4, dim=16, rot_dim=8, vdim=16, q_rank=24, kv_rank=32, scale=0.2,
         rot={"base": 10000.0, "dims": 4, "scaling": {"factor": 2.0, "original": 32, "fast": 4.0, "slow": 0.5}}),
]


@pytest.mark.parametrize("m", LATENTS, ids=["three_heads", "one_head_stretched", "half_rotated"])
def test_latent_attention_in_pieces_equals_the_plain_function(m):
    g = torch.Generator().manual_seed(m["heads"])
    W, T, eps = 20, 61, 1e-5
    w = latent_tensors(g, W, m)
    x = torch.randn(T, W, generator=g)
    want = plain.latent_attention(x.double(), {k: v.double() for k, v in w.items()}, m, eps)
    part = build_latent(TorchOps("cpu"), W, m, w, eps, 64)
    for pieces in ((T,), (7, 1, 1, 20, 2, 30), (1,) * T):
        got = run_mixer_in_pieces(part, x, pieces)
        torch.testing.assert_close(got.double(), want, atol=3e-5, rtol=1e-4)


@pytest.mark.parametrize("spot,pieces", [(0, (64,)), (0, (63, 1)), (15, (20, 44)), (16, (3, 2, 59)), (47, (63, 1)), (62, (64,))])
def test_latent_attention_one_key_decides(spot, pieces):
    """The latent rows are made so that one key's score stands far out: the last token's result must then be that
    key's value row through the output maps, whichever page it lies on; and with every score far below the sink,
    the result must be nearly zero."""
    m = LATENTS[0]
    g = torch.Generator().manual_seed(4)
    W, T, eps = 20, 64, 1e-5
    w = latent_tensors(g, W, m)
    w["sink"] = torch.zeros(m["heads"])
    x = 0.05 * torch.randn(T, W, generator=g)
    x[spot] = 6.0 * torch.randn(W, generator=g)                  # one token unlike the others...
    x[T - 1] = x[spot]                                           # ...and the last one asks for it
    w64 = {k: v.double() for k, v in w.items()}
    want = plain.latent_attention(x.double(), w64, m, eps)
    part = build_latent(TorchOps("cpu"), W, m, w, eps, 64)
    got = run_mixer_in_pieces(part, x, pieces)
    torch.testing.assert_close(got.double(), want, atol=3e-5, rtol=1e-4)
    # the sink: its share of the softmax takes the result down by exactly its factor
    w_big = dict(w, sink=torch.full((m["heads"],), 30.0))
    part = build_latent(TorchOps("cpu"), W, m, w_big, eps, 64)
    sunk = run_mixer_in_pieces(part, x, pieces)
    torch.testing.assert_close(sunk.double(), plain.latent_attention(x.double(), {k: v.double() for k, v in w_big.items()}, m, eps),
                               atol=3e-5, rtol=1e-4)
    assert float(sunk[T - 1].abs().max()) < 1e-3 * float(got[T - 1].abs().max()) + 1e-6 or float(got[T - 1].abs().max()) < 1e-4


GLAS = [(dict(heads=3, dim=8, vdim=12, tau=4.0), 5), (dict(heads=1, dim=16, vdim=8, tau=1.0), 3),
        (dict(heads=2, dim=6, vdim=6, tau=16.0), 1)]


@pytest.mark.parametrize("m,rank", GLAS, ids=["three_heads", "tau_one", "rank_one"])
def test_gla_in_pieces_equals_the_plain_recurrence(m, rank):
    g = torch.Generator().manual_seed(m["heads"])
    W, T, eps = 24, 45, 1e-5
    w = gla_tensors(g, W, m, rank)
    x = torch.randn(T, W, generator=g)
    want, _ = plain.gla(x.double(), {k: v.double() for k, v in w.items()}, m, eps)
    part = build_gla(TorchOps("cpu"), W, m, w, eps)
    for pieces in ((T,), (4, 1, 1, 2, 37), (1,) * T):
        got = run_mixer_in_pieces(part, x, pieces)
        torch.testing.assert_close(got.double(), want, atol=3e-5, rtol=1e-4)


def test_gla_remembers_a_far_token_through_decays_near_one():
    """With the decay's bias large the state forgets nothing: a key written at the start is read out 200 tokens
    later; with the bias very negative the state keeps only the newest token."""
    m, rank = dict(heads=2, dim=8, vdim=8, tau=2.0), 2
    g = torch.Generator().manual_seed(8)
    W, T, eps = 16, 200, 1e-6
    w = gla_tensors(g, W, m, rank)
    x = 0.3 * torch.randn(T, W, generator=g)
    for bias in (12.0, -40.0):
        w["a2.b"] = torch.full((m["heads"] * m["dim"],), bias)
        want, S = plain.gla(x.double(), {k: v.double() for k, v in w.items()}, m, eps)
        part = build_gla(TorchOps("cpu"), W, m, w, eps)
        got = run_mixer_in_pieces(part, x, (150, 2, 1, 1, 46))
        torch.testing.assert_close(got.double(), want, atol=5e-5, rtol=1e-4)
    k_last = (x[-1].double() @ w["k"].double().T).view(2, 8)
    v_last = (x[-1].double() @ w["v"].double().T).view(2, 8)
    torch.testing.assert_close(S, k_last[:, :, None] * v_last[:, None, :], atol=1e-6, rtol=0)      # bias -40: only the newest


def test_router_and_clamped_experts_stand_ins():
    g = torch.Generator().manual_seed(6)
    T, W, E, I, top, limit = 33, 20, 7, 12, 3, 0.6
    x = torch.randn(T, W, generator=g)
    w = {"router": torch.randn(E, W, generator=g), "router.b": torch.randn(E, generator=g)}
    for e in range(E):
        w.update({f"e{e}.gate": torch.randn(I, W, generator=g) * 0.4, f"e{e}.up": torch.randn(I, W, generator=g) * 0.4,
                  f"e{e}.down": torch.randn(W, I, generator=g) * 0.3})
    w64 = {k: v.double() for k, v in w.items()}
    mlp = {"router": {"experts": E, "top": top}, "expert": {"ff": I, "limit": limit}}
    ops = TorchOps("cpu")
    z = x @ w["router"].T
    ids, weights = ops.moe_route(z, w["router.b"], top, 1, 1, 0.0, law="softmax_top")
    want_ids, want_w = plain.route(x.double(), w64, top)
    assert torch.equal(ids.long().sort(-1).values, want_ids.sort(-1).values)
    torch.testing.assert_close(weights.sum(-1), torch.ones(T))
    gu = torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]) for e in range(E)])
    down = torch.stack([w[f"e{e}.down"] for e in range(E)])
    got = ops.moe_experts(x, ids, weights, gu, down, activation="clamped", limit=limit, slope=1.702)
    torch.testing.assert_close(got.double(), plain.moe_ff(x.double(), w64, mlp), atol=3e-5, rtol=1e-4)
    # the clamps act: some gate above the limit, some up beyond it on both sides
    assert bool(((x @ w["e0.gate"].T) > limit).any()) and bool(((x @ w["e0.up"].T).abs() > limit).any())


def test_norms_on_both_sides_and_the_weighted_stream():
    g = torch.Generator().manual_seed(7)
    T, W, n = 9, 28, 4
    ops = TorchOps("cpu")
    h = torch.randn(T, W, generator=g)
    y = torch.randn(T, W, generator=g)
    w1, w2 = 1 + 0.2 * torch.randn(W, generator=g), 1 + 0.2 * torch.randn(W, generator=g)
    want = h.double() + plain.norm_around_zero(y.double(), w1.double() - 1, 1e-5)
    x = torch.empty(T, W)
    ops.post_norm_add(h, y, w1, 1e-5, w2, 1e-5, x)
    torch.testing.assert_close(h.double(), want, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(x.double(), plain.norm_around_zero(want, w2.double() - 1, 1e-5), atol=1e-5, rtol=1e-5)
    results = torch.randn(n + 1, T, W, generator=g)
    weights = torch.randn(n, generator=g)
    normed = torch.empty(T, W)
    ops.depth_mix(results, n, weights, results[n], w1, 1e-5, normed)
    want = sum(weights[j].double() * results[j].double() for j in range(n))
    torch.testing.assert_close(results[n].double(), want, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(normed.double(), plain.norm_around_zero(want, w1.double() - 1, 1e-5), atol=1e-5, rtol=1e-5)


# ------------------------------------------------------------------ the engine's host side against the plain model
LENGTHS = {"a": 5, "b": 17, "c": 33, "d": 100, "e": 64, "f": 131, "g": 1, "h": 47}


@pytest.mark.parametrize("cut", ["whole", "tail_decoded", "portions", "mixed"])
def test_engine_matches_plain_under_every_cut(model, cut):
    folder, cfg, w = model
    reqs = {rid: tt.random_tokens(cfg["vocab"], n, seed=ord(rid)) for rid, n in LENGTHS.items()}
    steps = {"whole": tt.whole, "tail_decoded": tt.tail_decoded, "portions": tt.portions, "mixed": tt.mixed}[cut](reqs)
    # the pool holds exactly the trace's peak and there are four slots: pages and slots are used again
    runner = runner_for(folder, tt.peak_tokens(steps), check_invariants=True)
    got = tt.run_in_process(runner, steps)
    for rid, toks in reqs.items():
        want = plain.logits(cfg, w, toks)
        for p in range(len(toks)):
            torch.testing.assert_close(got[(rid, p)].double(), want[p], atol=3e-4, rtol=1e-4,
                                       msg=lambda m: f"request {rid} position {p} (first wrong place): {m}")
    assert not runner.cache.live and all(g.pages.in_use() == 0 for g in runner.cache.groups)


def test_stream_after_every_layer_is_the_weighted_sum(tmp_path_factory):
    """The plain model's streams after each layer, against what the decoder holds: the last one feeds the head, so
    the logits agree only if every weighted sum did; here the sums themselves, with weights that make them differ
    strongly from the newest result alone."""
    folder = make_folder(tmp_path_factory, "b")
    cfg, w = plain.read_folder(folder)
    toks = tt.random_tokens(cfg["vocab"], 21, seed=5)
    _, after = plain.forward(cfg, w, toks, return_layers=True)
    only_newest = copy.deepcopy(w)
    for i in range(len(cfg["layers"])):
        only_newest[f"l{i}.dwa"] = torch.zeros(i + 2, dtype=torch.float64)
        only_newest[f"l{i}.dwa"][-1] = 1.0
    _, chained = plain.forward(cfg, only_newest, toks, return_layers=True)
    assert float((after[-1] - chained[-1]).abs().max()) > 1e-2 * float(after[-1].abs().max())
    got = tt.run_in_process(runner_for(folder, 64), tt.portions({"r": toks}, sizes=(2, 5, 1, 13)))
    want = plain.logits(cfg, w, toks)
    for p in range(len(toks)):
        torch.testing.assert_close(got[("r", p)].double(), want[p], atol=3e-4, rtol=1e-4)


def test_a_freed_slot_starts_from_zero_again(tmp_path_factory):
    """A request that takes over the slot and pages of a longer one must not see what that one left."""
    folder = make_folder(tmp_path_factory, "a")
    cfg, w = plain.read_folder(folder)
    runner = runner_for(folder, 128, max_live=1)
    first = tt.random_tokens(cfg["vocab"], 90, seed=1)
    second = tt.random_tokens(cfg["vocab"], 30, seed=2)
    tt.run_in_process(runner, tt.whole({"x": first}))
    got = tt.run_in_process(runner, tt.portions({"y": second}, sizes=(2, 3, 1, 9)))
    want = plain.logits(cfg, w, second)
    for p in range(len(second)):
        torch.testing.assert_close(got[("y", p)].double(), want[p], atol=3e-4, rtol=1e-4)


def test_greedy_generation_through_the_engine_on_the_cpu(tmp_path_factory):
    from return_amd import SamplingParams
    from return_amd.engine import Engine
    folder = make_folder(tmp_path_factory, "b")
    cfg, w = plain.read_folder(folder)
    prompts = [tt.random_tokens(cfg["vocab"], n, seed=n) for n in (1, 9, 30)]
    want = [plain.greedy(cfg, w, p, 6) for p in prompts]
    from return_amd.config import EngineConfig
    from return_amd.engine import ModelRunner
    ec = EngineConfig(dtype="float32", device="cpu", page_size=16, max_token=256, max_reside=4, max_step_tokens=32,
                      prefill_chunk=12, use_graphs=False, tune_products=False)
    eng = Engine(runner=ModelRunner(folder, engine_config=ec, ops=TorchOps("cpu")))
    got = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=6))
    assert [r.output_ids for r in got] == want
