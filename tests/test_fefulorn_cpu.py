"""Fefulorn on the CPU: configuration, spec and tensor names, the torch stand-ins of its kernels against the plain
implementation mechanism by mechanism (each mixer in pieces on scattered pages and on a slot that held something,
inputs made so that one key at a window's edge decides), and the engine's host side (cache and state manager, step
function, values handed from the first blending layer to the later ones, slots and pages used again) against the
plain model under every cut."""
import copy
import math

import pytest
import torch

from tests import trace_tools as tt
from tests.fefulorn_cases import (CASES, FEFU_A, attention_tensors, build_attention, build_latent, build_ssm,
                                  latent_tensors, make_folder, random_case, run_in_pieces, runtime, ssm_tensors)
from tests.plain import fefulorn_plain as plain
from tests.torch_ops import TorchOps

RANDOM_SEEDS = [201, 202, 203, 204, 205, 206, 207, 208]
F64 = torch.float64


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
    from return_amd.config.fefulorn import FefulornConfig
    cfg = FefulornConfig.from_dict(FEFU_A)
    assert [layer["type"] for layer in cfg.layers] == ["mamba2", "attention", "attention", "latent_attention",
                                                       "attention", "attention"]
    assert FefulornConfig.from_dict(cfg.to_dict()) == cfg
    for change in (lambda c: c["layers"][0].update(type="gla"),
                   lambda c: c["layers"][0]["mixer"].update(groups=3),
                   lambda c: c["layers"][0]["mixer"].update(norm_groups=5),
                   lambda c: c["layers"][0]["mixer"].pop("conv"),
                   lambda c: c["layers"][1]["mixer"].update(kv_heads=3),
                   lambda c: c["layers"][1]["mixer"].pop("scale"),
                   lambda c: c["layers"][1]["mixer"]["rot"].update(dims=3),
                   lambda c: c["layers"][1]["mixer"]["rot"].update(dims=10),
                   lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].update(factor=0.0),
                   lambda c: c["layers"][1]["mixer"]["mask"].update(size=0),
                   lambda c: c["layers"][3]["mixer"].update(kv_rank=0),
                   lambda c: c["layers"][0]["mlp"].update(kind="dense"),
                   lambda c: c["layers"][0]["mlp"]["router"].update(top=5),
                   lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4),
                   lambda c: c["layers"][0]["mlp"]["shared"].pop("limit"),
                   lambda c: c.update(layers=[]),
                   lambda c: c.pop("norm")):
        bad = copy.deepcopy(FEFU_A)
        change(bad)
        with pytest.raises(ConfigError):
            FefulornConfig.from_dict(bad)


def test_spec_names_the_tensors_and_gives_every_layer_its_own_cache(model):
    from return_amd.config import load_config, lookup_architecture
    folder, cfg, w = model
    config = load_config(folder)
    spec = lookup_architecture(config.architecture)[1](config)
    assert set(spec.expected_tensors()) == set(w)
    assert [call.cache for call in spec.schedule] == list(range(len(cfg["layers"])))
    blending = [i for i, layer in enumerate(cfg["layers"]) if layer["type"] == "attention" and layer["mixer"].get("v_mix")]
    for i, layer in enumerate(cfg["layers"]):
        assert (f"l{i}.norm2" in w) == (layer["mlp"] is not None)
        assert (f"l{i}.mix.vmix" in w) == (i in blending)
        params = spec.blocks[i].parts["mixer"][1].params
        assert bool(params.get("first_of_blend")) == (bool(blending) and i == blending[0])


def test_a_stored_model_may_leave_sizes_to_defaults_and_hold_unused_tensors(tmp_path_factory):
    """config.json need not name kv_heads, vdim or q_rank where they are what the other sizes say; a file may hold the
    blend weight of a layer that does not blend and the second norm of a layer without feed-forward."""
    import json
    import os
    from safetensors.torch import load_file, save_file
    raw = copy.deepcopy(FEFU_A)
    raw["layers"][4]["mixer"].update(vdim=10, v_mix=False)        # values as wide as keys, heads ungrouped
    raw["layers"] = raw["layers"][3:5]
    from tests.conftest import make_folder as make
    folder = make(tmp_path_factory, "fefulorn_defaults", dict(raw, architectures=["Fefulorn"]), dict(seed=5, std=0.1))
    path = os.path.join(folder, "config.json")
    with open(path) as f:
        stored = json.load(f)
    stored["layers"][0]["mixer"].pop("q_rank")
    for key in ("kv_heads", "vdim", "v_mix"):
        stored["layers"][1]["mixer"].pop(key)
    with open(path, "w") as f:
        json.dump(stored, f)
    st = os.path.join(folder, "model.safetensors")
    tensors = load_file(st)
    tensors["l1.mix.vmix"] = torch.tensor(0.5, dtype=torch.bfloat16)
    save_file(tensors, st)
    cfg, w = plain.read_folder(folder)
    toks = tt.random_tokens(cfg["vocab"], 12, seed=3)
    got = tt.run_in_process(runner_for(folder, 64), tt.whole({"r": toks}))
    torch.testing.assert_close(torch.stack([got[("r", p)] for p in range(12)]).double(), plain.logits(cfg, w, toks),
                               atol=2e-4, rtol=1e-4)


# ------------------------------------------------------------------ the stand-ins, mechanism by mechanism
def test_linearly_stretched_rotary_tables_are_the_rule_in_64_bit():
    from return_amd.parts.position import RotaryPosition
    rt = runtime(TorchOps("cpu"), positions=300)
    for base, dims, factor in ((100.0, 4, 3.0), (200000.0, 32, 1.0), (10000.0, 16, 2.0), (10.0, 2, 8.0)):
        part = RotaryPosition({"head_dim": dims + 2, "rotary_dim": dims, "theta": base, "max_position": None,
                               "exact_tables": True, "linear_factor": factor}, {}, rt)
        cos, sin, n = part.tables()
        f = base ** (-2.0 * torch.arange(dims // 2, dtype=F64) / dims) / factor
        a = torch.arange(300, dtype=F64)[:, None] * f[None, :]
        assert n == dims and cos.shape == (300, dims // 2)
        torch.testing.assert_close(cos.double(), a.cos(), atol=1e-6, rtol=0)
        torch.testing.assert_close(sin.double(), a.sin(), atol=1e-6, rtol=0)


ATTENTIONS = [
    dict(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.4, mask={"size": 7}, rot={"base": 100.0, "dims": 4, "scaling": {"factor": 3.0}}, v_mix=True),
    dict(heads=3, kv_heads=3, dim=10, vdim=4, scale=0.3, mask={"size": 20}, rot={"base": 1000.0, "dims": 10}, v_mix=True),
    dict(heads=2, kv_heads=1, dim=16, vdim=16, scale=0.25, v_mix=True),
]


@pytest.mark.parametrize("m", ATTENTIONS, ids=["grouped_wide_values", "narrow_values_all_rotated", "no_window_no_rotation"])
def test_blending_attention_in_pieces_equals_the_plain_function(m):
    """Two layers of the same shape, the first hands its values to the second; every cut gives the plain result."""
    from return_amd.parts.share import TokenRows
    g = torch.Generator().manual_seed(m["heads"])
    W, T = 24, 41
    w1, w2 = attention_tensors(g, W, m), attention_tensors(g, W, m)
    x1, x2 = torch.randn(T, W, generator=g), torch.randn(T, W, generator=g)
    d = lambda w: {k: v.double() for k, v in w.items()}
    y1, v_first = plain.attention(x1.double(), d(w1), m, None)
    y2, _ = plain.attention(x2.double(), d(w2), m, v_first)
    y2_alone, _ = plain.attention(x2.double(), d(w2), m, None)
    assert (y2 - y2_alone).abs().max() > 1e-3                     # the blend does something
    for pieces in ([T], [1] * T, [5, 2, 1, 17, 16]):
        rt = runtime(TorchOps("cpu"))
        rows = TokenRows({}, {}, rt)
        parts = [build_attention(rt, W, m, w1, {"rows": rows}, first_of_blend=True), build_attention(rt, W, m, w2, {"rows": rows})]
        got1, got2 = run_in_pieces(parts, [x1, x2], pieces)
        torch.testing.assert_close(got1.double(), y1, atol=2e-5, rtol=1e-5)
        torch.testing.assert_close(got2.double(), y2, atol=2e-5, rtol=1e-5)


def deciding_rows(T, W, query_at, key_at, g):
    """Rows that are small noise but for two that point the same way, the key's row far out and the query's row less
    far: where queries and keys are the same map of a row, the query's score with that key stands far above its score
    with itself and with every other key."""
    x = 0.01 * torch.randn(T, W, generator=g)
    u = torch.randn(W, generator=g)
    x[key_at], x[query_at] = 4.0 * u, 1.5 * u
    return x, u


def test_a_key_just_inside_the_window_decides_and_one_just_outside_does_not():
    """One key's score stands far above the others of one query. When it is the window's last key the output is that
    key's value; one place further back the output must not know it. As a prompt, decoded, and cut between the two."""
    m = dict(heads=2, kv_heads=2, dim=8, vdim=6, scale=1.0, mask={"size": 9}, v_mix=False)
    g = torch.Generator().manual_seed(7)
    W, T, q_at = 16, 30, 25
    w = attention_tensors(g, W, m)
    w["k"], w["k.b"], w["q.b"] = w["q"].clone(), torch.zeros_like(w["k.b"]), torch.zeros_like(w["q.b"])
    d = {k: v.double() for k, v in w.items()}
    for key_at, inside in ((q_at - 8, True), (q_at - 9, False)):
        x, u = deciding_rows(T, W, q_at, key_at, g)
        # the scale that puts the key's score 20 above the query's score with itself, in the weaker head
        m["scale"] = 20.0 / (3.75 * float(((d["q"] @ u.double()).view(2, 8) ** 2).sum(-1).min()))
        want, _ = plain.attention(x.double(), d, m, None)
        alone = plain.attention_values(x.double(), d, m)[key_at].reshape(-1) @ d["o"].T     # if only that key counts
        assert ((want[q_at] - alone).abs().max() < 1e-4) == inside
        for pieces in ([T], [q_at] + [1] * (T - q_at), [key_at + 1, 3, T - key_at - 4]):
            rt = runtime(TorchOps("cpu"))
            got, = run_in_pieces([build_attention(rt, W, m, w)], [x], pieces)
            torch.testing.assert_close(got.double(), want, atol=2e-5, rtol=1e-5)


LATENTS = [
    dict(heads=3, dim=8, vdim=6, q_rank=10, kv_rank=12, scale=0.4, mask={"size": 6}),
    dict(heads=1, dim=5, vdim=9, q_rank=7, kv_rank=5, scale=0.3),
    dict(heads=4, dim=16, vdim=16, q_rank=24, kv_rank=32, scale=0.2, mask={"size": 19}),
]


@pytest.mark.parametrize("m", LATENTS, ids=["short_window", "one_head_no_window", "window_over_a_page"])
def test_latent_attention_in_pieces_equals_the_plain_function(m):
    g = torch.Generator().manual_seed(m["heads"])
    W, T, eps = 20, 45, 1e-5
    w = latent_tensors(g, W, m)
    x = torch.randn(T, W, generator=g)
    want = plain.latent_attention(x.double(), {k: v.double() for k, v in w.items()}, m, eps)
    for pieces in ([T], [1] * T, [6, 2, 1, 20, 16]):
        rt = runtime(TorchOps("cpu"))
        got, = run_in_pieces([build_latent(rt, W, m, w, eps)], [x], pieces)
        torch.testing.assert_close(got.double(), want, atol=2e-5, rtol=1e-5)


SSMS = [
    dict(heads=4, vdim=8, state=6, groups=2, norm_groups=1, conv=3),
    dict(heads=3, vdim=10, state=7, groups=3, norm_groups=5, conv=2),
    dict(heads=2, vdim=16, state=16, groups=1, norm_groups=2, conv=5),
]


@pytest.mark.parametrize("m", SSMS, ids=["grouped", "norm_parts_through_heads", "long_filter"])
def test_state_space_mixer_in_pieces_equals_the_plain_function(m):
    g = torch.Generator().manual_seed(m["heads"])
    W, T, eps = 24, 37, 1e-5
    w = ssm_tensors(g, W, m)
    x = torch.randn(T, W, generator=g)
    want, _, _ = plain.mamba2(x.double(), {k: v.double() for k, v in w.items()}, m, eps)
    for pieces in ([T], [1] * T, [2, 1, 9, 2, 23]):
        rt = runtime(TorchOps("cpu"))
        got, = run_in_pieces([build_ssm(rt, W, m, w, eps)], [x], pieces)
        torch.testing.assert_close(got.double(), want, atol=2e-5, rtol=1e-5)


def test_state_space_memory_keeps_what_it_should_and_forgets_what_it_should():
    """With a decay of one (a step size of nearly zero times a rate of nearly zero) nothing is forgotten over 150
    tokens: the state is the sum of all writes; with a huge rate only the newest write is left."""
    m = dict(heads=2, vdim=4, state=3, groups=1, norm_groups=1, conv=2)
    g = torch.Generator().manual_seed(3)
    W, T, eps = 12, 150, 1e-5
    w = ssm_tensors(g, W, m)
    x = torch.randn(T, W, generator=g)
    for a_log, keeps in ((-30.0, True), (12.0, False)):
        w["A_log"] = torch.full((2,), a_log)
        d = {k: v.double() for k, v in w.items()}
        want, S, _ = plain.mamba2(x.double(), d, m, eps)
        _, S_last, _ = plain.mamba2(x[-1:].double(), d, m, eps, tail=(x[-2:-1].double() @ d["in"].T)[:, 8:8 + 8 + 6])
        assert ((S - S_last).abs().max() > 1e-3) == keeps
        rt = runtime(TorchOps("cpu"))
        got, = run_in_pieces([build_ssm(rt, W, m, w, eps)], [x], [100, 1, 1, 48], pages=tuple(range(12)))
        torch.testing.assert_close(got.double(), want, atol=5e-5, rtol=1e-4)


def test_router_takes_the_best_of_the_kept_groups_and_leaves_the_scores_as_they_are():
    ops = TorchOps("cpu")
    g = torch.Generator().manual_seed(1)
    for E, top, count, keep in ((12, 4, 3, 2), (8, 2, 4, 1), (6, 6, 1, 1), (9, 1, 9, 3), (16, 4, 2, 2)):
        z = 2.0 * torch.randn(50, E, generator=g)
        ids, weights = ops.moe_route(z, None, top, count, keep, 0.0, law="softmax_groups")
        want_ids, want_w = plain.route(z.double(), top, count, keep)
        assert torch.equal(ids.long().sort(-1).values, want_ids.sort(-1).values)
        torch.testing.assert_close(weights.double().sort(-1).values, want_w.sort(-1).values, atol=1e-6, rtol=1e-5)
        assert bool((weights.sum(-1) < 1.0 - 1e-4).any()) or top == E     # nothing is renormed
    # a group that holds the second and third largest scores loses to the group with the largest one
    z = torch.tensor([[5.0, -9.0, 4.0, 4.5, -9.0, -9.0]])
    ids, _ = ops.moe_route(z, None, 1, 3, 1, 0.0, law="softmax_groups")
    assert ids.tolist() == [[0]]
    ids, _ = ops.moe_route(z, None, 2, 3, 1, 0.0, law="softmax_groups")
    assert sorted(ids.tolist()[0]) == [0, 1]                       # the second choice comes from the kept group


def test_experts_with_the_shared_one_equal_the_plain_function():
    from return_amd.parts.moe import GroupedRoutedExperts
    g = torch.Generator().manual_seed(2)
    W, T = 20, 33
    for E, top, groups, ff, limit, shared in ((6, 2, (3, 2), 12, 0.7, (10, 1.2)), (4, 4, None, 8, 2.0, None),
                                              (5, 1, None, 16, 1.0, (4, 0.4))):
        mlp = {"expert": {"ff": ff, "limit": limit}, "router": {"experts": E, "top": top}}
        if groups:
            mlp["router"]["groups"] = {"count": groups[0], "keep": groups[1]}
        r = lambda *shape, s=1.0: s * torch.randn(*shape, generator=g)
        w = {"router": r(E, W, s=0.5)}
        for e in range(E):
            w.update({f"e{e}.gate": r(ff, W, s=0.4), f"e{e}.up": r(ff, W, s=0.4), f"e{e}.down": r(W, ff, s=0.3)})
        params = {"hidden_size": W, "expert_size": ff, "experts": E, "top": top, "groups": groups[0] if groups else 1,
                  "keep": groups[1] if groups else 1, "router": "softmax_groups", "activation": "clamped", "limit": limit}
        names = GroupedRoutedExperts.tensor_names("", E)
        del names["correction"]
        if shared:
            mlp["shared"] = {"ff": shared[0], "limit": shared[1]}
            params["shared"] = {"size": shared[0], "limit": shared[1]}
            w.update({"shared.gate": r(shared[0], W, s=0.4), "shared.up": r(shared[0], W, s=0.4),
                      "shared.down": r(W, shared[0], s=0.3), "shared.sg": r(1, W, s=0.4)})
            names.update({"shared_gate": "shared.gate", "shared_up": "shared.up", "shared_down": "shared.down",
                          "shared_weight": "shared.sg"})
        assert set(GroupedRoutedExperts.tensor_shapes(params)) == set(names)
        rt = runtime(TorchOps("cpu"))
        part = GroupedRoutedExperts(params, {role: w[name] for role, name in names.items()}, rt)
        x = torch.randn(T, W, generator=g)
        want = plain.moe(x.double(), {k: v.double() for k, v in w.items()}, mlp)
        torch.testing.assert_close(part.forward(x).double(), want, atol=2e-5, rtol=1e-5)


def test_both_norms_of_a_layer_in_one_pass_are_the_two_norms():
    ops = TorchOps("cpu")
    g = torch.Generator().manual_seed(4)
    h = torch.randn(7, 20, generator=g)
    a, b = torch.randn(7, 20, generator=g), torch.randn(7, 20, generator=g)
    w1, w2 = 1 + 0.2 * torch.randn(20, generator=g), 1 + 0.2 * torch.randn(20, generator=g)
    want_h = h.double() + a.double() + b.double()
    x1, x2 = torch.empty(7, 20), torch.empty(7, 20)
    ops.add_rmsnorm_pair(h, a, b, w1, 1e-5, x1, w2, 1e-6, x2)
    torch.testing.assert_close(h.double(), want_h, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(x1.double(), plain.norm_plain(want_h, w1.double(), 1e-5), atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(x2.double(), plain.norm_plain(want_h, w2.double(), 1e-6), atol=1e-5, rtol=1e-5)


def test_the_stream_after_every_layer_is_the_plain_one(model):
    """The decoder's stream with everything pending added, layer by layer (a whole prompt)."""
    folder, cfg, w = model
    runner = runner_for(folder, 64)
    toks = tt.random_tokens(cfg["vocab"], 21, seed=9)
    want = []
    plain.forward(cfg, w, toks, want)
    seen = []
    from return_amd.parts.runtime import Pair
    for i, block in enumerate(runner.model.blocks):
        def wrapped(h, pending, step, cache, write_cache=True, _f=block.forward):
            h, out = _f(h, pending, step, cache, write_cache)
            total = h.clone()
            for part in ((out.first, out.second) if isinstance(out, Pair) else (out,)):
                total += part.float()
            seen.append(total)
            return h, out
        block.forward = wrapped
    tt.run_in_process(runner, tt.whole({"r": toks}))
    assert len(seen) == len(want)
    for got, ref in zip(seen, want):
        torch.testing.assert_close(got.double(), ref, atol=3e-4, rtol=1e-4)


# ------------------------------------------------------------------ the engine's host side under every cut
def _requests(cfg, seed):
    lens = [70, 1, 23, 41, 2, 64]
    return {f"r{i}": tt.random_tokens(cfg["vocab"], n, seed=seed + i) for i, n in enumerate(lens)}


def _check(got, cfg, w, requests, atol=3e-4):
    for rid, toks in requests.items():
        want = plain.logits(cfg, w, toks)
        rows = torch.stack([got[(rid, p)] for p in range(len(toks))]).double()
        torch.testing.assert_close(rows, want, atol=atol, rtol=1e-4)


def test_engine_equals_plain_under_every_cut(model):
    folder, cfg, w = model
    requests = _requests(cfg, 11)
    for name, steps in (("whole", tt.whole(requests)), ("tail", tt.tail_decoded(requests, tail=20)),
                        ("portions", tt.portions(requests)), ("mixed", tt.mixed(requests, seed=3))):
        runner = runner_for(folder, tt.peak_tokens(steps, 16) + 16, page=16)
        _check(tt.run_in_process(runner, steps), cfg, w, requests)


def test_pages_of_four_and_slots_used_again(tmp_path_factory):
    folder = make_folder(tmp_path_factory, "a")
    cfg, w = plain.read_folder(folder)
    requests = {f"r{i}": tt.random_tokens(cfg["vocab"], n, seed=40 + i) for i, n in enumerate([30, 9, 55, 3, 26, 47, 12])}
    steps = tt.mixed(requests, seed=5, max_live=3, decode_tail=5, sizes=(6, 2, 13, 3))
    runner = runner_for(folder, tt.peak_tokens(steps, 4) + 8, page=4, max_live=3)
    _check(tt.run_in_process(runner, steps), cfg, w, requests)


def test_a_batch_of_unequal_requests_equals_each_alone(tmp_path_factory):
    folder = make_folder(tmp_path_factory, "b")
    cfg, w = plain.read_folder(folder)
    requests = {f"r{i}": tt.random_tokens(cfg["vocab"], n, seed=60 + i) for i, n in enumerate([37, 2, 18, 5])}
    together = [{"step": 0, "entries": [{"id": r, "tokens": t, "want": list(range(len(t)))} for r, t in requests.items()],
                 "end": list(requests)}]
    got = tt.run_in_process(runner_for(folder, 128), together)
    alone = tt.run_in_process(runner_for(folder, 128), tt.whole(requests))
    for key in alone:
        torch.testing.assert_close(got[key], alone[key], atol=1e-5, rtol=1e-5)
    _check(got, cfg, w, requests)


def test_greedy_generation_through_the_engine_equals_plain(tmp_path_factory):
    from return_amd.config import EngineConfig
    from return_amd.engine import Engine, ModelRunner
    from return_amd.sampling import SamplingParams
    folder = make_folder(tmp_path_factory, "a")
    cfg, w = plain.read_folder(folder)
    ec = EngineConfig(dtype="float32", device="cpu", page_size=16, max_token=256, max_reside=4, max_step_tokens=32,
                      prefill_chunk=16, use_graphs=False, tune_products=False, check_invariants=True)
    eng = Engine(runner=ModelRunner(folder, engine_config=ec, ops=TorchOps("cpu")))
    prompts = [tt.random_tokens(cfg["vocab"], n, seed=80 + n) for n in (5, 29, 1, 14, 40)]
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=9))
    for prompt, out in zip(prompts, outs):
        assert list(out.output_ids) == plain.greedy(cfg, w, prompt, 9)
