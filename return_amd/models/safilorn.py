"""Safilorn as a ModelSpec: a decoder whose layers are described one by one in config.json.

Every layer has RMS norms (weights stored around zero, applied as 1 + w) on both sides of each sublayer:
h += norm1b(mixer(norm1(h))); h += norm2b(ff(norm2(h))), the feed-forward optional. The mixer is an attention over
a latent row per token (queries through a latent too, a rotated key part shared by the heads with stretched
rotary frequencies, a learned sink in the softmax, a gate per head) or a gated linear attention with a decay per
key channel; the feed-forward a dense gated one with biases or routed experts with clamped activations and a
softmax over the chosen logits. After every layer the stream becomes a weighted sum of the embedding's output
(the table's rows times embedding.scale) and of all layers' results so far. Tensor names: "embed", "final.norm",
"head", and "l<i>." + norm1, norm1b, norm2, norm2b, dwa, mix.*, mlp.*.
"""
from __future__ import annotations

from ..config.base import register_architecture
from ..config.safilorn import SafilornConfig
from ..parts.moe import GroupedRoutedExperts
from ..parts.spec import BlockSpec, LayerCall, ModelSpec, PartSpec


def _latent_attention(cfg, i, m, positions):
    p = f"l{i}.mix."
    rot = m["rot"]
    stretch = rot.get("scaling")
    key = tuple(float(stretch[k]) for k in ("factor", "original", "fast", "slow")) if stretch else ()
    position = f"rotary_{int(m['rot_dim'])}_{int(rot['dims'])}_{float(rot['base'])!r}_{key!r}"
    positions.setdefault(position, PartSpec("rotary", {
        "head_dim": int(m["rot_dim"]), "rotary_dim": int(rot["dims"]), "theta": float(rot["base"]),
        "max_position": None, "exact_tables": True, "scaling": dict(stretch) if stretch else None}))
    params = {"hidden_size": cfg.width, "num_heads": int(m["heads"]), "head_dim": int(m["dim"]),
              "rot_dim": int(m["rot_dim"]), "value_dim": int(m["vdim"]), "q_rank": int(m["q_rank"]) if m.get("q_rank") else None,
              "kv_rank": int(m["kv_rank"]), "scale": float(m["scale"]), "eps": float(cfg.norm["eps"]),
              "position": position, "sink": True, "gate": True}
    tensors = {"dq": p + "dq", "dq_norm": p + "dq.norm", "uq": p + "uq", "dkv": p + "dkv", "dkv_norm": p + "dkv.norm",
               "uk": p + "uk", "uv": p + "uv", "sink": p + "sink", "gate": p + "g", "o": p + "o"}
    return PartSpec("latent_attention", params, tensors)


def _gla(cfg, i, m):
    p = f"l{i}.mix."
    params = {"hidden_size": cfg.width, "num_heads": int(m["heads"]), "head_dim": int(m["dim"]),
              "value_dim": int(m["vdim"]), "tau": float(m["tau"]), "eps": float(cfg.norm["eps"]),
              "decay_rank": int(m["rank"]) if m.get("rank") else None}
    tensors = {"q_proj": p + "q", "k_proj": p + "k", "v_proj": p + "v", "g_proj": p + "g", "o_proj": p + "o",
               "o_norm": p + "norm", "a1_proj": p + "a1", "a2_proj": p + "a2", "a2_bias": p + "a2.b"}
    return PartSpec("gated_linear_attention", params, tensors)


def _feed_forward(cfg, i, mlp):
    p = f"l{i}.mlp."
    if mlp["kind"] == "dense":
        return PartSpec("swiglu", {"hidden_size": cfg.width, "intermediate_size": int(mlp["ff"]), "bias": True},
                        {"gate_proj": p + "gate", "up_proj": p + "up", "down_proj": p + "down",
                         "gate_bias": p + "gate.b", "up_bias": p + "up.b", "down_bias": p + "down.b"})
    r = mlp["router"]
    params = {"hidden_size": cfg.width, "expert_size": int(mlp["expert"]["ff"]), "experts": int(r["experts"]),
              "top": int(r["top"]), "router": "softmax_top", "activation": "clamped",
              "limit": float(mlp["expert"]["limit"]), "slope": 1.702}
    return PartSpec("routed_experts", params,
                    GroupedRoutedExperts.tensor_names(p, int(r["experts"]), "router_bias", "router.b"))


def build_spec(cfg: SafilornConfig) -> ModelSpec:
    W, eps = cfg.width, float(cfg.norm["eps"])
    norm = lambda name: PartSpec("rms_norm", {"size": W, "eps": eps, "offset": 1.0}, {"weight": name})
    positions, blocks, mixes, ignorable = {}, [], [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        mixer = _latent_attention(cfg, i, layer["mixer"], positions) if layer["type"] == "latent_attention" \
            else _gla(cfg, i, layer["mixer"])
        parts = {"mixer_norm": ("norm", norm(p + "norm1")), "mixer": ("mixer", mixer),
                 "mixer_post_norm": ("norm", norm(p + "norm1b"))}
        if layer.get("mlp") is not None:
            parts["feed_forward_norm"] = ("norm", norm(p + "norm2"))
            parts["feed_forward"] = ("feed_forward", _feed_forward(cfg, i, layer["mlp"]))
            parts["feed_forward_post_norm"] = ("norm", norm(p + "norm2b"))
        else:
            # a layer without feed-forward has no use for its second pair of norms: a file that stores them loads
            ignorable += [p + "norm2", p + "norm2b"]
        blocks.append(BlockSpec(parts, "pre_post_norm"))
        mixes.append(PartSpec("depth_weighted", {"count": i + 2}, {"weights": p + "dwa"}))
    schedule = [LayerCall(block=i, cache=i, writes_cache=True, stream_mix=i) for i in range(len(cfg.layers))]
    return ModelSpec(
        architecture=cfg.architecture, hidden_size=W, vocab_size=cfg.vocab, max_position=None,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": W,
                                               "scale": float(cfg.embedding["scale"])}, {"weight": "embed"}),
        positions=positions, blocks=blocks, schedule=schedule, final_norm=norm("final.norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": W}, {"weight": "head"}),
        ignorable=ignorable, stream_mixes=mixes)


register_architecture("Safilorn", SafilornConfig, build_spec)
