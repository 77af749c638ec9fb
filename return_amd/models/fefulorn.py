"""Fefulorn as a ModelSpec: a decoder whose layers are described one by one in config.json.

A layer runs its two sublayers side by side on the same stream, each behind a norm of its own:
h += mixer(norm1(h)) + ff(norm2(h)), the feed-forward optional. The mixer is a grouped attention with biases on
q, k and v, a rotation over the first elements of a head with linearly stretched positions, a sliding window and
values that may be blended with those of the first such layer; an attention over a latent row per token with a
sliding window and no positions; or a state-space layer with a scalar decay per head and token. The feed-forward
is a mixture of experts with clamped activations, a softmax router whose experts form groups, and a shared
expert behind a gate of its own. The embedding's rows enter the stream times embedding.scale, the logits leave
times logit_scale. Tensor names: "embed", "final.norm", "head", and "l<i>." + norm1, norm2, mix.*, mlp.*.
"""
from __future__ import annotations

from ..config.base import register_architecture
from ..config.fefulorn import FefulornConfig
from ..parts.moe import GroupedRoutedExperts
from ..parts.spec import BlockSpec, LayerCall, ModelSpec, PartSpec

VALUE_ROWS = "first_values"        # the shared part through which the first blending layer hands its values on


def _attention(cfg, i, m, positions, first_blend):
    p = f"l{i}.mix."
    heads, dim = int(m["heads"]), int(m["dim"])
    rot = m.get("rot")
    position = None
    if rot is not None and int(rot.get("dims") or 0):
        factor = float((rot.get("scaling") or {}).get("factor", 1.0))
        position = f"rotary_{dim}_{int(rot['dims'])}_{float(rot['base'])!r}_{factor!r}"
        positions.setdefault(position, PartSpec("rotary", {
            "head_dim": dim, "rotary_dim": int(rot["dims"]), "theta": float(rot["base"]), "max_position": None,
            "exact_tables": True, "linear_factor": factor}))
    blends = bool(m.get("v_mix"))
    if blends:
        positions.setdefault(VALUE_ROWS, PartSpec("token_rows", {}))
    params = {"hidden_size": cfg.width, "num_heads": heads, "num_kv_heads": int(m.get("kv_heads") or heads),
              "head_dim": dim, "value_dim": int(m.get("vdim") or dim), "scale": float(m["scale"]),
              "window": int(m["mask"]["size"]) if m.get("mask") else None, "position": position,
              "value_rows": VALUE_ROWS if blends else None, "first_of_blend": blends and i == first_blend}
    tensors = {"q_proj": p + "q", "q_bias": p + "q.b", "k_proj": p + "k", "k_bias": p + "k.b", "v_proj": p + "v",
               "v_bias": p + "v.b", "o_proj": p + "o"}
    if blends:
        tensors["blend"] = p + "vmix"
    return PartSpec("blend_attention", params, tensors)


def _latent_attention(cfg, i, m):
    p = f"l{i}.mix."
    params = {"hidden_size": cfg.width, "num_heads": int(m["heads"]), "head_dim": int(m["dim"]), "rot_dim": 0,
              "value_dim": int(m["vdim"]), "q_rank": int(m["q_rank"]) if m.get("q_rank") else None,
              "kv_rank": int(m["kv_rank"]), "scale": float(m["scale"]), "eps": float(cfg.norm["eps"]),
              "position": None, "sink": False, "gate": False,
              "window": int(m["mask"]["size"]) if m.get("mask") else None}
    tensors = {"dq": p + "dq", "dq_norm": p + "dq.norm", "uq": p + "uq", "dkv": p + "dkv", "dkv_norm": p + "dkv.norm",
               "uk": p + "uk", "uv": p + "uv", "o": p + "o"}
    return PartSpec("latent_attention", params, tensors)


def _state_space(cfg, i, m):
    p = f"l{i}.mix."
    params = {"hidden_size": cfg.width, "num_heads": int(m["heads"]), "value_dim": int(m["vdim"]),
              "state_dim": int(m["state"]), "groups": int(m["groups"]), "norm_groups": int(m["norm_groups"]),
              "conv_taps": int(m["conv"]), "eps": float(cfg.norm["eps"])}
    tensors = {"in_proj": p + "in", "conv": p + "conv", "conv_bias": p + "conv.b", "dt_bias": p + "dt_bias",
               "A_log": p + "A_log", "skip": p + "D", "o_norm": p + "norm", "o_proj": p + "o"}
    return PartSpec("scalar_state_space", params, tensors)


def _feed_forward(cfg, i, mlp):
    p = f"l{i}.mlp."
    r = mlp["router"]
    groups = r.get("groups") or {}
    count = int(groups.get("count", 1))
    params = {"hidden_size": cfg.width, "expert_size": int(mlp["expert"]["ff"]), "experts": int(r["experts"]),
              "top": int(r["top"]), "groups": count, "keep": int(groups.get("keep") or count),
              "router": "softmax_groups", "activation": "clamped", "limit": float(mlp["expert"]["limit"]), "slope": 1.702}
    tensors = GroupedRoutedExperts.tensor_names(p, int(r["experts"]))
    del tensors["correction"]
    if mlp.get("shared") is not None:
        params["shared"] = {"size": int(mlp["shared"]["ff"]), "limit": float(mlp["shared"]["limit"])}
        tensors.update({"shared_gate": p + "shared.gate", "shared_up": p + "shared.up", "shared_down": p + "shared.down",
                        "shared_weight": p + "shared.sg"})
    return PartSpec("routed_experts", params, tensors)


def build_spec(cfg: FefulornConfig) -> ModelSpec:
    W, eps = cfg.width, float(cfg.norm["eps"])
    norm = lambda name, **kw: PartSpec("rms_norm", {"size": W, "eps": eps, **kw}, {"weight": name})
    positions, blocks, ignorable = {}, [], []
    blending = [i for i, layer in enumerate(cfg.layers) if layer["type"] == "attention" and layer["mixer"].get("v_mix")]
    first_blend = blending[0] if blending else None
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        m = layer["mixer"]
        if layer["type"] == "attention":
            mixer = _attention(cfg, i, m, positions, first_blend)
            if not m.get("v_mix"):
                ignorable.append(p + "mix.vmix")          # a layer that does not blend has no use for the weight
        elif layer["type"] == "latent_attention":
            mixer = _latent_attention(cfg, i, m)
        else:
            mixer = _state_space(cfg, i, m)
        parts = {"mixer_norm": ("norm", norm(p + "norm1")), "mixer": ("mixer", mixer)}
        if layer.get("mlp") is not None:
            parts["feed_forward_norm"] = ("norm", norm(p + "norm2"))
            parts["feed_forward"] = ("feed_forward", _feed_forward(cfg, i, layer["mlp"]))
        else:
            ignorable.append(p + "norm2")
        blocks.append(BlockSpec(parts, "parallel_pre_norm"))
    schedule = [LayerCall(block=i, cache=i, writes_cache=True) for i in range(len(cfg.layers))]
    return ModelSpec(
        architecture=cfg.architecture, hidden_size=W, vocab_size=cfg.vocab, max_position=None,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": W,
                                               "scale": float(cfg.embedding["scale"])}, {"weight": "embed"}),
        positions=positions, blocks=blocks, schedule=schedule,
        final_norm=norm("final.norm", gain=float(cfg.logit_scale)),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": W}, {"weight": "head"}),
        ignorable=ignorable)


register_architecture("Fefulorn", FefulornConfig, build_spec)
