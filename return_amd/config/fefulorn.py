"""Configuration of the Fefulorn decoder, read from its config.json keys.

The file names the design under "architecture" and describes every layer by itself:

    vocab, width                      sizes of the embedding and of the residual stream
    embedding.scale                   factor on the embedding's rows as they enter the stream
    norm.eps                          epsilon of every RMS norm
    logit_scale                       factor on the logits (1 unless given)
    layers[i].type                    "attention", "latent_attention" or "mamba2": the layer's mixer
    layers[i].mixer                   attention: heads, kv_heads (heads unless given), dim (a head's query and key),
                                      vdim (a head's value; dim unless given), scale, mask {size} (none: every earlier
                                      key), rot {base, dims, scaling {factor}} (none: no rotation), v_mix (true: the
                                      values are blended with those of the first such layer)
                                      latent_attention: heads, dim, vdim, kv_rank, q_rank (may be left to the stored
                                      tensors), scale, mask {size}
                                      mamba2: heads, vdim, state, groups, norm_groups, conv (taps)
    layers[i].mlp                     {"kind": "moe", "expert": {"ff", "limit"}, "router": {"experts", "top",
                                      "groups": {"count", "keep"}}, "shared": {"ff", "limit"}} (groups and shared
                                      optional), or null for a layer without feed-forward
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, List

from .base import ConfigError, ModelConfig

MIXERS = ("attention", "latent_attention", "mamba2")


def _int(where: str, d: dict, key: str, least: int = 1) -> int:
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)) or float(v) != int(v) or int(v) < least:
        raise ConfigError(f"Fefulorn: {where}.{key} must be an integer of at least {least}, got {v!r}")
    return int(v)


def _float(where: str, d: dict, key: str, positive: bool = False) -> float:
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (positive and not float(v) > 0):
        raise ConfigError(f"Fefulorn: {where}.{key} must be a{' positive' if positive else ''} number, got {v!r}")
    return float(v)


def _mask(where: str, m: dict):
    mask = m.get("mask")
    if mask is not None:
        _int(where + ".mask", mask, "size")


@dataclasses.dataclass(frozen=True)
class FefulornConfig(ModelConfig):
    vocab: int
    width: int
    layers: List[Dict[str, Any]]
    norm: Dict[str, Any]
    embedding: Dict[str, Any] = dataclasses.field(default_factory=lambda: {"scale": 1.0})
    logit_scale: float = 1.0

    def validate(self, raw):
        if self.vocab < 1 or self.width < 1:
            raise ConfigError(f"Fefulorn: vocab {self.vocab} and width {self.width} must be positive")
        _float("norm", self.norm, "eps")
        _float("embedding", self.embedding, "scale")
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("Fefulorn: layers must be a list with at least one layer")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict) or layer.get("type") not in MIXERS:
                raise ConfigError(f"Fefulorn: {where}.type must be one of {MIXERS}, got "
                                  f"{layer.get('type') if isinstance(layer, dict) else layer!r}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"Fefulorn: {where}.mixer must be a dictionary")
            w = where + ".mixer"
            heads = _int(w, m, "heads")
            if layer["type"] == "attention":
                dim = _int(w, m, "dim")
                if m.get("vdim") is not None:
                    _int(w, m, "vdim")
                kv = _int(w, m, "kv_heads") if m.get("kv_heads") is not None else heads
                if heads % kv:
                    raise ConfigError(f"Fefulorn: {w}: {heads} heads are not a multiple of {kv} kv_heads")
                _float(w, m, "scale", positive=True)
                _mask(w, m)
                rot = m.get("rot")
                if rot is not None and int(rot.get("dims") or 0):
                    dims = _int(w + ".rot", rot, "dims", 2)
                    if dims % 2 or dims > dim or _float(w + ".rot", rot, "base") <= 0:
                        raise ConfigError(f"Fefulorn: {w}.rot: dims {dims} must be even and at most dim {dim}, base positive")
                    if rot.get("scaling") is not None:
                        _float(w + ".rot.scaling", rot["scaling"], "factor", positive=True)
                if not isinstance(m.get("v_mix", False), bool):
                    raise ConfigError(f"Fefulorn: {w}.v_mix must be true or false")
            elif layer["type"] == "latent_attention":
                for key in ("dim", "vdim", "kv_rank"):
                    _int(w, m, key)
                if m.get("q_rank") is not None:
                    _int(w, m, "q_rank")
                _float(w, m, "scale", positive=True)
                _mask(w, m)
            else:
                for key in ("vdim", "state", "groups", "norm_groups", "conv"):
                    _int(w, m, key)
                if heads % int(m["groups"]) or (heads * int(m["vdim"])) % int(m["norm_groups"]):
                    raise ConfigError(f"Fefulorn: {w}: {heads} heads of {m['vdim']} in {m['groups']} groups, normed in "
                                      f"{m['norm_groups']} parts")
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if not isinstance(mlp, dict) or mlp.get("kind", "moe") != "moe":
                raise ConfigError(f"Fefulorn: {where}.mlp.kind must be 'moe' (or mlp null), got {mlp!r}")
            _int(where + ".mlp.expert", mlp.get("expert"), "ff")
            _float(where + ".mlp.expert", mlp.get("expert"), "limit", positive=True)
            r = mlp.get("router")
            experts, top = _int(where + ".mlp.router", r, "experts"), _int(where + ".mlp.router", r, "top")
            count = keep = 1
            if r.get("groups") is not None:
                count = _int(where + ".mlp.router.groups", r["groups"], "count")
                keep = _int(where + ".mlp.router.groups", r["groups"], "keep") if r["groups"].get("keep") is not None else count
            if experts % count or keep > count or top > keep * (experts // count):
                raise ConfigError(f"Fefulorn: {where}.mlp.router: top {top} of {experts} experts in {count} groups of "
                                  f"which {keep} stay")
            if mlp.get("shared") is not None:
                _int(where + ".mlp.shared", mlp["shared"], "ff")
                _float(where + ".mlp.shared", mlp["shared"], "limit", positive=True)

    def to_dict(self):
        out = {"architecture": self.architecture}
        for f in dataclasses.fields(self):
            if f.name != "architecture" and getattr(self, f.name) is not None:
                out[f.name] = getattr(self, f.name)
        return out
