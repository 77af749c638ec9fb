"""Configuration of the Safilorn decoder, read from its config.json keys.

The file names the design under "architecture" and describes every layer by itself:

    vocab, width                      sizes of the embedding and of the residual stream
    embedding.scale                   factor on the embedding's rows as they enter the stream
    norm.eps                          epsilon of every RMS norm
    layers[i].type                    "latent_attention" or "gla": the layer's mixer
    layers[i].mixer                   latent_attention: heads, dim (unrotated part of a head's query and key),
                                      rot_dim (rotated part), vdim, kv_rank and q_rank (sizes of the two latents;
                                      q_rank may be left to the stored tensors), scale, rot {base, dims, scaling {factor, original, fast, slow}}
                                      gla: heads, dim, vdim, tau (the decay is sigmoid(z)^(1/tau)); the rank of
                                      the decay's two-factor map is what the stored tensors have
    layers[i].mlp                     {"kind": "dense", "ff"}, {"kind": "moe", "expert": {"ff", "limit"},
                                      "router": {"experts", "top"}}, or null for a layer without feed-forward
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, List

from .base import ConfigError, ModelConfig

MIXERS = ("latent_attention", "gla")


def _int(where: str, d: dict, key: str, least: int = 1) -> int:
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)) or float(v) != int(v) or int(v) < least:
        raise ConfigError(f"Safilorn: {where}.{key} must be an integer of at least {least}, got {v!r}")
    return int(v)


def _float(where: str, d: dict, key: str, positive: bool = False) -> float:
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (positive and not float(v) > 0):
        raise ConfigError(f"Safilorn: {where}.{key} must be a{' positive' if positive else ''} number, got {v!r}")
    return float(v)


@dataclasses.dataclass(frozen=True)
class SafilornConfig(ModelConfig):
    vocab: int
    width: int
    layers: List[Dict[str, Any]]
    norm: Dict[str, Any]
    embedding: Dict[str, Any] = dataclasses.field(default_factory=lambda: {"scale": 1.0})

    def validate(self, raw):
        if self.vocab < 1 or self.width < 1:
            raise ConfigError(f"Safilorn: vocab {self.vocab} and width {self.width} must be positive")
        _float("norm", self.norm, "eps")
        _float("embedding", self.embedding, "scale")
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("Safilorn: layers must be a list with at least one layer")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict) or layer.get("type") not in MIXERS:
                raise ConfigError(f"Safilorn: {where}.type must be one of {MIXERS}, got "
                                  f"{layer.get('type') if isinstance(layer, dict) else layer!r}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"Safilorn: {where}.mixer must be a dictionary")
            w = where + ".mixer"
            for key in ("heads", "dim", "vdim"):
                _int(w, m, key)
            if layer["type"] == "latent_attention":
                rot_dim = _int(w, m, "rot_dim", 2)
                if m.get("q_rank") is not None:
                    _int(w, m, "q_rank")
                _int(w, m, "kv_rank")
                _float(w, m, "scale")
                rot = m.get("rot")
                dims = _int(w + ".rot", rot, "dims", 2)
                if dims % 2 or dims > rot_dim or _float(w + ".rot", rot, "base") <= 0:
                    raise ConfigError(f"Safilorn: {w}.rot: dims {dims} must be even and at most rot_dim {rot_dim}, base positive")
                if rot.get("scaling") is not None:
                    for key in ("factor", "original", "fast", "slow"):
                        _float(w + ".rot.scaling", rot["scaling"], key, positive=True)
            else:
                _float(w, m, "tau", positive=True)
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
                raise ConfigError(f"Safilorn: {where}.mlp.kind must be 'dense' or 'moe' (or mlp null), got {mlp!r}")
            if mlp["kind"] == "dense":
                _int(where + ".mlp", mlp, "ff")
            else:
                _int(where + ".mlp.expert", mlp.get("expert"), "ff")
                _float(where + ".mlp.expert", mlp.get("expert"), "limit", positive=True)
                r = mlp.get("router")
                experts, top = _int(where + ".mlp.router", r, "experts"), _int(where + ".mlp.router", r, "top")
                if top > experts:
                    raise ConfigError(f"Safilorn: {where}.mlp.router: top {top} of {experts} experts")

    def to_dict(self):
        out = {"architecture": self.architecture}
        for f in dataclasses.fields(self):
            if f.name != "architecture" and getattr(self, f.name) is not None:
                out[f.name] = getattr(self, f.name)
        return out
