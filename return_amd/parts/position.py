"""Rotary position encoding, half-split pairing (or, with pairing "interleaved", element 2i with 2i + 1).

x1 = x[:R/2], x2 = x[R/2:R]; o1 = x1*cos - x2*sin, o2 = x2*cos + x1*sin in 32-bit;
dimensions from R on pass through: rollout/attention.py:10-25, rollout/fused.py:59-83.
Angles are position * inv_freq with inv_freq[j] = theta^(-2j/R), and the tables are
cos and sin of them times attention_scaling: rollout/monkey_patch/qwen3.py:121-127
(the reference stores the tables in bf16; here they stay 32-bit).

With params scaling {factor, original, fast, slow} the frequencies are stretched for contexts beyond `original`
positions (the rule known as YaRN): pair i makes original * f_i / (2 pi) turns over the original context; with
d(t) = R ln(original / (2 pi t)) / (2 ln theta) the pair that makes t turns, pairs up to lo = max(floor(d(fast)), 0)
keep their frequency, pairs from hi = min(ceil(d(slow)), R - 1) on turn `factor` times slower, the ones between
are blended linearly, f_i (1 - r_i) + f_i / factor r_i with r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), and
cos and sin are multiplied by 0.1 ln(factor) + 1.

With params linear_factor s every frequency is divided by s (positions stretched linearly: the angle of pair i is
position * theta^(-2i/R) / s).
"""
from __future__ import annotations

import math

import torch

from .registry import register_part


class RotaryPosition:
    @staticmethod
    def tensor_shapes(params):
        return {}

    def __init__(self, params, tensors, rt, shared=None):
        self.head_dim = int(params["head_dim"])
        self.rotary_dim = int(params.get("rotary_dim", self.head_dim))
        self.theta = float(params["theta"])
        # which elements form a pair: "half" (i with i + R/2) or "interleaved" (2i with 2i + 1); the same
        # angle table serves both, pair i turns by position * theta^(-2i/R)
        self.pairing = params.get("pairing", "half")
        if self.pairing not in ("half", "interleaved"):
            raise ValueError(f"rotary pairing {self.pairing!r}: 'half' or 'interleaved'")
        # no limit of the model's own: as many positions as the engine's cache can hold for one request
        limit = params.get("max_position")
        self.max_position = int(limit if limit is not None else getattr(rt, "position_limit", 0) or 0)
        if self.max_position < 1:
            raise ValueError("rotary positions: neither the model nor the engine says how many positions there are")
        self.scaling = float(params.get("attention_scaling", 1.0))
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {self.head_dim}")
        self.rt = rt
        half = self.rotary_dim // 2
        stretch = params.get("scaling")
        linear = float(params.get("linear_factor") or 1.0)
        if not linear > 0:
            raise ValueError(f"rotary positions: linear_factor {linear} must be positive")
        if linear != 1.0 and (stretch or not params.get("exact_tables")):
            raise ValueError("rotary positions: linearly stretched positions are built for exact_tables without another scaling")
        if stretch:
            if not params.get("exact_tables"):
                raise ValueError("rotary positions: stretched frequencies are built for exact_tables only")
            factor, original = float(stretch["factor"]), float(stretch["original"])
            pair_of = lambda turns: self.rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))
            lo = max(math.floor(pair_of(float(stretch["fast"]))), 0)
            hi = min(math.ceil(pair_of(float(stretch["slow"]))), self.rotary_dim - 1)
            i = torch.arange(0, half, dtype=torch.float64)
            ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
            inv_freq = self.theta ** (-i / half)
            inv_freq = inv_freq / factor * ramp + inv_freq * (1.0 - ramp)
            self.scaling *= 0.1 * math.log(factor) + 1.0
            angle = torch.outer(torch.arange(self.max_position, dtype=torch.float64), inv_freq)
        elif params.get("exact_tables"):
            # frequencies and angles in 64-bit, so that the 32-bit tables are the rounded true values
            inv_freq = self.theta ** (-torch.arange(0, half, dtype=torch.float64) / half) / linear
            angle = torch.outer(torch.arange(self.max_position, dtype=torch.float64), inv_freq)
        else:
            inv_freq = 1.0 / (self.theta ** (torch.arange(0, half, dtype=torch.float32) / half))
            angle = torch.outer(torch.arange(self.max_position, dtype=torch.float32), inv_freq)
        self.cos = (angle.cos() * self.scaling).float().to(rt.device).contiguous()
        self.sin = (angle.sin() * self.scaling).float().to(rt.device).contiguous()

    def tables(self):
        """(cos, sin, rotary_dim): fp32 [max_position, rotary_dim/2] each."""
        return self.cos, self.sin, self.rotary_dim

    def apply(self, q, k, positions):
        """Rotate q and k ([T, heads, D], compute dtype) in place by their tokens' positions."""
        if self.pairing != "half":
            raise NotImplementedError("interleaved pairs are rotated by the mixers that prepare q and k with the tables")
        self.rt.ops.rope(q, positions, self.cos, self.sin, self.rotary_dim)
        if k is not None:
            self.rt.ops.rope(k, positions, self.cos, self.sin, self.rotary_dim)


register_part("position", "rotary", RotaryPosition)
