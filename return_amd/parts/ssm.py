"""State-space mixer with one decay per head and token: the memory is a matrix S [N, P] per head and request.

With H heads of P channels, a state of N per head, G groups of heads that share B and C, and inner = H P:
    [z | x | B | C | dt] = W_in h                    z, x: inner; B, C: G N; dt: H
    x, B, C  <- silu(causal conv over time, a filter and a bias per channel)
    delta    = softplus(dt + dt_bias)                one per head and token, no clamp
    S        <- exp(-exp(A_log[h]) delta) S + delta B x^T;   y = S^T C + skip[h] x      (head h reads group h // (H / G))
    out      = W_o (rmsnorm over each of `norm_groups` equal parts of (y * silu(z)), times a weight per channel)
The step size, the decay, the state and the norm are 32-bit. Kept between steps per request: the last taps-1 inputs
of the convolution and S.

It is the outer-product memory of a linear attention with k = delta B, v = x, q = C and a decay that is the same
for every row of S, and runs on the recurrence kernels of the delta rule (rule "scalar"): the state has the same
layout, [slot, head, P, N]. The rows of W_in and the convolution's channels are put into the order [C | B | x] when
the part is built, which is the order [q | k | v] that those kernels read.
Parameters: hidden_size, num_heads, value_dim (P), state_dim (N), groups, norm_groups, conv_taps, eps.
"""
from __future__ import annotations

import torch

from ..cache.spec import StateSpec
from .delta import _a_log_init, _dt_bias_init
from .registry import register_part


class ScalarStateSpace:
    @staticmethod
    def tensor_shapes(params):
        W, H, P, N, G = (params["hidden_size"], params["num_heads"], params["value_dim"], params["state_dim"],
                         params["groups"])
        inner, taps = H * P, params["conv_taps"]
        return {"in_proj": (2 * inner + 2 * G * N + H, W), "conv": (inner + 2 * G * N, taps),
                "conv_bias": (inner + 2 * G * N,), "dt_bias": (H,), "A_log": (H,), "skip": (H,), "o_norm": (inner,),
                "o_proj": (W, inner)}

    @staticmethod
    def random_init(params, role):
        if role == "conv":
            return lambda shape, gen: 0.3 * torch.randn(*shape, generator=gen, dtype=torch.float32, device=gen.device)
        if role == "conv_bias":
            return lambda shape, gen: 0.1 * torch.randn(*shape, generator=gen, dtype=torch.float32, device=gen.device)
        if role == "skip":
            return lambda shape, gen: 1.0 + 0.2 * torch.randn(*shape, generator=gen, dtype=torch.float32, device=gen.device)
        return {"A_log": _a_log_init, "dt_bias": _dt_bias_init, "o_norm": "norm"}.get(role, "matrix")

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        W = int(params["hidden_size"])
        self.H, self.P, self.N = int(params["num_heads"]), int(params["value_dim"]), int(params["state_dim"])
        self.G, self.parts = int(params["groups"]), int(params["norm_groups"])
        self.taps, self.eps = int(params["conv_taps"]), float(params["eps"])
        H, P, N, G = self.H, self.P, self.N, self.G
        self.inner = inner = H * P
        if H % G or inner % self.parts:
            raise ValueError(f"{H} heads of {P} in {G} groups, normed in {self.parts} parts")
        if hasattr(rt.ops, "delta_rule_fits") and not rt.ops.delta_rule_fits(N, P):
            raise ValueError(f"heads of {N} x {P} are beyond the recurrence kernel")
        self.c_conv = 2 * G * N + inner
        # stored order of the conv's channels [x | B | C] -> [C | B | x]
        order = torch.cat([torch.arange(inner + G * N, inner + 2 * G * N), torch.arange(inner, inner + G * N),
                           torch.arange(0, inner)])
        w_in = rt.matrix(tensors["in_proj"])

        def padded(m):
            pad = -m.shape[0] % 16
            return m if not pad else torch.cat([m, torch.zeros(pad, W, dtype=rt.dtype, device=rt.device)], dim=0)
        conv_rows = padded(w_in[inner:inner + self.c_conv][order.to(w_in.device)])
        gate_rows = padded(w_in[:inner])
        dt_rows = padded(w_in[inner + self.c_conv:])
        self.at_gate, self.at_dt = conv_rows.shape[0], conv_rows.shape[0] + gate_rows.shape[0]
        # x goes into one product: [C | B | x | z | dt], each piece filled up to a multiple of 16 rows
        self.w_in = rt.product(torch.cat([conv_rows, gate_rows, dt_rows], dim=0).contiguous())
        self.w_conv = rt.vector32(tensors["conv"])[order.to(rt.device)].contiguous()
        self.conv_bias = rt.vector32(tensors["conv_bias"])[order.to(rt.device)].contiguous()
        self.a_log, self.dt_bias, self.skip = (rt.vector32(tensors[n]) for n in ("A_log", "dt_bias", "skip"))
        self.w_norm = rt.vector32(tensors["o_norm"])
        self.w_o = rt.product(rt.matrix(tensors["o_proj"]))

    def cache_spec(self):
        return StateSpec((("conv", (self.taps - 1, self.c_conv), self.rt.dtype_name),
                          ("S", (self.H, self.P, self.N), "float32")))      # S column by column

    def forward(self, x, step, cache, write_cache=True):
        rt, ops = self.rt, self.rt.ops
        if not write_cache:
            raise ValueError("a state-space mixer advances its state with every call; it cannot only read it")
        T = x.shape[0]
        z = ops.linear(x, self.w_in)                                           # [T, C | B | x | gate | dt]
        qkv = rt.empty(T, self.c_conv)
        ops.causal_conv(z[:, :self.c_conv], self.w_conv, cache.tensors["conv"], step, qkv, silu=True, bias=self.conv_bias)
        o = rt.empty(T, self.inner)
        ops.scalar_rule(qkv, z[:, self.at_dt:self.at_dt + self.H], self.a_log, self.dt_bias, self.skip,
                        z[:, self.at_gate:self.at_gate + self.inner], self.w_norm, self.parts, self.eps,
                        cache.tensors["S"], step, o, self.H, self.G, self.N, self.P)
        return ops.linear(o, self.w_o)


register_part("mixer", "scalar_state_space", ScalarStateSpace)
