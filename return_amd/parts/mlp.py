"""SwiGLU feed-forward: down(silu(gate(x)) * up(x)); with params bias, every projection has a bias
(roles gate_bias, up_bias, down_bias), added in 32-bit before the activation and after the last product.

rollout/monkey_patch/qwen3.py:20-22 with gate and up fused into one weight, gate
rows first (qwen3.py:99-105); silu(g) * u in 32-bit: rollout/fused.py:103-114.
"""
from __future__ import annotations

import torch

from .registry import register_part


class SwiGLU:
    @staticmethod
    def tensor_shapes(params):
        H, I = params["hidden_size"], params["intermediate_size"]
        shapes = {"gate_proj": (I, H), "up_proj": (I, H), "down_proj": (H, I)}
        if params.get("bias"):
            shapes.update({"gate_bias": (I,), "up_bias": (I,), "down_bias": (H,)})
        return shapes

    @staticmethod
    def random_init(params, role):
        return "matrix"

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.inter = int(params["intermediate_size"])
        self.bias_in = self.bias_out = None
        if params.get("bias"):
            self.bias_in = torch.cat([rt.vector32(tensors["gate_bias"]), rt.vector32(tensors["up_bias"])]).contiguous()
            self.bias_out = rt.vector32(tensors["down_bias"])
        self.w_gate_up = rt.product(torch.cat([rt.matrix(tensors["gate_proj"]), rt.matrix(tensors["up_proj"])],
                                              dim=0).contiguous(), gated=self.bias_in is None)
        self.w_down = rt.product(rt.matrix(tensors["down_proj"]), residual=self.bias_out is None)
        if self.bias_in is None:
            self.first_product = (self.w_gate_up, True)        # (see PagedAttention)
            self.last_product = self.w_down

    def forward(self, x, step=None, sink=None):
        ops = self.rt.ops
        if self.bias_in is not None:
            gu = ops.linear(x, self.w_gate_up)             # [T, 2 I], gate columns first
            a = self.rt.empty(x.shape[0], self.inter)
            ops.silu_mul(gu, a, bias=self.bias_in)         # silu(gate + b_g) * (up + b_u)
            return ops.add_bias(ops.linear(a, self.w_down), self.bias_out)
        a = ops.linear_silu_mul(x, self.w_gate_up)         # [T, I] = silu(gate) * up, gate rows first
        return sink.project(a, self.w_down) if sink is not None else ops.linear(a, self.w_down)


register_part("feed_forward", "swiglu", SwiGLU)


class SquaredReLU:
    """Dense feed-forward down(relu(up(x))^2), no biases."""

    @staticmethod
    def tensor_shapes(params):
        H, I = params["hidden_size"], params["intermediate_size"]
        return {"up_proj": (I, H), "down_proj": (H, I)}

    @staticmethod
    def random_init(params, role):
        return "matrix"

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.w_up = rt.product(rt.matrix(tensors["up_proj"]))
        self.w_down = rt.product(rt.matrix(tensors["down_proj"]))

    def forward(self, x, step=None):
        ops = self.rt.ops
        return ops.linear(ops.relu_sq(ops.linear(x, self.w_up)), self.w_down)


register_part("feed_forward", "relu2", SquaredReLU)
