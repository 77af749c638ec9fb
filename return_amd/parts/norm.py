"""RMSNorm over the last axis, with the residual addition folded in.

y = x * rsqrt(mean(x^2) + eps) * (offset + w), all in 32-bit, rounded to the
compute dtype after the weight multiply: rollout/fused.py:6-17. Qwen3 uses
offset 0.0 (rollout/monkey_patch/qwen3.py:15-17). With params gain g the result is
that times g (a model's last norm whose logits leave times a constant: the constant
is multiplied into the 32-bit weight when the part is built).
"""
from __future__ import annotations

from .registry import register_part
from .runtime import Pair, ScaledRows, unscaled


class RMSNorm:
    takes_slabs = True          # forward's delta may be Slabs (the kernel set's add_rmsnorm adds them up)

    @staticmethod
    def tensor_shapes(params):
        return {"weight": (params["size"],)}

    @staticmethod
    def random_init(params, role):
        offset = float(params.get("offset", 0.0))
        if offset == 0.0:
            return "norm"
        # a weight stored as its distance from `offset`: drawn so that offset + w lies around one

        def draw(shape, gen):
            import torch
            return (1.0 - offset) + 0.1 * torch.randn(*shape, generator=gen, dtype=torch.float32, device=gen.device)
        return draw

    def __init__(self, params, tensors, rt, shared=None):
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.offset = float(params.get("offset", 0.0))
        self.rt = rt
        w = rt.vector32(tensors["weight"])
        self.weight = w + self.offset if self.offset != 0.0 else w
        self.gain = float(params.get("gain", 1.0))
        if self.gain != 1.0:
            self.weight = (self.weight * self.gain).contiguous()

    def forward(self, h, delta=None, out_rows=None):
        """h (fp32 [T, size]) += delta in place; returns norm(h) (only rows out_rows, if given)."""
        if isinstance(delta, ScaledRows):
            # the product before has added its result into h and left this norm's rows unfinished:
            # the next product applies 1/rms itself
            if delta.norm is not self or out_rows is not None:
                raise ValueError("rows prepared for another norm, or for all rows where some are wanted")
            return delta
        if isinstance(delta, Pair):
            # two outputs that both enter the stream: the first is added by a kernel of its own
            self.rt.ops.residual_add(h, delta.first)
            delta = delta.second
        rows = h.shape[0] if out_rows is None else out_rows.shape[0]
        out = self.rt.empty(rows, self.size)
        delta, factor = unscaled(delta)
        if factor != 1.0:
            self.rt.ops.add_rmsnorm(h, delta, self.weight, self.eps, out, out_rows, delta_scale=factor)
        else:
            self.rt.ops.add_rmsnorm(h, delta, self.weight, self.eps, out, out_rows)
        return out


class Factor:
    """A constant that an arrangement multiplies a sublayer's output by before it enters the stream
    (params["factor"]); it has no tensors."""

    @staticmethod
    def tensor_shapes(params):
        return {}

    def __init__(self, params, tensors, rt, shared=None):
        self.factor = float(params["factor"])


register_part("norm", "rms_norm", RMSNorm)
register_part("norm", "factor", Factor)
