"""Routed feed-forward: a mixture of small gated feed-forward layers, of which each token uses a few.

Expert e: down_e(silu(gate_e x) * (up_e x)), no biases. Router: z = W_r x in 32-bit, s = sigmoid(z);
the choice is made on s + correction (a stored vector, one entry per expert), the weights use s alone.
Experts form ``groups`` equal groups of neighbours; a group's score is the sum of its two largest
choice scores, and only experts of the ``keep`` best groups can be chosen (groups 1: no such limit).
The ``top`` eligible experts with the largest choice scores are taken; their weights are their s
divided by the sum of those s (+ norm_eps); the output is the weighted sum of their outputs.

Two more laws, by parameter: router "softmax_top" takes the `top` largest logits z = W_r x + b_r (a stored
bias, role router_bias; no groups, no correction) and weighs them by the softmax over those logits alone;
activation "clamped" with `limit` L and `slope` a (1.702 unless given) makes an expert
down(g sigmoid(a g) (u + 1)) with g = min(gate x, L), u = clamp(up x, -L, L).

Router "softmax_groups": s = softmax(z) over all experts; a group's score is its largest s, only experts of the
`keep` best groups can be chosen, the `top` of them with the largest s are taken, and their weights are their s as
they are (no second tensor, nothing is renormed). With params shared {size, limit} one more expert of the same form
(roles shared_gate, shared_up, shared_down; its own width and limit) runs for every token and is added times
sigmoid(w_s . x), one number per token (role shared_weight, [1, H]).

The experts' matrices are kept stacked ([E, 2 I, H] with gate rows first, [E, H, I]); a step's (token,
choice) pairs are grouped by expert on the device and the products run over those groups, so nothing
of a step's routing comes back to the host.
"""
from __future__ import annotations

import torch

from .registry import register_part


class GroupedRoutedExperts:
    @staticmethod
    def tensor_shapes(params):
        H, I, E = params["hidden_size"], params["expert_size"], params["experts"]
        shapes = {"router": (E, H)}
        law = params.get("router", "sigmoid_groups")
        if law == "softmax_top":
            shapes["router_bias"] = (E,)
        elif law != "softmax_groups":
            shapes["correction"] = (E,)
        if params.get("shared"):
            Is = params["shared"]["size"]
            shapes.update({"shared_gate": (Is, H), "shared_up": (Is, H), "shared_down": (H, Is), "shared_weight": (1, H)})
        for e in range(E):
            shapes[f"gate_{e}"] = (I, H)
            shapes[f"up_{e}"] = (I, H)
            shapes[f"down_{e}"] = (H, I)
        return shapes

    @staticmethod
    def tensor_names(prefix, experts, second="correction", second_name="correction"):
        """role -> tensor name for experts stored as <prefix>e<i>.gate / .up / .down beside <prefix>router
        and the router's second tensor (role `second`, stored as <prefix><second_name>)."""
        names = {"router": prefix + "router", second: prefix + second_name}
        for e in range(experts):
            for role in ("gate", "up", "down"):
                names[f"{role}_{e}"] = f"{prefix}e{e}.{role}"
        return names

    @staticmethod
    def random_init(params, role):
        if role in ("correction", "router_bias"):
            return lambda shape, gen: 0.05 * torch.randn(*shape, generator=gen, dtype=torch.float32, device=gen.device)
        if role == "router":
            # logits of order one, so that the choice differs from token to token
            return lambda shape, gen: torch.randn(*shape, generator=gen, dtype=torch.float32,
                                                  device=gen.device) * (2.0 / params["hidden_size"] ** 0.5)
        return "matrix"

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.hidden, self.inter = int(params["hidden_size"]), int(params["expert_size"])
        self.experts, self.top = int(params["experts"]), int(params["top"])
        self.groups, self.keep = int(params.get("groups") or 1), int(params.get("keep") or params.get("groups") or 1)
        self.norm_eps = float(params.get("norm_eps", 1e-20))
        self.law = params.get("router", "sigmoid_groups")
        self.activation = params.get("activation", "silu")
        if self.law not in ("sigmoid_groups", "softmax_top", "softmax_groups") or self.activation not in ("silu", "clamped"):
            raise ValueError(f"routed experts: router {self.law!r}, activation {self.activation!r}")
        self.limit = float(params["limit"]) if self.activation == "clamped" else 0.0
        self.slope = float(params.get("slope", 1.702))
        if self.law == "softmax_top" and self.groups != 1:
            raise ValueError("routed experts: the softmax router has no groups")
        E = self.experts
        if E % self.groups or not 1 <= self.keep <= self.groups or not 1 <= self.top <= self.keep * (E // self.groups):
            raise ValueError(f"routed experts: {E} experts in {self.groups} groups, {self.keep} kept, top {self.top}")
        if hasattr(rt.ops, "check_moe_sizes"):
            rt.ops.check_moe_sizes(E, self.top, self.groups, self.keep)
        self.w_router = rt.product(rt.matrix(tensors["router"]), out_dtype=torch.float32)
        self.correction = None if self.law == "softmax_groups" else \
            rt.vector32(tensors["router_bias" if self.law == "softmax_top" else "correction"])
        self.w_gate_up = torch.stack([torch.cat([rt.matrix(tensors[f"gate_{e}"]), rt.matrix(tensors[f"up_{e}"])], dim=0)
                                      for e in range(E)]).contiguous()                  # [E, 2I, H]
        self.w_down = torch.stack([rt.matrix(tensors[f"down_{e}"]) for e in range(E)]).contiguous()   # [E, H, I]
        self.shared = None
        if params.get("shared"):
            if self.activation != "clamped":
                raise ValueError("routed experts: the shared expert is built for the clamped activation")
            self.shared_size, self.shared_limit = int(params["shared"]["size"]), float(params["shared"]["limit"])
            # [gate; up; the gate's one row], filled up with zero rows to a multiple of 16
            rows = [rt.matrix(tensors["shared_gate"]), rt.matrix(tensors["shared_up"]), rt.matrix(tensors["shared_weight"])]
            pad = -sum(r.shape[0] for r in rows) % 16
            if pad:
                rows.append(torch.zeros(pad, self.hidden, dtype=rt.dtype, device=rt.device))
            self.shared = rt.product(torch.cat(rows, dim=0).contiguous())
            self.shared_down = rt.product(rt.matrix(tensors["shared_down"]))

    def forward(self, x, step=None):
        ops = self.rt.ops
        z = ops.linear(x, self.w_router, out_dtype=torch.float32)                        # [T, E]
        if self.law == "softmax_top":
            ids, weights = ops.moe_route(z, self.correction, self.top, 1, 1, 0.0, law="softmax_top")
        elif self.law == "softmax_groups":
            ids, weights = ops.moe_route(z, None, self.top, self.groups, self.keep, 0.0, law="softmax_groups")
        else:
            ids, weights = ops.moe_route(z, self.correction, self.top, self.groups, self.keep, self.norm_eps)
        if self.activation == "clamped":
            if self.shared is not None:
                # the shared expert first; the kernel that sums a token's experts adds it behind its gate
                Is = self.shared_size
                gu = ops.linear(x, self.shared)                                          # [T, gate | up | weight | pad]
                a = self.rt.empty(x.shape[0], Is)
                ops.clamped_mul(gu, a, self.shared_limit, self.slope)
                return ops.moe_experts(x, ids, weights, self.w_gate_up, self.w_down, activation="clamped", limit=self.limit,
                                       slope=self.slope, extra=ops.linear(a, self.shared_down),
                                       extra_logits=gu[:, 2 * Is:2 * Is + 1])
            return ops.moe_experts(x, ids, weights, self.w_gate_up, self.w_down, activation="clamped", limit=self.limit,
                                   slope=self.slope)
        return ops.moe_experts(x, ids, weights, self.w_gate_up, self.w_down)


register_part("feed_forward", "grouped_routed_experts", GroupedRoutedExperts)
register_part("feed_forward", "routed_experts", GroupedRoutedExperts)
