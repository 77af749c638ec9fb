"""Gated delta rule with a decay per key channel: a mixer whose memory is a matrix S [D, V] per head,
of fixed size whatever the sequence's length.

For head h with its q/k head h // (heads / kv_heads), token by token:
    q, k, v    = silu(short causal conv(W_q x)), ... (one filter per channel, taps from the config)
    q, k       <- unit vectors per head, x / sqrt(sum x^2 + 1e-6); q also times D^-1/2
    beta       = sigmoid(W_b x)                                   one per head
    g          = exp(-exp(A_log[h]) * softplus(W_a2 (W_a1 x) + dt_bias))    one per head and key channel
    S          <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
    y          = W_o (o / rms(o) * w_norm * sigmoid(W_g2 (W_g1 x)))        rms over the head's V, w_norm [V]
Everything from the unit vectors to the norm of o is 32-bit. Kept between steps per request: the
last taps-1 inputs of the three convolutions and S.

Three products in front: q, k, v and b as one (the weights stacked, rows padded to a multiple of
16), the first factors of the two low-rank maps as one, and their second factors as one (a matrix of
two blocks on its diagonal); the convolution reads its columns of the first result in place, the
recurrence kernels read the rest.
"""
from __future__ import annotations

import torch

from ..cache.spec import StateSpec
from .conv import filter_init
from .registry import register_part

DEFAULT_RANK = 16


def _a_log_init(shape, generator):
    """Logarithm of a decay rate: log of U(0.02, 1)."""
    return torch.log(0.02 + 0.98 * torch.rand(*shape, generator=generator, dtype=torch.float32, device=generator.device))


def _dt_bias_init(shape, generator):
    """Bias of the decay's step size: U(-4, -1), so that softplus starts small and the memory long."""
    return -4.0 + 3.0 * torch.rand(*shape, generator=generator, dtype=torch.float32, device=generator.device)


class ChannelDeltaMixer:
    @staticmethod
    def tensor_shapes(params):
        W, H, G, D, V = (params["hidden_size"], params["num_heads"], params["num_kv_heads"], params["head_dim"],
                         params["value_dim"])
        taps = params["conv_taps"]
        ra, rg = params.get("decay_rank"), params.get("gate_rank")      # None: whatever the stored tensor has
        return {"q_proj": (G * D, W), "k_proj": (G * D, W), "v_proj": (H * V, W),
                "q_conv": (G * D, taps), "k_conv": (G * D, taps), "v_conv": (H * V, taps),
                "b_proj": (H, W), "A_log": (H,), "dt_bias": (H * D,), "o_norm": (V,),
                "a1_proj": (ra, W), "a2_proj": (H * D, ra), "g1_proj": (rg, W), "g2_proj": (H * V, rg),
                "o_proj": (W, H * V)}

    @staticmethod
    def random_init(params, role):
        if role in ("q_conv", "k_conv", "v_conv"):
            return filter_init
        return {"A_log": _a_log_init, "dt_bias": _dt_bias_init, "o_norm": "norm"}.get(role, "matrix")

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.hidden = W = int(params["hidden_size"])
        self.H, self.G = int(params["num_heads"]), int(params["num_kv_heads"])
        self.D, self.V = int(params["head_dim"]), int(params["value_dim"])
        self.taps = int(params["conv_taps"])
        self.eps = float(params["eps"])
        if self.H % self.G:
            raise ValueError(f"{self.H} heads are not a multiple of {self.G} q/k heads")
        self.ra, self.rg = tensors["a1_proj"].shape[0], tensors["g1_proj"].shape[0]
        if tensors["a2_proj"].shape[1] != self.ra or tensors["g2_proj"].shape[1] != self.rg:
            raise ValueError("the two factors of a low-rank map differ in their inner size")
        self.c_conv = 2 * self.G * self.D + self.H * self.V
        if hasattr(rt.ops, "delta_rule_fits") and not rt.ops.delta_rule_fits(self.D, self.V):
            raise ValueError(f"heads of {self.D} x {self.V} are beyond the delta-rule kernel")

        def stacked(rows, width):
            """Matrices one under the other, rows filled up with zeros to a multiple of 16."""
            pad = -sum(r.shape[0] for r in rows) % 16
            if pad:
                rows = rows + [torch.zeros(pad, width, dtype=rt.dtype, device=rt.device)]
            return torch.cat(rows, dim=0).contiguous()

        self.w_in = rt.product(stacked([rt.matrix(tensors[n]) for n in ("q_proj", "k_proj", "v_proj", "b_proj")], W))
        self.w_low = rt.product(stacked([rt.matrix(tensors["a1_proj"]), rt.matrix(tensors["g1_proj"])], W))
        # [a | c] = [a1 | g1 | 0] @ [[A2, 0], [0, G2], [0, 0]]^T: the two second factors as one product
        r_in = self.w_low.shape[0]
        n_a, n_c = self.H * self.D, self.H * self.V
        second = torch.zeros(n_a + n_c, r_in, dtype=rt.dtype, device=rt.device)
        second[:n_a, :self.ra] = rt.matrix(tensors["a2_proj"])
        second[n_a:, self.ra:self.ra + self.rg] = rt.matrix(tensors["g2_proj"])
        self.w_second = rt.product(second)
        self.w_conv = torch.cat([rt.vector32(tensors[n]) for n in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        self.a_log = rt.vector32(tensors["A_log"])
        self.dt_bias = rt.vector32(tensors["dt_bias"])
        self.w_norm = rt.vector32(tensors["o_norm"])
        self.w_o = rt.product(rt.matrix(tensors["o_proj"]))

    def cache_spec(self):
        return StateSpec((("conv", (self.taps - 1, self.c_conv), self.rt.dtype_name),
                          ("S", (self.H, self.V, self.D), "float32")))      # S column by column

    def forward(self, x, step, cache, write_cache=True):
        rt, ops = self.rt, self.rt.ops
        if not write_cache:
            raise ValueError("a delta-rule mixer advances its state with every call; it cannot only read it")
        T = x.shape[0]
        z = ops.linear(x, self.w_in)                                           # [T, q | k | v | b | pad]
        ag = ops.linear(ops.linear(x, self.w_low), self.w_second)              # [T, decay H*D | gate H*V]
        qkv = rt.empty(T, self.c_conv)
        ops.causal_conv(z[:, :self.c_conv], self.w_conv, cache.tensors["conv"], step, qkv, silu=True)
        o = rt.empty(T, self.H * self.V)
        ops.delta_rule(qkv, z[:, self.c_conv:self.c_conv + self.H], ag, self.a_log, self.dt_bias, self.w_norm, self.eps,
                       cache.tensors["S"], step, o, self.H, self.G, self.D, self.V)
        return ops.linear(o, self.w_o)


register_part("mixer", "channel_delta", ChannelDeltaMixer)


class GatedLinearAttention:
    """Linear attention with a decay per key channel: the memory is a matrix S [D, V] per head and request.

        q = W_q x * D^-1/2,  k = W_k x  (heads of D),  v = W_v x  (heads of V)
        alpha = sigmoid(W_a2 (W_a1 x) + b_a)^(1/tau)                   one per head and key channel
        S <- diag(alpha) S + k v^T;  o = S^T q                          (the read-out sees the token's own write)
        y = W_o (rmsnorm_V(o) w_norm * silu(W_g x))                     w_norm [V], the same for every head
    The decay, the state and the read-out's norm are 32-bit. It is the delta rule's recurrence without the
    correction term (u = v), without unit vectors and with another decay law, and runs on the same kernels
    (rule "outer"): the state has the same layout, [slot, head, V, D].
    Parameters: hidden_size, num_heads, head_dim, value_dim, tau, eps, decay_rank (None: what the stored
    tensors have).
    """

    @staticmethod
    def tensor_shapes(params):
        W, H, D, V = params["hidden_size"], params["num_heads"], params["head_dim"], params["value_dim"]
        r = params.get("decay_rank")
        return {"q_proj": (H * D, W), "k_proj": (H * D, W), "v_proj": (H * V, W), "g_proj": (H * V, W),
                "o_proj": (W, H * V), "o_norm": (V,), "a1_proj": (r, W), "a2_proj": (H * D, r), "a2_bias": (H * D,)}

    @staticmethod
    def random_init(params, role):
        if role == "a2_bias":
            # decays near one: sigmoid(U(2, 5))
            return lambda shape, gen: 2.0 + 3.0 * torch.rand(*shape, generator=gen, dtype=torch.float32, device=gen.device)
        return "norm" if role == "o_norm" else "matrix"

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        W = int(params["hidden_size"])
        self.H, self.D, self.V = int(params["num_heads"]), int(params["head_dim"]), int(params["value_dim"])
        self.tau, self.eps = float(params["tau"]), float(params["eps"])
        if not self.tau > 0:
            raise ValueError(f"gated linear attention: tau {self.tau} must be positive")
        if tensors["a2_proj"].shape[1] != tensors["a1_proj"].shape[0]:
            raise ValueError("the two factors of the decay's low-rank map differ in their inner size")
        if hasattr(rt.ops, "delta_rule_fits") and not rt.ops.delta_rule_fits(self.D, self.V):
            raise ValueError(f"heads of {self.D} x {self.V} are beyond the recurrence kernel")
        # x goes into one product: [W_q; W_k; W_v | W_g | W_a1], each piece filled up to a multiple of 16 rows so
        # that the slices begin at aligned columns
        def padded(rows):
            m = torch.cat(rows, dim=0)
            pad = -m.shape[0] % 16
            return m if not pad else torch.cat([m, torch.zeros(pad, W, dtype=rt.dtype, device=rt.device)], dim=0)
        qkv = padded([rt.matrix(tensors[n]) for n in ("q_proj", "k_proj", "v_proj")])
        gate = padded([rt.matrix(tensors["g_proj"])])
        low = padded([rt.matrix(tensors["a1_proj"])])
        self.n_qkv, self.n_gate, self.n_low = qkv.shape[0], gate.shape[0], low.shape[0]
        self.w_in = rt.product(torch.cat([qkv, gate, low], dim=0).contiguous())
        second = torch.zeros(self.H * self.D, self.n_low, dtype=rt.dtype, device=rt.device)
        second[:, :tensors["a1_proj"].shape[0]] = rt.matrix(tensors["a2_proj"])
        self.w_second = rt.product(second.contiguous())
        self.decay_bias = rt.vector32(tensors["a2_bias"])
        self.w_norm = rt.vector32(tensors["o_norm"])
        self.w_o = rt.product(rt.matrix(tensors["o_proj"]))

    def cache_spec(self):
        return StateSpec((("S", (self.H, self.V, self.D), "float32"),))      # S column by column

    def forward(self, x, step, cache, write_cache=True):
        rt, ops = self.rt, self.rt.ops
        if not write_cache:
            raise ValueError("a linear-attention mixer advances its state with every call; it cannot only read it")
        T, H, D, V = x.shape[0], self.H, self.D, self.V
        z = ops.linear(x, self.w_in)                                           # [T, q | k | v | gate | low]
        lo = self.n_qkv + self.n_gate
        low = z[:, lo:lo + self.n_low].contiguous()
        a = ops.linear(low, self.w_second)                                     # [T, H D] decay logits before the bias
        o = rt.empty(T, H * V)
        ops.outer_rule(z[:, :2 * H * D + H * V], a, z[:, self.n_qkv:self.n_qkv + H * V], self.decay_bias, self.tau,
                       self.w_norm, self.eps, cache.tensors["S"], step, o, H, D, V)
        return ops.linear(o, self.w_o)


register_part("mixer", "gated_linear_attention", GatedLinearAttention)
