"""Grouped-query attention over the paged cache, with optional per-head RMSNorm on
queries and keys and a position encoding that is handed in.

Order of operations as in rollout/monkey_patch/qwen3.py:25-56: q/k/v projections
(three GEMMs there, one fused GEMM here), view as heads, q_norm and k_norm over the
head dimension with one weight [D] for all heads, K and V of the new tokens written
to the cache (qwen3.py:40-42), attention of the new queries over everything the
cache then holds (qwen3.py:43-45), output projection. The reference rotates inside
the attention kernel when it reads (rollout/attention.py:89-96, 116-125) and keeps K
un-rotated in the pool; here K is rotated once when it is written, which gives the
same scores because a request's positions never change.
Scale is D^-0.5 unless given (rollout/attention.py:195). Query head h reads kv head
h // (Hq/Hkv) (rollout/attention.py:65).

Beyond the reference, each off unless its parameter is given:
  values "keys"        there is no value projection: a token's value is its key as projected (with its
                       bias), before the rotation. The key pool holds the rotated keys, the value pool the
                       unrotated ones.
  bias True            q, k (and v, where there is one) and the output projection have biases
                       (roles q_bias, k_bias, v_bias, o_bias), added in the projection
  head_temperature     a learned factor per query head on the scale (role "temp", [Hq])
  softcap c            score <- c tanh(score / c), after scale and temperature
  window w, keep_first n   position i reads j <= i with i - j < w or j < n; the first n keys keep
                       their true positions
  sink True            softmax with one added to the denominator: a key of score 0 that has no value
"""
from __future__ import annotations

import torch

from ..cache.spec import PagedKVSpec
from .registry import register_part


class PagedAttention:
    @staticmethod
    def tensor_shapes(params):
        H, Hq, Hkv, D = (params["hidden_size"], params["num_heads"], params["num_kv_heads"],
                         params["head_dim"])
        shapes = {"q_proj": (Hq * D, H), "k_proj": (Hkv * D, H), "v_proj": (Hkv * D, H),
                  "o_proj": (H, Hq * D)}
        if params.get("values", "projected") == "keys":
            del shapes["v_proj"]
        if params.get("bias"):
            shapes.update({"q_bias": (Hq * D,), "k_bias": (Hkv * D,), "o_bias": (H,)})
            if "v_proj" in shapes:
                shapes["v_bias"] = (Hkv * D,)
        if params.get("head_temperature"):
            shapes["temp"] = (Hq,)
        if params.get("qk_norm_eps") is not None:
            shapes["q_norm"] = (D,)
            shapes["k_norm"] = (D,)
        return shapes

    @staticmethod
    def random_init(params, role):
        if role in ("q_norm", "k_norm", "temp"):
            return "norm"
        return "matrix"

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.hidden = int(params["hidden_size"])
        self.n_q = int(params["num_heads"])
        self.n_kv = int(params["num_kv_heads"])
        self.d = int(params["head_dim"])
        if self.n_q % self.n_kv:
            raise ValueError(f"{self.n_q} query heads are not a multiple of {self.n_kv} kv heads")
        if hasattr(rt.ops, "check_attention_sizes"):      # sizes the kernels do not take are refused now, not at the first step
            rt.ops.check_attention_sizes(self.n_q, self.n_kv, self.d, rt.dtype)
        self.scale = float(params["scale"]) if params.get("scale") is not None else self.d ** -0.5
        self.window = params.get("window")
        self.eps = params.get("qk_norm_eps")
        self.position = (shared or {}).get(params["position"]) if params.get("position") else None
        if params.get("position") and self.position is None:
            raise KeyError(f"attention names position encoding {params['position']!r}, which the model lacks")
        self.values_are_keys = params.get("values", "projected") == "keys"
        self.keep_first = int(params.get("keep_first") or 0)
        self.softcap = float(params.get("softcap") or 0.0)
        self.sink = bool(params.get("sink"))
        self.temp = rt.vector32(tensors["temp"]) if params.get("head_temperature") else None
        self.extras = {}
        if self.temp is not None or self.softcap or self.keep_first or self.sink:
            self.extras = dict(head_scale=self.temp, softcap=self.softcap, keep_first=self.keep_first, sink=self.sink)
        self.bias_in = self.bias_o = None
        names = ("q_proj", "k_proj") if self.values_are_keys else ("q_proj", "k_proj", "v_proj")
        if params.get("bias"):
            self.bias_in = torch.cat([rt.vector32(tensors[n[0] + "_bias"]) for n in names]).contiguous()
            self.bias_o = rt.vector32(tensors["o_bias"])
            if not self.values_are_keys:
                raise ValueError("attention: biases are built for the form whose values are its keys only")
        if self.values_are_keys and self.eps is not None:
            raise ValueError("attention: per-head norms are not built for the form whose values are its keys")
        self.w_qkv = rt.product(torch.cat([rt.matrix(tensors[n]) for n in names], dim=0).contiguous())
        self.w_o = rt.product(rt.matrix(tensors["o_proj"]), residual=self.bias_o is None)
        self.w_qn = rt.vector32(tensors["q_norm"]) if self.eps is not None else None
        self.w_kn = rt.vector32(tensors["k_norm"]) if self.eps is not None else None
        self._fusable = (self.position is None or hasattr(self.position, "tables")) and not self.values_are_keys
        # x goes into one product only and the output comes out of one: a norm before may be left to
        # the first (ScaledRows as x), a norm after may be finished inside the second (sink)
        self.first_product = (self.w_qkv, False)
        self.last_product = self.w_o if self.bias_o is None else None

    def cache_spec(self):
        return PagedKVSpec(self.n_kv, self.d, self.window, self.keep_first)

    def step_needs(self):
        """The q-tile list that the kernel set's attention reads for requests with more than one token."""
        ops = self.rt.ops
        rows = ops.prefill_tile_rows(self.d, self.rt.dtype) if hasattr(ops, "prefill_tile_rows") else None
        return {"prefill_tile_rows": set(rows)} if rows else {}

    def forward(self, x, step, cache, write_cache=True, sink=None):
        rt, ops = self.rt, self.rt.ops
        project = sink.project if sink is not None else ops.linear
        T, Hq, Hkv, D = x.shape[0], self.n_q, self.n_kv, self.d
        tables = step.groups[cache.group]
        qkv = ops.linear(x, self.w_qkv)                              # [T, (Hq+2Hkv)*D]
        if self.values_are_keys:
            if self.position is not None and not hasattr(self.position, "tables"):
                raise ValueError("attention whose values are its keys rotates by tables only")
            cos, sin, rot = self.position.tables() if self.position is not None else (None, None, 0)
            q = rt.empty(T, Hq, D)
            ops.qk_prepare(qkv, Hq, Hkv, D, self.bias_in, step.positions, cos, sin, rot, q,
                           cache.k_pool if write_cache else None, cache.v_pool if write_cache else None,
                           tables.slot_mapping)
            o = rt.empty(T, Hq, D)
            ops.attention(q, o, cache.k_pool, cache.v_pool, step, cache.group, self.scale,
                          int(self.window) if self.window else 0, **self.extras)
            y = project(o.view(T, Hq * D), self.w_o)
            return ops.add_bias(y, self.bias_o) if self.bias_o is not None else y
        if self._fusable and not self.extras and write_cache and hasattr(ops, "attention_qkv"):
            # every request brings one token: the kernel set may prepare q, k and v inside its attention
            cos, sin, rot = self.position.tables() if self.position is not None else (None, None, 0)
            o = rt.empty(T, Hq, D)
            if ops.attention_qkv(qkv, o, cache.k_pool, cache.v_pool, step, cache.group, self.scale,
                                 int(self.window) if self.window else 0, Hq, Hkv, D, self.w_qn, self.w_kn,
                                 float(self.eps) if self.eps is not None else 0.0, cos, sin, rot):
                return project(o.view(T, Hq * D), self.w_o)
        q = rt.empty(T, Hq, D)
        if self._fusable:
            cos, sin, rot = self.position.tables() if self.position is not None else (None, None, 0)
            ops.qkv_prepare(qkv, Hq, Hkv, D, self.w_qn, self.w_kn,
                            float(self.eps) if self.eps is not None else 0.0,
                            step.positions, cos, sin, rot, q,
                            cache.k_pool if write_cache else None,
                            cache.v_pool if write_cache else None, tables.slot_mapping)
        else:
            # a position encoding without rotary tables: norm, its own apply(), then the write
            k = rt.empty(T, Hkv, D)
            v = rt.empty(T, Hkv, D)
            ops.split_heads(qkv, Hq, Hkv, D, q, k, v)
            if self.eps is not None:
                ops.head_rmsnorm(q, self.w_qn, float(self.eps))
                ops.head_rmsnorm(k, self.w_kn, float(self.eps))
            # (a position encoding that asks for more of the step than positions, step_needs(), is given the step)
            if hasattr(self.position, "step_needs"):
                self.position.apply(q, k, step.positions, step)
            else:
                self.position.apply(q, k, step.positions)
            if write_cache:
                ops.kv_write(k, v, cache.k_pool, cache.v_pool, tables.slot_mapping)
        o = rt.empty(T, Hq, D)
        ops.attention(q, o, cache.k_pool, cache.v_pool, step, cache.group, self.scale,
                      int(self.window) if self.window else 0, **self.extras)
        return project(o.view(T, Hq * D), self.w_o)


register_part("mixer", "attention", PagedAttention)


class BlendAttention:
    """Grouped-query attention with biases on q, k and v, values of a width of their own, and values that may be
    blended with those of an earlier layer.

        q = W_q x + b_q (Hq heads of D),  k = W_k x + b_k (Hkv heads of D),  v = W_v x + b_v (Hkv heads of Dv)
        the first `rotary_dim` elements of every head of q and k turn by the position (the model's position part)
        v <- (1 - lambda) v + lambda v_first     in every layer that blends but the first such layer, whose v is
                                                 v_first for the same token; lambda is a stored number (role "blend")
        score = q . k * scale over the keys j with 0 <= i - j < window (None: every j <= i), softmax, W_o.
    The blended v is what the cache keeps. The biases are added, the rotation is done and the values are blended in
    32-bit by one kernel that also writes the cache rows. The cache rows of keys and values have one width, the
    larger of D and Dv (in bfloat16 a multiple of 16, so that the matrix-core kernels take it): the stacked weight
    of the first product and the output projection are filled up with zero rows and columns when the part is built,
    so a padded element is an exact zero everywhere and the attention kernels of the other designs serve unchanged.
    Parameters: hidden_size, num_heads, num_kv_heads, head_dim, value_dim (None: head_dim), scale (None: D^-1/2),
    window, position, value_rows (name of the model's shared part through which the first blending layer hands its
    values on; None: this layer does not blend), first_of_blend (this layer is that first one).
    """

    @staticmethod
    def tensor_shapes(params):
        H, Hq, Hkv, D = params["hidden_size"], params["num_heads"], params["num_kv_heads"], params["head_dim"]
        Dv = params.get("value_dim") or D
        shapes = {"q_proj": (Hq * D, H), "q_bias": (Hq * D,), "k_proj": (Hkv * D, H), "k_bias": (Hkv * D,),
                  "v_proj": (Hkv * Dv, H), "v_bias": (Hkv * Dv,), "o_proj": (H, Hq * Dv)}
        if params.get("value_rows"):
            shapes["blend"] = ()
        return shapes

    @staticmethod
    def random_init(params, role):
        if role == "blend":
            return lambda shape, gen: 0.2 + 0.6 * torch.rand(tuple(shape), generator=gen, dtype=torch.float32, device=gen.device)
        if role.endswith("_bias"):
            return lambda shape, gen: 0.1 * torch.randn(*shape, generator=gen, dtype=torch.float32, device=gen.device)
        return "matrix"

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        W = self.hidden = int(params["hidden_size"])
        self.n_q, self.n_kv = int(params["num_heads"]), int(params["num_kv_heads"])
        self.d, self.dv = int(params["head_dim"]), int(params.get("value_dim") or params["head_dim"])
        if self.n_q % self.n_kv:
            raise ValueError(f"{self.n_q} query heads are not a multiple of {self.n_kv} kv heads")
        # one width for the rows of q, k and v
        self.dp = max(self.d, self.dv)
        if rt.dtype == torch.bfloat16:
            self.dp = -(-self.dp // 16) * 16
        if hasattr(rt.ops, "check_attention_sizes"):
            rt.ops.check_attention_sizes(self.n_q, self.n_kv, self.dp, rt.dtype)
        self.scale = float(params["scale"]) if params.get("scale") is not None else self.d ** -0.5
        self.window = int(params["window"]) if params.get("window") else None
        self.position = (shared or {}).get(params["position"]) if params.get("position") else None
        if params.get("position") and self.position is None:
            raise KeyError(f"attention names position encoding {params['position']!r}, which the model lacks")
        if self.position is not None and (not hasattr(self.position, "tables") or
                                          getattr(self.position, "pairing", "half") != "half"):
            raise ValueError("attention with biases rotates by tables, element i with i + rotary_dim / 2")
        self.value_rows = (shared or {}).get(params["value_rows"]) if params.get("value_rows") else None
        if params.get("value_rows") and self.value_rows is None:
            raise KeyError(f"attention names shared rows {params['value_rows']!r}, which the model lacks")
        self.first_of_blend = bool(params.get("first_of_blend"))
        self.blend = float(tensors["blend"].float()) if self.value_rows is not None and not self.first_of_blend else None

        def padded(name, heads, width):
            """[heads * width, ...] -> [heads * dp, ...], every head's rows filled up with zeros."""
            t = tensors[name]
            out = torch.zeros((heads, self.dp) + tuple(t.shape[1:]), dtype=t.dtype, device=t.device)
            out[:, :width] = t.reshape((heads, width) + tuple(t.shape[1:]))
            return out.reshape((heads * self.dp,) + tuple(t.shape[1:]))

        rows = [padded("q_proj", self.n_q, self.d), padded("k_proj", self.n_kv, self.d), padded("v_proj", self.n_kv, self.dv)]
        self.w_qkv = rt.product(rt.matrix(torch.cat(rows, dim=0).contiguous()))
        self.bias = rt.vector32(torch.cat([padded("q_bias", self.n_q, self.d), padded("k_bias", self.n_kv, self.d),
                                           padded("v_bias", self.n_kv, self.dv)]))
        o = tensors["o_proj"].reshape(W, self.n_q, self.dv)
        o_pad = torch.zeros(W, self.n_q, self.dp, dtype=o.dtype, device=o.device)
        o_pad[:, :, :self.dv] = o
        self.w_o = rt.product(rt.matrix(o_pad.reshape(W, self.n_q * self.dp).contiguous()), residual=True)
        self.first_product = (self.w_qkv, False)          # (see PagedAttention)
        self.last_product = self.w_o

    def cache_spec(self):
        return PagedKVSpec(self.n_kv, self.dp, self.window, 0)

    def step_needs(self):
        ops = self.rt.ops
        rows = ops.prefill_tile_rows(self.dp, self.rt.dtype) if hasattr(ops, "prefill_tile_rows") else None
        return {"prefill_tile_rows": set(rows)} if rows else {}

    def forward(self, x, step, cache, write_cache=True, sink=None):
        rt, ops = self.rt, self.rt.ops
        project = sink.project if sink is not None else ops.linear
        T, Hq, Hkv, D = x.shape[0], self.n_q, self.n_kv, self.dp
        tables = step.groups[cache.group]
        qkv = ops.linear(x, self.w_qkv)                              # [T, (Hq + 2 Hkv) * D]
        cos, sin, rot = self.position.tables() if self.position is not None else (None, None, 0)
        first = None
        if self.value_rows is not None:
            if self.first_of_blend:
                first = rt.empty(T, Hkv * self.dv, dtype=torch.float32)      # (the true width: layers of other row widths read it)
                self.value_rows.put(step, first)
            else:
                first = self.value_rows.get(step)
        q = rt.empty(T, Hq, D)
        ops.qkv_blend_prepare(qkv, Hq, Hkv, D, self.bias, step.positions, cos, sin, rot, q,
                              cache.k_pool if write_cache else None, cache.v_pool if write_cache else None,
                              tables.slot_mapping, first, self.blend)
        o = rt.empty(T, Hq, D)
        ops.attention(q, o, cache.k_pool, cache.v_pool, step, cache.group, self.scale,
                      int(self.window) if self.window else 0)
        return project(o.view(T, Hq * D), self.w_o)


register_part("mixer", "blend_attention", BlendAttention)


class DifferentialAttention:
    """Grouped-query attention with two score maps per head over the same values.

    q has Hq heads of two maps [map 1 | map 2] of size D each, k has Hkv heads of the same two maps, v has
    Hkv heads of size Dv. Each map is a softmax attention of its own (score q_m . k_m * scale over the
    keys the mask leaves), a1 and a2; with one number for the layer,
        lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + lambda_init,
    the head gives  o = a1 - lambda a2,  o <- o / sqrt(mean(o^2) + eps) * (1 - lambda_init)  (the norm over the
    head's Dv values, no weight), and the heads side by side go through the output projection.
    Parameters: hidden_size, num_heads, num_kv_heads, head_dim (D, of one map), value_dim, scale,
    lambda_init, eps, position (a rotary encoding of the model's, applied to each map of q and k; None:
    none), chunk (c: position i reads j <= i with floor(i / c) = floor(j / c); None: all j <= i), window
    (None: none). The cache keeps both maps of a token's key in one row (2 D) and the value in a row of Dv.
    """

    @staticmethod
    def tensor_shapes(params):
        H, Hq, Hkv, D, Dv = (params["hidden_size"], params["num_heads"], params["num_kv_heads"],
                             params["head_dim"], params["value_dim"])
        return {"q_proj": (Hq * 2 * D, H), "k_proj": (Hkv * 2 * D, H), "v_proj": (Hkv * Dv, H),
                "o_proj": (H, Hq * Dv), "lq1": (D,), "lk1": (D,), "lq2": (D,), "lk2": (D,)}

    @staticmethod
    def random_init(params, role):
        if role in ("lq1", "lk1", "lq2", "lk2"):
            # small vectors: lambda stays near lambda_init
            return lambda shape, gen: 0.1 * torch.randn(*shape, generator=gen, dtype=torch.float32, device=gen.device)
        return "matrix"

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.hidden = int(params["hidden_size"])
        self.n_q, self.n_kv = int(params["num_heads"]), int(params["num_kv_heads"])
        self.d, self.dv = int(params["head_dim"]), int(params["value_dim"])
        if self.n_q % self.n_kv:
            raise ValueError(f"{self.n_q} query heads are not a multiple of {self.n_kv} kv heads")
        self.scale = float(params["scale"]) if params.get("scale") is not None else self.d ** -0.5
        self.lambda_init = float(params["lambda_init"])
        self.eps = float(params["eps"])
        self.chunk = int(params["chunk"]) if params.get("chunk") else None
        self.window = int(params["window"]) if params.get("window") else None
        self.position = (shared or {}).get(params["position"]) if params.get("position") else None
        if params.get("position") and self.position is None:
            raise KeyError(f"attention names position encoding {params['position']!r}, which the model lacks")
        if self.position is not None and not hasattr(self.position, "tables"):
            raise ValueError("differential attention rotates by tables only")
        if hasattr(rt.ops, "check_attention_diff_sizes"):
            rt.ops.check_attention_diff_sizes(self.n_q, self.n_kv, self.d, self.dv, rt.dtype)
        dot = lambda a, b: float((tensors[a].double() * tensors[b].double()).sum())
        import math
        self.lam = math.exp(dot("lq1", "lk1")) - math.exp(dot("lq2", "lk2")) + self.lambda_init
        self.w_qkv = rt.product(torch.cat([rt.matrix(tensors[n]) for n in ("q_proj", "k_proj", "v_proj")],
                                          dim=0).contiguous())
        self.w_o = rt.product(rt.matrix(tensors["o_proj"]))

    def cache_spec(self):
        return PagedKVSpec(self.n_kv, 2 * self.d, self.window, 0, self.dv, self.chunk)

    def step_needs(self):
        ops = self.rt.ops
        rows = ops.diff_prefill_tile_rows(self.d, self.dv, self.rt.dtype) if hasattr(ops, "diff_prefill_tile_rows") else None
        return {"prefill_tile_rows": set(rows)} if rows else {}

    def forward(self, x, step, cache, write_cache=True):
        rt, ops = self.rt, self.rt.ops
        T, Hq, Hkv, D, Dv = x.shape[0], self.n_q, self.n_kv, self.d, self.dv
        tables = step.groups[cache.group]
        qkv = ops.linear(x, self.w_qkv)                              # [T, (Hq + Hkv) * 2D + Hkv * Dv]
        cos, sin, rot = self.position.tables() if self.position is not None else (None, None, 0)
        interleaved = getattr(self.position, "pairing", "half") == "interleaved"
        q = rt.empty(T, Hq, 2 * D)
        ops.maps_qkv_prepare(qkv, Hq, Hkv, 2, D, Dv, step.positions, cos, sin, rot, interleaved, q,
                             cache.k_pool if write_cache else None, cache.v_pool if write_cache else None,
                             tables.slot_mapping)
        o = rt.empty(T, Hq, Dv)
        ops.attention_diff(q, o, cache.k_pool, cache.v_pool, step, cache.group, self.scale, self.lam, self.eps,
                           1.0 - self.lambda_init, window=self.window or 0, chunk=self.chunk or 0)
        return ops.linear(o.view(T, Hq * Dv), self.w_o)


register_part("mixer", "differential_attention", DifferentialAttention)


class LatentAttention:
    """Attention whose keys and values are read out of one narrow latent row per token.

    With H heads, per head D unrotated and R rotated query/key elements, values of Dv, and latents of
    q_rank and C = kv_rank elements:
        c_q = rmsnorm(W_dq x) w_dq,  q = W_uq c_q           heads of [D unrotated | R rotated]
        [c' | k_r] = W_dkv x,  c = rmsnorm(c') w_dkv        k_r: R elements, one rotated key part for all heads
        head h:  k_h = [W_uk,h c | rot(k_r)],  v_h = W_uv,h c
        score = (q_h . k_h) * scale, causal, softmax whose denominator also holds exp(sink_h) (a learned number
        per head that has no key and no value, params sink), output times sigmoid(W_g x)_h (params gate),
        heads side by side through W_o.
    The cache keeps c (value pool, rows of C) and rot(k_r) (key pool, rows of R) of every token and nothing per
    head. The products with W_uk and W_uv are moved to the query's side, where they cost one row per new token
    instead of one per key read:  q_h . (W_uk,h c) = (W_uk,h^T q_h) . c  and  sum_j p_j W_uv,h c_j = W_uv,h (sum_j p_j c_j),
    so every head reads the same rows [c | rot(k_r)] with a query of C + R elements, and one kernel serves
    whole prompts, portions and single tokens.
    Parameters: hidden_size, num_heads, head_dim (D), rot_dim (R; 0: no rotated part at all, the key pool's rows
    are empty), value_dim, q_rank, kv_rank, scale, eps, position (a rotary encoding of the model's over the R
    elements; None: none), sink, gate (each off unless true), window (w: position i reads j with 0 <= i - j < w;
    None: every j <= i); q_rank None: what the stored tensors have.
    """

    @staticmethod
    def tensor_shapes(params):
        W, H, D, R, Dv = (params["hidden_size"], params["num_heads"], params["head_dim"], params["rot_dim"],
                          params["value_dim"])
        Q, C = params["q_rank"], params["kv_rank"]
        shapes = {"dq": (Q, W), "dq_norm": (Q,), "uq": (H * (D + R), Q), "dkv": (C + R, W), "dkv_norm": (C,),
                  "uk": (H * D, C), "uv": (H * Dv, C), "o": (W, H * Dv)}
        if params.get("sink"):
            shapes["sink"] = (H,)
        if params.get("gate"):
            shapes["gate"] = (H, W)
        return shapes

    @staticmethod
    def random_init(params, role):
        if role in ("dq_norm", "dkv_norm"):
            return "norm"
        if role == "sink":
            return lambda shape, gen: torch.randn(*shape, generator=gen, dtype=torch.float32, device=gen.device)
        return "matrix"

    def __init__(self, params, tensors, rt, shared=None):
        self.rt = rt
        self.hidden = W = int(params["hidden_size"])
        self.H, self.D, self.R, self.Dv = (int(params[k]) for k in ("num_heads", "head_dim", "rot_dim", "value_dim"))
        self.Q, self.C = int(tensors["dq"].shape[0]), int(params["kv_rank"])
        if tensors["uq"].shape[1] != self.Q or tensors["dq_norm"].shape[0] != self.Q:
            raise ValueError("the query latent's two maps and its norm differ in the latent's size")
        self.scale = float(params["scale"]) if params.get("scale") is not None else (self.D + self.R) ** -0.5
        self.eps = float(params["eps"])
        self.position = (shared or {}).get(params["position"]) if params.get("position") else None
        if params.get("position") and self.position is None:
            raise KeyError(f"attention names position encoding {params['position']!r}, which the model lacks")
        if self.position is not None and not hasattr(self.position, "tables"):
            raise ValueError("latent attention rotates by tables only")
        if hasattr(rt.ops, "check_attention_latent_sizes"):
            rt.ops.check_attention_latent_sizes(self.H, self.C, self.R, rt.dtype)
        self.sink = rt.vector32(tensors["sink"]) if params.get("sink") else None
        self.window = int(params["window"]) if params.get("window") else None
        # x goes into one product: [W_dq; W_dkv; W_g], rows filled up with zeros to a multiple of 16
        rows = [rt.matrix(tensors["dq"]), rt.matrix(tensors["dkv"])]
        self.gated = bool(params.get("gate"))
        if self.gated:
            rows.append(rt.matrix(tensors["gate"]))
        pad = -sum(r.shape[0] for r in rows) % 16
        if pad:
            rows.append(torch.zeros(pad, W, dtype=rt.dtype, device=rt.device))
        self.w_in = rt.product(torch.cat(rows, dim=0).contiguous())
        self.w_dq_norm, self.w_dkv_norm = rt.vector32(tensors["dq_norm"]), rt.vector32(tensors["dkv_norm"])
        self.w_uq = rt.product(rt.matrix(tensors["uq"]))
        # per head: W_uk,h [D, C] (q's unrotated part times it gives the query over c) and W_uv,h^T [C, Dv]
        self.w_uk = rt.matrix(tensors["uk"]).view(self.H, self.D, self.C).contiguous()
        self.w_uv_t = rt.matrix(tensors["uv"]).view(self.H, self.Dv, self.C).transpose(1, 2).contiguous()
        self.w_o = rt.product(rt.matrix(tensors["o"]))

    def cache_spec(self):
        return PagedKVSpec(1, self.R, self.window, 0, self.C)

    def step_needs(self):
        ops = self.rt.ops
        rows = ops.latent_prefill_tile_rows(self.H, self.C, self.R, self.rt.dtype) \
            if hasattr(ops, "latent_prefill_tile_rows") else None
        return {"prefill_tile_rows": set(rows)} if rows else {}

    def forward(self, x, step, cache, write_cache=True):
        rt, ops = self.rt, self.rt.ops
        T, H, D, R, C, Q = x.shape[0], self.H, self.D, self.R, self.C, self.Q
        tables = step.groups[cache.group]
        z = ops.linear(x, self.w_in)                                  # [T, Q | C + R | H | pad]
        cos, sin, rot = self.position.tables() if self.position is not None else (None, None, 0)
        cq = rt.empty(T, Q)
        ops.latent_kv_prepare(z, Q, C, R, self.w_dq_norm, self.w_dkv_norm, self.eps, step.positions, cos, sin, rot, cq,
                              cache.k_pool if write_cache else None, cache.v_pool if write_cache else None,
                              tables.slot_mapping)
        q = ops.linear(cq, self.w_uq)                                 # [T, H (D + R)]
        q_flat = q.view(T, H, D + R)[:, :, :D].transpose(0, 1)        # [H, T, D], a view
        q_lat = ops.batched_product(q_flat, self.w_uk)                # [H, T, C]
        qq = rt.empty(T, H, C + R)
        ops.latent_q_prepare(q, q_lat, D, R, step.positions, cos, sin, rot, qq)
        o_lat = rt.empty(H, T, C)
        if self.window:
            ops.attention_latent(qq, o_lat, cache.k_pool, cache.v_pool, step, cache.group, self.scale, self.sink,
                                 window=self.window)
        else:
            ops.attention_latent(qq, o_lat, cache.k_pool, cache.v_pool, step, cache.group, self.scale, self.sink)
        o = ops.batched_product(o_lat, self.w_uv_t)                   # [H, T, Dv]
        y = rt.empty(T, H * self.Dv)
        ops.heads_gate(o, z[:, Q + C + R:Q + C + R + H] if self.gated else None, y)
        return ops.linear(y, self.w_o)


register_part("mixer", "latent_attention", LatentAttention)
