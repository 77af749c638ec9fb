"""A stand-in kernel set in plain torch, for tests only.

It has the method names and arguments of return_amd.kernels.hip_ops.HipOps, so that
(a) the engine's host logic (cache, step, scheduler) can be exercised on the CPU,
and (b) every HIP kernel has a plain reference of the same call to be compared with
on the GPU. Formulas cite the reference like the plain model does. Nothing in
return_amd imports this file.
"""
from __future__ import annotations

import torch

from return_amd.parts.runtime import ScaledRows, Slabs


def _pool_rows(pool, pages, n):
    """The first n token rows that the listed pages of a pool [pages, kv heads, rows in a page, width] hold, [n, kv heads, width]."""
    rows = pool[pages].transpose(1, 2)
    return rows.reshape(rows.shape[0] * rows.shape[1], pool.shape[1], pool.shape[3])[:n].float()


class TorchOps:
    def __init__(self, device="cpu"):
        self.device = torch.device(device)

    # rollout/monkey_patch/qwen3.py:73-75
    def embed(self, table, ids, out, scale=1.0):
        out.copy_(table[ids.long()].float() * scale)

    # rollout/fused.py:6-17 with the residual addition of qwen3.py:63,67 in front
    def add_rmsnorm(self, h, delta, weight, eps, out, rows=None, delta_scale=1.0):
        if isinstance(delta, Slabs):                        # shares of a product: their sum, rounded as the product would be
            delta = delta.tensor.sum(0).to(out.dtype)
        if rows is None:
            if delta is not None:
                h += delta_scale * delta.float()
            v = h
        else:
            v = h[rows.long()]
            if delta is not None:
                v = v + delta_scale * delta[rows.long()].float()
        rstd = 1.0 / torch.sqrt((v * v).sum(-1, keepdim=True) / v.shape[-1] + eps)
        out.copy_((v * rstd * weight).to(out.dtype))

    def residual_add(self, h, delta, scale=1.0):
        h += scale * delta.float()

    def stream_pair_rows(self, h, delta, delta_scale, h0, out):
        if delta is not None:
            h += delta_scale * delta.float()
        out.copy_(torch.cat([h, h0], dim=1).to(out.dtype))

    # rollout/fused.py:36-56 on a [-1, D] view
    def head_rmsnorm(self, x, weight, eps):
        v = x.float()
        rstd = 1.0 / torch.sqrt((v * v).sum(-1, keepdim=True) / v.shape[-1] + eps)
        x.copy_((v * rstd * weight).to(x.dtype))

    # rollout/attention.py:10-25
    def rope(self, x, positions, cos, sin, rotary_dim):
        half = rotary_dim // 2
        c = cos[positions.long()][:, None, :]
        s = sin[positions.long()][:, None, :]
        v = x.float()
        x1, x2 = v[..., :half], v[..., half:rotary_dim]
        o = torch.cat([x1 * c - x2 * s, x2 * c + x1 * s, v[..., rotary_dim:]], dim=-1)
        x.copy_(o.to(x.dtype))

    def split_heads(self, qkv, n_q, n_kv, D, q, k, v):
        T = qkv.shape[0]
        q.copy_(qkv[:, :n_q * D].view(T, n_q, D))
        k.copy_(qkv[:, n_q * D:(n_q + n_kv) * D].view(T, n_kv, D))
        v.copy_(qkv[:, (n_q + n_kv) * D:].view(T, n_kv, D))

    # rollout/cache.py:334-337
    def kv_write(self, k, v, k_pool, v_pool, slot_mapping):
        P = k_pool.shape[2]                                 # pools are [pages, kv heads, rows in a page, D]
        page, row = slot_mapping.long() // P, slot_mapping.long() % P
        k_pool[page, :, row] = k
        v_pool[page, :, row] = v

    def qkv_prepare(self, qkv, n_q, n_kv, D, w_q, w_k, eps, positions, cos, sin, rotary_dim, q_out,
                    k_pool, v_pool, slot_mapping):
        T = qkv.shape[0]
        q = qkv[:, :n_q * D].reshape(T, n_q, D).float()
        k = qkv[:, n_q * D:(n_q + n_kv) * D].reshape(T, n_kv, D).float()
        v = qkv[:, (n_q + n_kv) * D:].reshape(T, n_kv, D)

        def norm(x, w):
            return x * (1.0 / torch.sqrt((x * x).sum(-1, keepdim=True) / D + eps)) * w

        def rot(x):
            half = rotary_dim // 2
            c = cos[positions.long()][:, None, :]
            s = sin[positions.long()][:, None, :]
            x1, x2 = x[..., :half], x[..., half:rotary_dim]
            return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s, x[..., rotary_dim:]], dim=-1)

        if w_q is not None:
            q, k = norm(q, w_q), norm(k, w_k)
        if rotary_dim:
            q, k = rot(q), rot(k)
        q_out.copy_(q.to(q_out.dtype))
        if k_pool is not None:
            self.kv_write(k.to(qkv.dtype), v, k_pool, v_pool, slot_mapping)

    # rollout/fused.py:103-114
    def silu_mul(self, gu, out, bias=None):
        I = out.shape[1]
        g, u = gu[:, :I].float(), gu[:, I:].float()
        if bias is not None:
            g, u = g + bias[:I], u + bias[I:]
        out.copy_((g * torch.sigmoid(g) * u).to(out.dtype))

    # rollout/monkey_patch/qwen3.py:21 (F.linear)
    def linear(self, x, w, out_dtype=None):
        if isinstance(x, ScaledRows):                       # rows whose norm this product finishes
            y = (x.tensor.float() @ w.float().t()) * self._rstd(x)
            return y.to(out_dtype or x.tensor.dtype)
        return (x.float() @ w.float().t()).to(out_dtype or x.dtype)

    # A norm finished inside the products around it, as HipOps offers for steps of few rows
    # (norm(h) W^T = rstd * ((h * w_norm) W^T), rollout/fused.py:6-17): here for up to 16 rows of any
    # dtype, with the sum of squares in SHARES columns so that the adding-up is exercised too.
    SHARES = 3

    @staticmethod
    def _rstd(rows):
        return 1.0 / torch.sqrt(rows.partials.sum(-1, keepdim=True) / rows.size + rows.eps)

    def linear_residual(self, x, w):
        """As HipOps: for more than 16 rows the product comes as two shares over halves of K."""
        if isinstance(x, ScaledRows) or x.shape[0] <= 16 or x.shape[1] % 2:
            return self.linear(x, w)
        half = x.shape[1] // 2
        return Slabs(torch.stack([x[:, :half].float() @ w[:, :half].float().t(),
                                  x[:, half:].float() @ w[:, half:].float().t()]))

    def can_defer_norm(self, M, w_last, w_first, gated_first):
        return 1 <= M <= 16 and w_first.shape[1] == w_last.shape[0] >= self.SHARES

    def linear_add_norm(self, x, w, h, norm_weight, eps):
        y = self.linear(x, w)                               # (rounded to the compute dtype like a stored result)
        h += y.float()
        sq = h * h
        cut = [sq[:, i::self.SHARES].sum(-1) for i in range(self.SHARES)]
        return ScaledRows((h * norm_weight).to(y.dtype), torch.stack(cut, dim=1), h.shape[1], eps)

    # rollout/monkey_patch/qwen3.py:20-22
    def linear_silu_mul(self, x, w_gate_up):
        gu = self.linear(x, w_gate_up)
        out = torch.empty(gu.shape[0], w_gate_up.shape[0] // 2, dtype=gu.dtype, device=gu.device)
        self.silu_mul(gu, out)
        return out

    # rollout/attention.py:126-139 over the tables of rollout/cache.py:282-328,
    # gathered as opd/test_parallel.py:14-42 does
    def attention(self, q, out, k_pool, v_pool, step, group, scale, window=0, head_scale=None, softcap=0.0,
                  keep_first=0, sink=False):
        g = step.groups[group]
        n_q, n_kv = q.shape[1], k_pool.shape[1]
        cu_q, cu_p = step.cu_q.tolist(), g.cu_pages.tolist()
        q_start, kv_start = step.q_start.tolist(), g.kv_start.tolist()
        table = g.page_table.long()
        for s in range(step.n_seqs):
            a, b = cu_q[s], cu_q[s + 1]
            pages = table[cu_p[s]:cu_p[s + 1]]
            end = q_start[s] + (b - a)                      # keys held after this step
            k = k_pool[pages].transpose(1, 2).reshape(-1, n_kv, k_pool.shape[3])[:end - kv_start[s]].float()
            v = v_pool[pages].transpose(1, 2).reshape(-1, n_kv, v_pool.shape[3])[:end - kv_start[s]].float()
            k_pos = torch.arange(kv_start[s], end, device=q.device)
            q_pos = torch.arange(q_start[s], end, device=q.device)
            kk = k.repeat_interleave(n_q // n_kv, dim=1)
            vv = v.repeat_interleave(n_q // n_kv, dim=1)
            score = torch.einsum("qhd,khd->hqk", q[a:b].float(), kk) * scale
            if head_scale is not None:
                score = score * head_scale.float()[:, None, None]
            if softcap:
                score = softcap * torch.tanh(score / softcap)
            hide = k_pos[None, :] > q_pos[:, None]
            if window:
                far = k_pos[None, :] <= q_pos[:, None] - window
                if keep_first:
                    far = far & (k_pos[None, :] >= keep_first)
                hide = hide | far
            score = score.masked_fill(hide[None], float("-inf"))
            if sink:                                        # one more key of score 0 that has no value
                zero = torch.zeros_like(score[..., :1])
                prob = torch.cat([score, zero], dim=-1).softmax(-1)[..., :-1]
            else:
                prob = score.softmax(-1)
            out[a:b] = torch.einsum("hqk,khd->qhd", prob, vv).to(out.dtype)

    # ---- attention with two score maps per head over the same values
    def maps_qkv_prepare(self, qkv, n_q, n_kv, maps, D, Dv, positions, cos, sin, rotary_dim, interleaved, q_out,
                         k_pool, v_pool, slot_mapping):
        T, R = qkv.shape[0], int(rotary_dim)
        qw, kw = n_q * maps * D, n_kv * maps * D
        q = qkv[:, :qw].reshape(T, n_q * maps, D).float()
        k = qkv[:, qw:qw + kw].reshape(T, n_kv * maps, D).float()
        v = qkv[:, qw + kw:].reshape(T, n_kv, Dv)

        def rot(x):
            if R == 0:
                return x
            c, s = cos[positions.long()][:, None, :], sin[positions.long()][:, None, :]
            if interleaved:
                u, w = x[..., 0:R:2], x[..., 1:R:2]
                turned = torch.stack([u * c - w * s, w * c + u * s], dim=-1).reshape(*x.shape[:-1], R)
            else:
                u, w = x[..., :R // 2], x[..., R // 2:R]
                turned = torch.cat([u * c - w * s, w * c + u * s], dim=-1)
            return torch.cat([turned, x[..., R:]], dim=-1)

        q_out.copy_(rot(q).reshape(T, n_q, maps * D).to(q_out.dtype))
        if k_pool is not None:
            P = k_pool.shape[2]
            page, row = slot_mapping.long() // P, slot_mapping.long() % P
            k_pool[page, :, row] = rot(k).reshape(T, n_kv, maps * D).to(k_pool.dtype)
            v_pool[page, :, row] = v

    def attention_diff(self, q, out, k_pool, v_pool, step, group, scale, lam, eps, out_scale, window=0, chunk=0):
        g = step.groups[group]
        n_q, n_kv, D = q.shape[1], k_pool.shape[1], q.shape[2] // 2
        cu_q, cu_p = step.cu_q.tolist(), g.cu_pages.tolist()
        q_start, kv_start = step.q_start.tolist(), g.kv_start.tolist()
        table = g.page_table.long()
        for s in range(step.n_seqs):
            a, b = cu_q[s], cu_q[s + 1]
            pages = table[cu_p[s]:cu_p[s + 1]]
            end = q_start[s] + (b - a)
            k = _pool_rows(k_pool, pages, end - kv_start[s]).repeat_interleave(n_q // n_kv, dim=1)
            v = _pool_rows(v_pool, pages, end - kv_start[s]).repeat_interleave(n_q // n_kv, dim=1)
            k_pos = torch.arange(kv_start[s], end, device=q.device)
            q_pos = torch.arange(q_start[s], end, device=q.device)
            hide = k_pos[None, :] > q_pos[:, None]
            if window:
                hide = hide | (k_pos[None, :] <= q_pos[:, None] - window)
            if chunk:
                hide = hide | (k_pos[None, :] // chunk != q_pos[:, None] // chunk)
            qq = q[a:b].float()
            maps = []
            for m in range(2):
                score = torch.einsum("qhd,khd->hqk", qq[..., m * D:(m + 1) * D], k[..., m * D:(m + 1) * D]) * scale
                maps.append(torch.einsum("hqk,khd->qhd", score.masked_fill(hide[None], float("-inf")).softmax(-1), v))
            o = maps[0] - lam * maps[1]
            o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * out_scale
            out[a:b] = o.to(out.dtype)

    # ---- routed experts
    def moe_route(self, z, bias, top, groups, keep, norm_eps, law="sigmoid_groups"):
        T, E = z.shape
        if law == "softmax_top":
            val, ids = (z.float() + (bias if bias is not None else 0.0)).topk(top, dim=-1)
            return ids.int(), torch.softmax(val, dim=-1)
        if law == "softmax_groups":
            s = torch.softmax(z.float(), dim=-1)
            c = s.clone()
            if groups > 1 and keep < groups:
                per = E // groups
                stay = torch.zeros(T, groups, dtype=torch.bool, device=z.device)
                stay.scatter_(1, c.view(T, groups, per).max(-1).values.topk(keep, dim=-1).indices, True)
                c = c.masked_fill(~stay[:, :, None].expand(T, groups, per).reshape(T, E), float("-inf"))
            ids = c.topk(top, dim=-1).indices
            return ids.int(), s.gather(1, ids)
        s = torch.sigmoid(z.float())
        c = s + (bias if bias is not None else 0.0)
        if groups > 1 and keep < groups:
            per = E // groups
            score = c.view(T, groups, per).topk(min(2, per), dim=-1).values.sum(-1)
            stay = torch.zeros(T, groups, dtype=torch.bool, device=z.device)
            stay.scatter_(1, score.topk(keep, dim=-1).indices, True)
            c = c.masked_fill(~stay[:, :, None].expand(T, groups, per).reshape(T, E), float("-inf"))
        ids = c.topk(top, dim=-1).indices
        w = s.gather(1, ids)
        return ids.int(), w / (w.sum(-1, keepdim=True) + norm_eps)

    def moe_experts(self, x, ids, weights, w_gate_up, w_down, activation="silu", limit=0.0, slope=1.702, extra=None,
                    extra_logits=None):
        T, H = x.shape
        I = w_gate_up.shape[1] // 2
        out = torch.zeros(T, H, dtype=torch.float32, device=x.device)
        for t in range(T):
            for k in range(ids.shape[1]):
                e = int(ids[t, k])
                gu = (x[t].float() @ w_gate_up[e].float().t()).to(x.dtype).float()
                if activation == "clamped":
                    g, u = gu[:I].clamp(max=limit), gu[I:].clamp(-limit, limit)
                    a = (g * torch.sigmoid(slope * g) * (u + 1.0)).to(x.dtype)
                else:
                    a = (gu[:I] * torch.sigmoid(gu[:I]) * gu[I:]).to(x.dtype)
                out[t] += weights[t, k] * (a.float() @ w_down[e].float().t()).to(x.dtype).float()
        if extra is not None:                               # one more term of every token's sum, behind its gate
            out += extra.float() * torch.sigmoid(extra_logits.float())
        return out.to(x.dtype)

    def clamped_mul(self, gu, out, limit, slope=1.702):
        """gu [T, >= 2 I] (gate columns first) -> out [T, I] = g sigmoid(slope g) (u + 1), g = min(gate, limit),
        u = clamp(up, -limit, limit)."""
        I = out.shape[1]
        g, u = gu[:, :I].float().clamp(max=limit), gu[:, I:2 * I].float().clamp(-limit, limit)
        out.copy_((g * torch.sigmoid(slope * g) * (u + 1.0)).to(out.dtype))
        return out

    def add_rmsnorm_pair(self, h, a, b, w1, eps1, out1, w2, eps2, out2):
        """h += a + b (each may be None); out1 = rmsnorm(h) w1, out2 = rmsnorm(h) w2."""
        if a is not None:
            h += a.float()
        if b is not None:
            h += b.float()
        ms = (h * h).sum(-1, keepdim=True) / h.shape[-1]
        out1.copy_((h / torch.sqrt(ms + eps1) * w1).to(out1.dtype))
        out2.copy_((h / torch.sqrt(ms + eps2) * w2).to(out2.dtype))

    # ---- attention with biases, one row width for q, k and v, values blended with an earlier layer's
    def qkv_blend_prepare(self, qkv, n_q, n_kv, D, bias, positions, cos, sin, rotary_dim, q_out, k_pool, v_pool,
                          slot_mapping, first=None, blend=None):
        T = qkv.shape[0]
        x = qkv.float() + bias
        q = self._turn(x[:, :n_q * D].reshape(T, n_q, D), positions, cos, sin, rotary_dim)
        k = self._turn(x[:, n_q * D:(n_q + n_kv) * D].reshape(T, n_kv, D), positions, cos, sin, rotary_dim)
        v = x[:, (n_q + n_kv) * D:]
        if first is not None:                               # [T, n_kv Dv]: the heads' true width, Dv <= D
            Dv = first.shape[1] // n_kv
            if blend is None:
                first.copy_(v.reshape(T, n_kv, D)[:, :, :Dv].reshape(T, n_kv * Dv))
            else:
                other = torch.zeros(T, n_kv, D, device=v.device)
                other[:, :, :Dv] = first.reshape(T, n_kv, Dv)
                v = (1.0 - blend) * v + blend * other.reshape(T, n_kv * D)
        q_out.copy_(q.to(q_out.dtype))
        if k_pool is None:
            return
        P = k_pool.shape[2]
        page, row = slot_mapping.long() // P, slot_mapping.long() % P
        k_pool[page, :, row] = k.to(k_pool.dtype)
        v_pool[page, :, row] = v.reshape(T, n_kv, D).to(v_pool.dtype)

    def scalar_rule(self, qkv, dt, a_log, dt_bias, skip, gate, norm_w, norm_groups, eps, state, step, out, H, G, D, V):
        """S <- exp(-exp(a_log) delta) S + delta k v^T, o = S^T q + skip v with delta = softplus(dt + dt_bias);
        out = rmsnorm over norm_groups parts of (o * silu(gate)), times norm_w. qkv rows [q: G D | k: G D | v: H V]."""
        cu, slots = step.cu_q_host, step.slot_ids_host
        T = qkv.shape[0]
        q = qkv[:, :G * D].float().view(T, G, D).repeat_interleave(H // G, dim=1)
        k = qkv[:, G * D:2 * G * D].float().view(T, G, D).repeat_interleave(H // G, dim=1)
        v = qkv[:, 2 * G * D:].float().view(T, H, V)
        delta = torch.nn.functional.softplus(dt.float() + dt_bias, threshold=30.0)        # [T, H]
        decay = torch.exp(-torch.exp(a_log)[None, :] * delta)
        o = torch.empty(T, H, V, dtype=torch.float32, device=qkv.device)
        for s in range(step.n_seqs):
            S = state[slots[s]].transpose(1, 2)               # kept [H, V, D]; a view [H, D, V], updated in place
            for t in range(cu[s], cu[s + 1]):
                S *= decay[t][:, None, None]
                S += (delta[t][:, None] * k[t])[:, :, None] * v[t][:, None, :]
                o[t] = torch.einsum("hdv,hd->hv", S, q[t]) + skip[:, None] * v[t]
        c = gate.float()
        y = (o.reshape(T, H * V) * (c * torch.sigmoid(c))).view(T, norm_groups, -1)
        y = y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)
        out.copy_((y.reshape(T, H * V) * norm_w).to(out.dtype))
        return out

    # ---- the parts beside the usual ones, each as its kernel is called
    def relu_sq(self, x):
        x.copy_((torch.relu(x.float()) ** 2).to(x.dtype))
        return x

    def add_bias(self, x, bias):
        x.copy_((x.float() + bias).to(x.dtype))
        return x

    def causal_conv(self, x, w, tail, step, out, add_input=False, silu=False, bias=None):
        taps = w.shape[1]
        cu, slots = step.cu_q_host, step.slot_ids_host
        for s in range(step.n_seqs):
            a, b = cu[s], cu[s + 1]
            seq = torch.cat([tail[slots[s]].float(), x[a:b].float()], dim=0)       # [taps-1 + n, C]
            y = torch.zeros(b - a, x.shape[1], dtype=torch.float32, device=x.device)
            for j in range(taps):
                y += w[:, j] * seq[j:j + (b - a)]
            if bias is not None:
                y = y + bias
            if add_input:
                y = y + x[a:b].float()
            if silu:
                y = y * torch.sigmoid(y)
            out[a:b] = y.to(out.dtype)
            if taps > 1:
                tail[slots[s]] = seq[-(taps - 1):].to(tail.dtype)
        return out

    def delta_rule_fits(self, D, V):
        return True

    def delta_rule(self, qkv, beta, ag, a_log, dt_bias, norm_w, eps, state, step, out, H, G, D, V):
        cu, slots = step.cu_q_host, step.slot_ids_host
        T = qkv.shape[0]
        q = qkv[:, :G * D].float().view(T, G, D)
        k = qkv[:, G * D:2 * G * D].float().view(T, G, D)
        v = qkv[:, 2 * G * D:].float().view(T, H, V)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        beta = torch.sigmoid(beta.float())
        a = ag[:, :H * D].float() + dt_bias
        g = torch.exp(-torch.exp(a_log)[None, :, None] * torch.nn.functional.softplus(a).view(T, H, D))
        gate = torch.sigmoid(ag[:, H * D:].float()).view(T, H, V)
        rep = H // G
        for s in range(step.n_seqs):
            S = state[slots[s]].transpose(1, 2)               # kept [H, V, D]; a view [H, D, V], updated in place
            for t in range(cu[s], cu[s + 1]):
                kt, qt = k[t].repeat_interleave(rep, 0), q[t].repeat_interleave(rep, 0)    # [H, D]
                S *= g[t][:, :, None]
                u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, kt))
                S += kt[:, :, None] * u[:, None, :]
                o = torch.einsum("hdv,hd->hv", S, qt)
                o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * norm_w * gate[t]
                out[t] = o.reshape(-1).to(out.dtype)
        return out

    def outer_rule(self, qkv, a, gate, decay_bias, tau, norm_w, eps, state, step, out, H, D, V):
        """S <- diag(alpha) S + k v^T, o = S^T q with alpha = sigmoid(a + bias)^(1/tau); the read-out normed over the
        head's V, weighed, times silu(gate)."""
        cu, slots = step.cu_q_host, step.slot_ids_host
        T = qkv.shape[0]
        q = qkv[:, :H * D].float().view(T, H, D) * D ** -0.5
        k = qkv[:, H * D:2 * H * D].float().view(T, H, D)
        v = qkv[:, 2 * H * D:2 * H * D + H * V].float().view(T, H, V)
        alpha = torch.exp(-torch.nn.functional.softplus(-(a.float() + decay_bias)) / tau).view(T, H, D)
        c = gate.float().view(T, H, V)
        for s in range(step.n_seqs):
            S = state[slots[s]].transpose(1, 2)               # kept [H, V, D]; a view [H, D, V], updated in place
            for t in range(cu[s], cu[s + 1]):
                S *= alpha[t][:, :, None]
                S += k[t][:, :, None] * v[t][:, None, :]
                o = torch.einsum("hdv,hd->hv", S, q[t])
                o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * norm_w * (c[t] * torch.sigmoid(c[t]))
                out[t] = o.reshape(-1).to(out.dtype)
        return out

    # ---- norms on both sides of a sublayer, and the stream as a weighted sum of all results so far
    def post_norm_add(self, h, y, weight, eps, next_weight=None, next_eps=0.0, out=None):
        v = y.float()
        h += v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * weight
        if next_weight is not None:
            out.copy_((h / torch.sqrt((h * h).mean(-1, keepdim=True) + next_eps) * next_weight).to(out.dtype))

    def depth_mix(self, results, count, weights, out, norm_weight=None, eps=0.0, normed=None):
        acc = torch.zeros_like(out)
        for j in range(count):
            acc += weights[j] * results[j]
        out.copy_(acc)
        if norm_weight is not None:
            normed.copy_((acc / torch.sqrt((acc * acc).mean(-1, keepdim=True) + eps) * norm_weight).to(normed.dtype))

    def post_norm_mix(self, results, count, weights, y, weight, eps, out, norm_weight=None, norm_eps=0.0, normed=None):
        self.post_norm_add(results[count - 1], y, weight, eps)
        self.depth_mix(results, count, weights, out, norm_weight, norm_eps, normed)

    # ---- attention over a latent row per token
    def batched_product(self, a, b):
        """[B, M, K] x [B, K, N] -> [B, M, N], rounded to a's dtype."""
        return torch.bmm(a.float(), b.float()).to(a.dtype)

    def latent_kv_prepare(self, z, Q, C, R, wq_norm, wkv_norm, eps, positions, cos, sin, rotary_dim, cq_out,
                          k_pool, v_pool, slot_mapping):
        def norm(x, w):
            return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w
        cq_out.copy_(norm(z[:, :Q].float(), wq_norm).to(cq_out.dtype))
        if k_pool is None:
            return
        c = norm(z[:, Q:Q + C].float(), wkv_norm)
        kr = self._turn(z[:, Q + C:Q + C + R].float(), positions, cos, sin, rotary_dim)
        P = k_pool.shape[2]
        page, row = slot_mapping.long() // P, slot_mapping.long() % P
        if R:
            k_pool[page, 0, row] = kr.to(k_pool.dtype)
        v_pool[page, 0, row] = c.to(v_pool.dtype)

    @staticmethod
    def _turn(x, positions, cos, sin, rotary_dim):
        """The first rotary_dim elements of the last axis turn, element i with i + rotary_dim / 2."""
        if not rotary_dim:
            return x
        half = rotary_dim // 2
        shape = (x.shape[0],) + (1,) * (x.dim() - 2) + (half,)
        c, s = cos[positions.long()].view(shape), sin[positions.long()].view(shape)
        u, v = x[..., :half], x[..., half:rotary_dim]
        return torch.cat([u * c - v * s, v * c + u * s, x[..., rotary_dim:]], dim=-1)

    def latent_q_prepare(self, q, q_lat, D, R, positions, cos, sin, rotary_dim, qq_out):
        T, H = qq_out.shape[0], qq_out.shape[1]
        C = q_lat.shape[2]
        qq_out[:, :, :C] = q_lat.transpose(0, 1)
        turned = self._turn(q.view(T, H, D + R)[:, :, D:].float(), positions, cos, sin, rotary_dim)
        qq_out[:, :, C:] = turned.to(qq_out.dtype)

    def attention_latent(self, qq, out, k_pool, v_pool, step, group, scale, sink=None, window=0):
        """qq [T, H, C + R]; every head reads the rows [c | turned key part] of the two pools; out [H, T, C]."""
        g = step.groups[group]
        C = v_pool.shape[3]
        cu_q, cu_p = step.cu_q.tolist(), g.cu_pages.tolist()
        q_start, kv_start = step.q_start.tolist(), g.kv_start.tolist()
        table = g.page_table.long()
        for s in range(step.n_seqs):
            a, b = cu_q[s], cu_q[s + 1]
            pages = table[cu_p[s]:cu_p[s + 1]]
            end = q_start[s] + (b - a)
            kr = _pool_rows(k_pool, pages, end - kv_start[s])[:, 0]
            c = _pool_rows(v_pool, pages, end - kv_start[s])[:, 0]
            k_pos = torch.arange(kv_start[s], end, device=qq.device)
            q_pos = torch.arange(q_start[s], end, device=qq.device)
            q = qq[a:b].float()
            score = (torch.einsum("qhc,kc->hqk", q[..., :C], c) + torch.einsum("qhr,kr->hqk", q[..., C:], kr)) * scale
            hide = k_pos[None, :] > q_pos[:, None]
            if window:
                hide = hide | (k_pos[None, :] <= q_pos[:, None] - window)
            score = score.masked_fill(hide[None], float("-inf"))
            if sink is not None:                            # one more term in the denominator, with no value
                extra = sink.float()[:, None, None].expand(-1, b - a, 1)
                prob = torch.cat([score, extra], dim=-1).softmax(-1)[..., :-1]
            else:
                prob = score.softmax(-1)
            out[:, a:b] = torch.einsum("hqk,kc->hqc", prob, c).to(out.dtype)

    def heads_gate(self, o, gate, out):
        """o [H, T, Dv], gate [T, H] logits (or None) -> out [T, H Dv] = o * sigmoid(gate) head by head."""
        v = o.float().transpose(0, 1)
        if gate is not None:
            v = v * torch.sigmoid(gate.float())[:, :, None]
        out.copy_(v.reshape(out.shape).to(out.dtype))

    def token_side(self, h, delta, token_ids, table, offset, gate, proj, weight, eps):
        if delta is not None:
            h += delta.float()
        S = gate.shape[0]
        e = table[token_ids.long()][:, offset:offset + S].float()
        a = h @ gate.float().t()
        g = 0.5 * a * (1 + torch.tanh(0.7978845608028654 * (a + 0.044715 * a ** 3))) * e
        y = g @ proj.float().t()
        h += y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps) * weight

    def qk_prepare(self, qk, n_q, n_kv, D, bias, positions, cos, sin, rotary_dim, q_out, k_pool, v_pool, slot_mapping):
        T = qk.shape[0]
        x = qk.float()
        if bias is not None:
            x = x + bias
        q = x[:, :n_q * D].reshape(T, n_q, D)
        k = x[:, n_q * D:].reshape(T, n_kv, D).to(qk.dtype)     # the value pool's rows; the keys are these, rotated

        def rot(x):
            if not rotary_dim:
                return x
            half = rotary_dim // 2
            c = cos[positions.long()][:, None, :]
            s = sin[positions.long()][:, None, :]
            x1, x2 = x[..., :half], x[..., half:rotary_dim]
            return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s, x[..., rotary_dim:]], dim=-1)

        q_out.copy_(rot(q).to(q_out.dtype))
        if k_pool is not None:
            self.kv_write(rot(k.float()).to(qk.dtype), k, k_pool, v_pool, slot_mapping)

    # rollout/model.py:15-61 with the draw made by inverse CDF in vocabulary order
    def sample(self, logits, temperature, top_k, top_p, u):
        M, V = logits.shape
        res = torch.empty(M, 2, dtype=torch.int32, device=logits.device)
        for r in range(M):
            row = logits[r].double()
            t = float(temperature[r])
            if t <= 0:
                tok = int(row.argmax())
            else:
                x = row / t
                vals, idx = torch.sort(x, descending=True, stable=True)
                k = int(top_k[r]) if int(top_k[r]) > 0 else V
                vals = vals.masked_fill(torch.arange(V, device=x.device) >= k, float("-inf"))
                cum = vals.softmax(-1).cumsum(-1)
                remove = cum > float(top_p[r])
                remove[1:] = remove[:-1].clone()
                remove[0] = False
                vals = vals.masked_fill(remove, float("-inf"))
                p = torch.zeros(V, dtype=torch.float64, device=x.device)
                p[idx] = vals.softmax(-1)
                c = p.cumsum(-1)
                tok = int((c > float(u[r]) * float(c[-1])).nonzero()[0]) if float(u[r]) < 1 else V - 1
            lp = float(row.log_softmax(-1)[tok])
            res[r, 0] = tok
            res[r, 1] = torch.tensor(lp, dtype=torch.float32).view(torch.int32)
        return res
