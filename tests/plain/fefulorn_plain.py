"""Plain implementation of the Fefulorn design: whole sequences, no cache, 64-bit, one function per mechanism.

A decoder whose config.json lists its layers one by one. A layer runs its two sublayers side by side on the same
stream, each behind a norm of its own:
    x <- x + mixer(norm1(x)) + ff(norm2(x)).
The mixer is a state-space layer with a scalar decay per head and token (Mamba-2), an attention whose keys and
values come out of one latent row per token (no positions, sliding window), or an ordinary grouped attention with
biases, a rotation over the first elements of a head with linearly stretched positions, a sliding window, and
values that are blended with the values of the first such layer. The feed-forward is a mixture of experts with
clamped activations, a softmax router with groups, and a shared expert with a gate of its own. This file shares
nothing with the package; tests hold the engine against it.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_plain(x, w, eps):
    return rms(x, eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def window_mask(T, window):
    """[T, T] true where query i reads key j: 0 <= i - j < window (window None: every j <= i)."""
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    seen = j <= i
    if window:
        seen &= (i - j) < int(window)
    return seen


# ------------------------------------------------------------------ rotation
def rotate_half_linear(x, positions, rot):
    """x [T, heads, D]: the first rot.dims elements of every head turn, element i with i + dims/2, by the angle
    position * base^(-2i/dims) / factor."""
    if not rot or not int(rot.get("dims") or 0):
        return x
    dims, base = int(rot["dims"]), float(rot["base"])
    factor = float((rot.get("scaling") or {}).get("factor", 1.0))
    f = base ** (-2.0 * torch.arange(dims // 2, dtype=F64) / dims) / factor
    a = positions.to(F64)[:, None] * f[None, :]
    cos, sin = a.cos()[:, None, :], a.sin()[:, None, :]
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


# ------------------------------------------------------------------ mixers
def softmax_attention(q, k, v, scale, window):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] -> [T, H, Dv]; query head h reads kv head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    k, v = k.repeat_interleave(H // G, dim=1), v.repeat_interleave(H // G, dim=1)
    s = torch.einsum("thd,shd->hts", q, k) * float(scale)
    s = s.masked_fill(~window_mask(T, window)[None], -math.inf)
    return torch.einsum("hts,shd->thd", torch.softmax(s, dim=-1), v)


def attention_values(h, w, m):
    """The values of an attention layer as projected, [T, kv heads, vdim], before any blending."""
    return (h @ w["v"].T + w["v.b"]).view(h.shape[0], int(m.get("kv_heads") or m["heads"]), int(m.get("vdim") or m["dim"]))


def attention(h, w, m, v_first=None, positions=None):
    """h [T, W] -> (y [T, W], the layer's values as projected). v_first: the values of the first layer that blends
    (None: this layer does not blend, or is that first layer)."""
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m.get("kv_heads") or m["heads"]), int(m["dim"]), int(m.get("vdim") or m["dim"])
    pos = torch.arange(T) if positions is None else positions
    q = rotate_half_linear((h @ w["q"].T + w["q.b"]).view(T, H, D), pos, m.get("rot"))
    k = rotate_half_linear((h @ w["k"].T + w["k.b"]).view(T, G, D), pos, m.get("rot"))
    v_own = attention_values(h, w, m)
    v = v_own
    if v_first is not None:
        lam = w["vmix"].to(F64)
        v = (1.0 - lam) * v_own + lam * v_first
    window = (m.get("mask") or {}).get("size")
    o = softmax_attention(q, k, v, m["scale"], window)
    return o.reshape(T, H * Dv) @ w["o"].T, v_own


def latent_attention(h, w, m, eps):
    """Attention over one latent row per token, no positions, sliding window."""
    T = h.shape[0]
    H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    cq = norm_plain(h @ w["dq"].T, w["dq.norm"], eps)
    q = (cq @ w["uq"].T).view(T, H, D)
    c = norm_plain(h @ w["dkv"].T, w["dkv.norm"], eps)
    k = (c @ w["uk"].T).view(T, H, D)
    v = (c @ w["uv"].T).view(T, H, Dv)
    window = (m.get("mask") or {}).get("size")
    o = softmax_attention(q, k, v, m["scale"], window)
    return o.reshape(T, H * Dv) @ w["o"].T


def causal_conv(x, taps, bias, tail=None):
    """x [T, C], taps [C, K] (the last column is the current token's), zeros (or `tail` [K-1, C]) before the start."""
    K = taps.shape[1]
    before = torch.zeros(K - 1, x.shape[1], dtype=x.dtype) if tail is None else tail
    xx = torch.cat([before, x], dim=0)
    y = sum(xx[i:i + x.shape[0]] * taps[:, i][None, :] for i in range(K)) + bias
    return y, xx[xx.shape[0] - (K - 1):]


def mamba2(h, w, m, eps, state=None, tail=None):
    """State-space layer, token by token. Returns (y [T, W], final state [heads, N, vdim], conv tail)."""
    T = h.shape[0]
    H, P, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    parts = int(m["norm_groups"])
    inner = H * P
    zxbcdt = h @ w["in"].T
    z, xbc, dt = zxbcdt[:, :inner], zxbcdt[:, inner:2 * inner + 2 * G * N], zxbcdt[:, 2 * inner + 2 * G * N:]
    xbc, tail = causal_conv(xbc, w["conv"], w["conv.b"], tail)
    xbc = silu(xbc)
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N).repeat_interleave(H // G, dim=1)
    C = xbc[:, inner + G * N:].view(T, G, N).repeat_interleave(H // G, dim=1)
    dt = softplus(dt + w["dt_bias"])                                         # [T, H]
    decay = torch.exp(-torch.exp(w["A_log"].to(F64))[None, :] * dt)          # [T, H]
    S = torch.zeros(H, N, P, dtype=F64) if state is None else state.clone()
    y = torch.empty(T, H, P, dtype=F64)
    for t in range(T):
        S = decay[t][:, None, None] * S + dt[t][:, None, None] * B[t][:, :, None] * x[t][:, None, :]
        y[t] = torch.einsum("hnp,hn->hp", S, C[t]) + w["D"][:, None] * x[t]
    y = y.reshape(T, inner) * silu(z)
    y = rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * w["norm"]
    return y @ w["o"].T, S, tail


# ------------------------------------------------------------------ feed-forward
def clamped_expert(h, gate, up, down, limit):
    g = torch.clamp(h @ gate.T, max=limit)
    u = torch.clamp(h @ up.T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def route(z, top, count, keep):
    """Router logits z [T, E] -> (ids [T, top], weights [T, top]): softmax over all experts; experts form `count`
    groups of neighbours, a group scores its largest member, only the `keep` best groups are eligible; the `top`
    best eligible experts are taken with their scores as weights."""
    T, E = z.shape
    s = torch.softmax(z, dim=-1)
    choice = s.clone()
    if count > 1:
        group_score = s.view(T, count, E // count).max(-1).values
        best = group_score.topk(keep, dim=-1).indices
        allowed = torch.zeros(T, count, dtype=torch.bool).scatter_(1, best, True)
        choice = choice.masked_fill(~allowed.repeat_interleave(E // count, dim=1), -1.0)
    ids = choice.topk(top, dim=-1).indices
    return ids, s.gather(1, ids)


def moe(h, w, mlp):
    """Routed experts plus, if the layer has one, the shared expert behind its gate."""
    r = mlp["router"]
    E, top = int(r["experts"]), int(r["top"])
    groups = r.get("groups") or {}
    ids, weights = route(h @ w["router"].T, top, int(groups.get("count", 1)), int(groups.get("keep", groups.get("count", 1))))
    limit = float(mlp["expert"]["limit"])
    out = torch.zeros_like(h)
    for e in range(E):
        y = clamped_expert(h, w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], limit)
        out = out + y * (weights * (ids == e)).sum(-1, keepdim=True)
    if mlp.get("shared"):
        y = clamped_expert(h, w["shared.gate"], w["shared.up"], w["shared.down"], float(mlp["shared"]["limit"]))
        out = out + y * torch.sigmoid(h @ w["shared.sg"].T)
    return out


# ------------------------------------------------------------------ the model
def sub(weights, prefix):
    """The tensors whose names begin with prefix, by the rest of their names, in 64-bit."""
    return {k[len(prefix):]: v.to(F64) for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, tokens, streams=None):
    """Logits [T, vocab] of one whole sequence. streams: a list that receives the stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = weights["embed"].to(F64)[torch.as_tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    v_first = None
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        a = norm_plain(x, weights[p + "norm1"].to(F64), eps)
        w = sub(weights, p + "mix.")
        if layer["type"] == "mamba2":
            y, _, _ = mamba2(a, w, m, eps)
        elif layer["type"] == "latent_attention":
            y = latent_attention(a, w, m, eps)
        else:
            blends = bool(m.get("v_mix"))
            y, v_own = attention(a, w, m, v_first if blends else None)
            if blends and v_first is None:
                v_first = v_own
        if layer.get("mlp") is not None:
            b = norm_plain(x, weights[p + "norm2"].to(F64), eps)
            y = y + moe(b, sub(weights, p + "mlp."), layer["mlp"])
        x = x + y
        if streams is not None:
            streams.append(x.clone())
    x = norm_plain(x, weights["final.norm"].to(F64), eps)
    return (x @ weights["head"].to(F64).T) * float(cfg.get("logit_scale", 1.0))


def read_folder(folder):
    """(config.json as a dictionary, name -> tensor in 64-bit) of a model folder."""
    import json
    import os
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            w[name] = f.get_tensor(name).to(F64)
    return cfg, w


def logits(config, tensors, tokens):
    return forward(config, tensors, tokens)


def greedy(config, tensors, prompt, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(logits(config, tensors, toks)[-1].argmax()))
    return toks[len(prompt):]
