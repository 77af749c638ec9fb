"""Plain implementation of the Safilorn design: whole sequences, no cache, 64-bit, one function per mechanism.

A decoder whose config.json lists its layers one by one. Every layer has norms on both sides of each sublayer,
    x <- x + post(mixer(pre(x)));  x <- x + post'(ff(pre'(x))),
all of them RMS norms times (1 + w), and after the layer the stream becomes a weighted sum of the embedding's
output and of every layer's result so far (weights stored with the layer). The mixer is an attention whose keys
and values come out of one narrow latent row per token (with a rotated key part shared by the heads, a sink in
the softmax and a gate per head), or a gated linear attention with a decay per key channel. The feed-forward is
a dense gated one with biases or a mixture of experts with clamped activations. This file shares nothing with
the package; tests hold the engine against it.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    """RMS norm whose stored weight is an offset from one."""
    return rms(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return rms(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------ rotation
def yarn_frequencies(rot):
    """Frequencies of the pairs and the factor on cos and sin, after the scaling rule."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def turn_dim(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half(x, positions, rot):
    """x [T, heads, D]: the first rot.dims elements of every head turn, element i with i + dims/2."""
    dims = int(rot["dims"])
    f, m = yarn_frequencies(rot)
    a = positions.to(F64)[:, None] * f[None, :]
    cos, sin = (a.cos() * m)[:, None, :], (a.sin() * m)[:, None, :]
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


# ------------------------------------------------------------------ mixers
def latent_attention(h, w, m, eps, positions=None):
    """h [T, W] -> [T, W]. w: the mixer's tensors by their short names; m: its sizes."""
    T = h.shape[0]
    H, D, R, Dv, C = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    pos = torch.arange(T) if positions is None else positions
    cq = norm_plain(h @ w["dq"].T, w["dq.norm"], eps)
    q = (cq @ w["uq"].T).view(T, H, D + R)
    q_flat, q_turn = q[..., :D], rotate_half(q[..., D:], pos, m["rot"])
    dkv = h @ w["dkv"].T
    c = norm_plain(dkv[:, :C], w["dkv.norm"], eps)
    k_turn = rotate_half(dkv[:, None, C:], pos, m["rot"])[:, 0]              # [T, R], one for all heads
    k_flat = (c @ w["uk"].T).view(T, H, D)
    v = (c @ w["uv"].T).view(T, H, Dv)
    s = (torch.einsum("thd,shd->hts", q_flat, k_flat) + torch.einsum("thr,sr->hts", q_turn, k_turn)) * float(m["scale"])
    mask = torch.arange(T)[None, :] <= torch.arange(T)[:, None]
    s = s.masked_fill(~mask[None], -math.inf)
    sink = w["sink"].to(F64)[:, None, None]
    top = torch.maximum(s.max(-1, keepdim=True).values, sink)
    e = torch.exp(s - top)
    p = e / (e.sum(-1, keepdim=True) + torch.exp(sink - top))                # the sink has no value
    o = torch.einsum("hts,shd->thd", p, v)
    gate = torch.sigmoid(h @ w["g"].T)                                       # [T, H]
    return (o * gate[:, :, None]).reshape(T, H * Dv) @ w["o"].T


def gla(h, w, m, eps, state=None):
    """Gated linear attention, token by token. Returns (y [T, W], final state [heads, D, Dv])."""
    T = h.shape[0]
    H, D, Dv, tau = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["tau"])
    q = (h @ w["q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w["k"].T).view(T, H, D)
    v = (h @ w["v"].T).view(T, H, Dv)
    z = (h @ w["a1"].T) @ w["a2"].T + w["a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / tau)).view(T, H, D)
    S = torch.zeros(H, D, Dv, dtype=F64) if state is None else state.clone()
    o = torch.empty(T, H, Dv, dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = norm_plain(o, w["norm"], eps).reshape(T, H * Dv)
    return (o * silu(h @ w["g"].T)) @ w["o"].T, S


# ------------------------------------------------------------------ feed-forward
def dense_ff(h, w):
    g = h @ w["gate"].T + w["gate.b"]
    u = h @ w["up"].T + w["up.b"]
    return (silu(g) * u) @ w["down"].T + w["down.b"]


def expert(h, gate, up, down, limit):
    g = (h @ gate.T).clamp(max=limit)
    u = (h @ up.T).clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def route(h, w, top):
    """(ids [T, top], weights [T, top]): the largest logits, softmax over those alone."""
    z = h @ w["router"].T + w["router.b"]
    val, ids = torch.topk(z, top, dim=-1)
    return ids, torch.softmax(val, dim=-1)


def moe_ff(h, w, mlp):
    top, limit = int(mlp["router"]["top"]), float(mlp["expert"]["limit"])
    ids, weights = route(h, w, top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(ids[t, j])
            out[t] += weights[t, j] * expert(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], limit)[0]
    return out


# ------------------------------------------------------------------ the model
def sub(tensors, prefix):
    return {k[len(prefix):]: v.to(F64) for k, v in tensors.items() if k.startswith(prefix)}


def forward(config, tensors, tokens, return_layers=False):
    """Logits [T, vocab] of a whole sequence (and the stream after every layer, if asked)."""
    eps = float(config["norm"]["eps"])
    t64 = {k: v.to(F64) for k, v in tensors.items()}
    x = t64["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float(config["embedding"]["scale"])
    results, after = [x], []
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h = norm_around_zero(x, t64[p + "norm1"], eps)
        w = sub(tensors, p + "mix.")
        if layer["type"] == "latent_attention":
            y = latent_attention(h, w, layer["mixer"], eps)
        elif layer["type"] == "gla":
            y, _ = gla(h, w, layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + norm_around_zero(y, t64[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = norm_around_zero(x, t64[p + "norm2"], eps)
            w = sub(tensors, p + "mlp.")
            y = dense_ff(h, w) if layer["mlp"]["kind"] == "dense" else moe_ff(h, w, layer["mlp"])
            x = x + norm_around_zero(y, t64[p + "norm2b"], eps)
        results.append(x)
        mix = t64[p + "dwa"]
        x = sum(mix[j] * results[j] for j in range(i + 2))
        after.append(x)
    logits = norm_around_zero(x, t64["final.norm"], eps) @ t64["head"].T
    return (logits, after) if return_layers else logits


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
