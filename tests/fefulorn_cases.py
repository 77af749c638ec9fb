"""Small Fefulorn configurations for the tests, each with random weights of its own, and helpers that build one
mixer of the package and run it piece by piece on a kernel set. The configurations differ from one another in every
size and option: which mixer comes first and which layer is the first that blends its values, grouped and ungrouped
heads, values narrower than, as wide as and wider than keys, rotation over all of a head, part of it and none,
stretched and unstretched positions, windows shorter and longer than a page, layers without a window, latents
narrower and wider than a head, states that are no multiple of four, norm parts of one and of several heads, filters
of two to five taps, layers without feed-forward, routers with and without groups, with top 1 and top = experts,
with and without the shared expert, widths that are no multiple of 8."""
from __future__ import annotations

import types

import torch


def _attn(heads, kv_heads, dim, vdim, scale, window=None, rot=None, v_mix=False, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "v_mix": v_mix}
    if window:
        m["mask"] = {"size": window}
    if rot:
        base, dims, factor = rot
        m["rot"] = {"base": base, "dims": dims}
        if factor is not None:
            m["rot"]["scaling"] = {"factor": factor}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def _latent(heads, dim, vdim, q_rank, kv_rank, scale, window=None, mlp=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def _ssm(heads, vdim, state, groups, norm_groups, conv, mlp=None):
    return {"type": "mamba2", "mlp": mlp,
            "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv}}


def _moe(ff, limit, experts, top, groups=None, shared=None):
    r = {"experts": experts, "top": top}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": r}
    if shared:
        mlp["shared"] = {"ff": shared[0], "limit": shared[1]}
    return mlp


# begins with the state-space mixer; the first blending layer is layer 2, a layer between does not blend; grouped
# heads; values wider than keys; a window shorter than a page; a layer without feed-forward
FEFU_A = {
    "architecture": "Fefulorn", "vocab": 211, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.5},
    "logit_scale": 0.7,
    "layers": [
        _ssm(4, 8, 6, 2, 1, 3, _moe(24, 0.7, 6, 2, (3, 2), (20, 1.2))),
        _attn(4, 2, 8, 12, 0.3, 11, (100.0, 4, 3.0), False, _moe(16, 2.0, 4, 4)),
        _attn(6, 3, 8, 12, 0.4, 40, (1000.0, 8, None), True, None),
        _latent(3, 8, 6, 10, 12, 0.4, 21, _moe(24, 1.0, 6, 1, (2, 1), (8, 0.5))),
        _attn(3, 3, 10, 12, 0.25, None, None, True, _moe(8, 1.5, 3, 1)),
        _attn(6, 3, 16, 12, 0.2, 9, (50.0, 2, 1.5), True, _moe(12, 1.0, 8, 3, (4, 2))),
    ]}
FEFU_A_INIT = dict(seed=41, std=0.12, embedding_std=0.4, norm_jitter=0.1)

# begins with the latent attention; nothing a power of two; a width that is no multiple of 8; one head; no scale on
# the logits; a state-space layer whose norm parts cut through heads
FEFU_B = {
    "architecture": "Fefulorn", "vocab": 97, "width": 76, "norm": {"eps": 3e-6}, "embedding": {"scale": 1.0},
    "layers": [
        _latent(1, 10, 14, 18, 20, 0.25, None, _moe(20, 1.5, 5, 2, None, (12, 2.0))),
        _ssm(3, 10, 7, 3, 5, 2, None),
        _attn(5, 1, 6, 4, 0.5, 17, (500.0, 6, 4.0), True, _moe(10, 0.8, 6, 3, (2, 2))),
        _ssm(2, 12, 5, 1, 2, 5, _moe(14, 1.0, 2, 2)),
        _attn(3, 1, 6, 4, 0.45, 33, None, True, None),
    ]}
FEFU_B_INIT = dict(seed=42, std=0.1, embedding_std=0.7, norm_jitter=0.2)

# sizes in multiples of 16 throughout (what the matrix-core kernels take), heads of 32 and 64
FEFU_C = {
    "architecture": "Fefulorn", "vocab": 128, "width": 96, "norm": {"eps": 1e-6}, "embedding": {"scale": 4.0},
    "logit_scale": 1.5,
    "layers": [
        _attn(4, 2, 32, 32, 0.18, 48, (10000.0, 16, 2.0), True, _moe(32, 1.25, 8, 2, (4, 2), (48, 1.5))),
        _latent(4, 32, 16, 48, 64, 0.15, 72, _moe(32, 1.0, 4, 2)),
        _ssm(4, 16, 16, 2, 2, 4, _moe(16, 3.0, 4, 4, None, (16, 1.0))),
        _attn(2, 2, 64, 32, 0.125, 20, (20000.0, 64, None), True, _moe(32, 1.0, 8, 3, (2, 1))),
        _latent(16, 16, 16, 32, 32, 0.25, None, None),
    ]}
FEFU_C_INIT = dict(seed=43, std=0.12, embedding_std=0.3, norm_jitter=0.05)

CASES = {"a": (FEFU_A, FEFU_A_INIT), "b": (FEFU_B, FEFU_B_INIT), "c": (FEFU_C, FEFU_C_INIT)}


def random_case(seed):
    """A configuration drawn from a seed: one to five layers, every size and option drawn on its own."""
    import random
    rng = random.Random(seed)
    layers = []
    kv_width = None                                 # layers that blend share the shape of their values
    for _ in range(rng.choice([1, 2, 3, 4, 5])):
        mlp = None
        if rng.random() < 0.8:
            count = rng.choice([1, 1, 2, 3, 4])
            per = rng.choice([1, 2, 3])
            keep = rng.randint(1, count)
            experts = count * per
            mlp = _moe(rng.choice([4, 8, 24, 40]), rng.choice([0.5, 1.0, 7.0]), experts, rng.randint(1, min(keep * per, 4)),
                       (count, keep) if count > 1 or rng.random() < 0.3 else None,
                       (rng.choice([4, 12, 32]), rng.choice([0.5, 1.5])) if rng.random() < 0.6 else None)
        kind = rng.choice(["attention", "attention", "latent_attention", "mamba2"])
        window = rng.choice([None, 2, 5, 16, 23, 64, 100])
        if kind == "attention":
            v_mix = rng.random() < 0.6
            kv = rng.choice([1, 2, 3])
            vdim = rng.choice([3, 8, 16, 24, 32])
            if v_mix:
                if kv_width is None:
                    kv_width = (kv, vdim)
                kv, vdim = kv_width
            dim = rng.choice([4, 6, 16, 32, 48, 64])
            rot = None
            if rng.random() < 0.75:
                rot = (rng.choice([10.0, 10000.0, 500000.0]), rng.choice(range(2, dim + 1, 2)), rng.choice([None, 1.0, 2.0, 8.0]))
            layers.append(_attn(kv * rng.choice([1, 2, 4]), kv, dim, vdim, rng.choice([dim ** -0.5, 0.2, 0.5]), window, rot, v_mix, mlp))
        elif kind == "latent_attention":
            dim = rng.choice([2, 5, 8, 16, 48])
            layers.append(_latent(rng.choice([1, 2, 3, 6, 9]), dim, rng.choice([3, 8, 16, 40]), rng.choice([4, 9, 32, 64]),
                                  rng.choice([4, 7, 16, 32, 48, 64, 96, 128]), rng.choice([dim ** -0.5, 0.2, 0.5]), window, mlp))
        else:
            groups = rng.choice([1, 2, 3])
            heads = groups * rng.choice([1, 2, 3])
            vdim = rng.choice([4, 8, 12, 16, 32])
            parts = rng.choice([d for d in (1, 2, 3, 4, 6, 8) if (heads * vdim) % d == 0])
            layers.append(_ssm(heads, vdim, rng.choice([3, 4, 8, 16, 33, 64]), groups, parts, rng.choice([2, 3, 4, 4, 8]), mlp))
    raw = {"architecture": "Fefulorn", "vocab": rng.choice([50, 97, 256]), "width": rng.choice([16, 24, 40, 64, 96, 200]),
           "norm": {"eps": rng.choice([1e-6, 1e-5])}, "embedding": {"scale": rng.choice([1.0, 2.5, 8.0])},
           "logit_scale": rng.choice([1.0, 0.5, 3.0]), "layers": layers}
    return raw, dict(seed=seed, std=0.15, embedding_std=0.5, norm_jitter=0.1)


def make_folder(tmp_path_factory, name, dtype="bfloat16"):
    from tests.conftest import make_folder as make
    raw, init = random_case(name) if isinstance(name, int) else CASES[name]
    return make(tmp_path_factory, "fefulorn_" + str(name), dict(raw, architectures=[raw["architecture"]]), init, dtype)


# ------------------------------------------------------------------ one mixer of the package, piece by piece
def _r(g, dtype):
    return lambda *shape, s=1.0: (s * torch.randn(*shape, generator=g)).to(dtype)


def attention_tensors(g, W, m, dtype=torch.float32):
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    r = _r(g, dtype)
    return {"q": r(H * D, W, s=W ** -0.5), "q.b": r(H * D, s=0.3), "k": r(G * D, W, s=W ** -0.5), "k.b": r(G * D, s=0.3),
            "v": r(G * Dv, W, s=W ** -0.5), "v.b": r(G * Dv, s=0.3), "o": r(W, H * Dv, s=(H * Dv) ** -0.5),
            "vmix": torch.tensor(0.35, dtype=dtype)}


def latent_tensors(g, W, m, dtype=torch.float32):
    H, D, Dv, Q, C = (m[k] for k in ("heads", "dim", "vdim", "q_rank", "kv_rank"))
    r = _r(g, dtype)
    return {"dq": r(Q, W, s=W ** -0.5), "dq.norm": 1 + 0.2 * r(Q), "uq": r(H * D, Q, s=Q ** -0.5 * 2),
            "dkv": r(C, W, s=W ** -0.5 * 2), "dkv.norm": 1 + 0.2 * r(C), "uk": r(H * D, C, s=C ** -0.5 * 2),
            "uv": r(H * Dv, C, s=C ** -0.5), "o": r(W, H * Dv, s=(H * Dv) ** -0.5)}


def ssm_tensors(g, W, m, dtype=torch.float32):
    H, P, N, G, K = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner, ch = H * P, H * P + 2 * G * N
    r = _r(g, dtype)
    return {"in": r(2 * inner + 2 * G * N + H, W, s=W ** -0.5 * 1.5), "conv": r(ch, K, s=0.5), "conv.b": r(ch, s=0.2),
            "dt_bias": (r(H) - 1.0).to(dtype), "A_log": (r(H, s=0.5) - 0.5).to(dtype), "D": 1 + 0.3 * r(H),
            "norm": 1 + 0.2 * r(inner), "o": r(W, inner, s=inner ** -0.5)}


def runtime(ops, dtype="float32", device="cpu", positions=512):
    from return_amd.parts.runtime import Runtime
    rt = Runtime(device, dtype, ops=ops)
    rt.position_limit = positions
    return rt


def build_attention(rt, W, m, w, shared=None, first_of_blend=False):
    """A BlendAttention of the package with the plain function's tensors; shared: {"rows": TokenRows} when it blends."""
    from return_amd.parts.attention import BlendAttention
    from return_amd.parts.position import RotaryPosition
    shared = dict(shared or {})
    rot = m.get("rot")
    if rot:
        shared["p"] = RotaryPosition({"head_dim": m["dim"], "rotary_dim": rot["dims"], "theta": rot["base"],
                                      "max_position": None, "exact_tables": True,
                                      "linear_factor": (rot.get("scaling") or {}).get("factor", 1.0)}, {}, rt)
    params = {"hidden_size": W, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
              "value_dim": m["vdim"], "scale": m["scale"], "window": (m.get("mask") or {}).get("size"),
              "position": "p" if rot else None, "value_rows": "rows" if m.get("v_mix") else None,
              "first_of_blend": first_of_blend}
    roles = {"q_proj": "q", "q_bias": "q.b", "k_proj": "k", "k_bias": "k.b", "v_proj": "v", "v_bias": "v.b", "o_proj": "o"}
    if m.get("v_mix"):
        roles["blend"] = "vmix"
    return BlendAttention(params, {role: w[name].to(rt.dtype).to(rt.device) for role, name in roles.items()}, rt, shared)


def build_latent(rt, W, m, w, eps):
    from return_amd.parts.attention import LatentAttention
    params = {"hidden_size": W, "num_heads": m["heads"], "head_dim": m["dim"], "rot_dim": 0, "value_dim": m["vdim"],
              "q_rank": m["q_rank"], "kv_rank": m["kv_rank"], "scale": m["scale"], "eps": eps, "position": None,
              "sink": False, "gate": False, "window": (m.get("mask") or {}).get("size")}
    roles = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o"}
    return LatentAttention(params, {role: w[name].to(rt.dtype).to(rt.device) for role, name in roles.items()}, rt, {})


def build_ssm(rt, W, m, w, eps):
    from return_amd.parts.ssm import ScalarStateSpace
    params = {"hidden_size": W, "num_heads": m["heads"], "value_dim": m["vdim"], "state_dim": m["state"],
              "groups": m["groups"], "norm_groups": m["norm_groups"], "conv_taps": m["conv"], "eps": eps}
    roles = {"in_proj": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "A_log": "A_log", "skip": "D",
             "o_norm": "norm", "o_proj": "o"}
    return ScalarStateSpace(params, {role: w[name].to(rt.dtype).to(rt.device) for role, name in roles.items()}, rt)


def run_in_pieces(parts, xs, pieces, P=16, pages=(2, 0, 3, 1), slot=1):
    """Every part of `parts` (mixers of one model, in order) forward over its rows xs[i] [T, W] of one request cut into
    the given pieces, each on pools of its own with the pages in a shuffled order (a paged mixer) or on a state slot
    that is not the first (a mixer with state); all parts see the same step, as the layers of a model do. Returns the
    list of results [T, W]."""
    from return_amd.cache.spec import PagedKVSpec
    rt = parts[0].rt
    dev, dt = rt.device, rt.dtype
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    T = xs[0].shape[0]
    caches, tile_rows = [], set()
    for part in parts:
        spec = part.cache_spec()
        if isinstance(spec, PagedKVSpec):
            if len(pages) * P < T:
                raise ValueError("too few pages for these rows")
            caches.append(types.SimpleNamespace(
                group=0, k_pool=torch.zeros(max(pages) + 2, spec.num_kv_heads, P, spec.head_dim, dtype=dt, device=dev),
                v_pool=torch.zeros(max(pages) + 2, spec.num_kv_heads, P,
                                   spec.head_dim if spec.value_dim is None else spec.value_dim, dtype=dt, device=dev)))
        else:
            caches.append(types.SimpleNamespace(tensors={
                name: torch.zeros(slot + 2, *shape, dtype=getattr(torch, kind), device=dev) for name, shape, kind in spec.tensors}))
        tile_rows |= set((part.step_needs() if hasattr(part, "step_needs") else {}).get("prefill_tile_rows", ()))
    outs, at = [[] for _ in parts], 0
    for n in pieces:
        pos = list(range(at, at + n))
        tiles = {rows: i32([[0, off] for off in range(0, n, rows)]) for rows in tile_rows} if n > 1 else {}
        paged = len(pages) * P >= T                 # (parts with state alone need no pages)
        grp = types.SimpleNamespace(page_table=i32(list(pages)), cu_pages=i32([0, len(pages)]), kv_start=i32([0]),
                                    slot_mapping=i32([pages[p // P] * P + p % P for p in pos]) if paged else None)
        step = types.SimpleNamespace(groups=[grp], n_seqs=1, n_tokens=n, cu_q=i32([0, n]), q_start=i32([at]),
                                     positions=i32(pos), all_decode=n == 1, max_q_len=n, slot_ids=i32([slot]),
                                     cu_q_host=[0, n], slot_ids_host=[slot], n_decode=1 if n == 1 else 0,
                                     n_prefill_tokens=0 if n == 1 else n, decode_segs=None, prefill_toks=None,
                                     prefill_tiles=tiles, q_lens=[n], q_starts=[at], max_decode_seq_len=at + n if n == 1 else 0,
                                     max_seq_len=at + n)
        for i, part in enumerate(parts):
            outs[i].append(part.forward(xs[i][at:at + n].to(dt).to(dev).contiguous(), step, caches[i]).float().cpu())
        at += n
    assert at == T
    return [torch.cat(o, dim=0) for o in outs]
