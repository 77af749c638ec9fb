"""Small Safilorn configurations for the tests, each with random weights of its own, and a helper that runs one
mixer of the package piece by piece on a kernel set. The configurations differ from one another in every size and
option: the order of the two mixers, head counts of one and of odd numbers, latents narrower and wider than a head,
rows that are no multiple of four, rotation over all of the rotated part and over its first elements only, with and
without stretched frequencies, decay exponents of one and more, layers without feed-forward, routers of top 1 and
top 3, a stream width that is no multiple of 8, embedding factors of 1 and others."""
from __future__ import annotations

import types

import torch


def _latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, dims, stretch=None, mlp=None):
    rot = {"base": base, "dims": dims}
    if stretch is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), stretch))
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                      "scale": scale, "rot": rot}}


def _gla(heads, dim, vdim, tau, rank, mlp=None):
    return {"type": "gla", "mlp": mlp, "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank}}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(ff, limit, experts, top):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


# begins with the recurrent mixer; odd head counts; a latent whose rows are no multiple of four; a layer without
# feed-forward; rotation over the first half of the rotated part in one layer
SAFI_A = {
    "architecture": "Safilorn", "vocab": 211, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
    "layers": [
        _gla(3, 8, 12, 4.0, 5, _moe(24, 0.7, 6, 3)),
        _latent(5, 8, 4, 12, 20, 24, 0.3, 100.0, 4, (4.0, 16, 8.0, 1.0), _dense(40)),
        _gla(1, 16, 8, 1.0, 3, None),
        _latent(2, 6, 8, 10, 12, 10, 0.45, 10000.0, 4, None, _moe(16, 2.0, 3, 1)),
    ]}
SAFI_A_INIT = dict(seed=31, std=0.12, embedding_std=0.4, norm_jitter=0.1)

# begins with attention; nothing a power of two; a width that is no multiple of 8; one head; a factor of 1
SAFI_B = {
    "architecture": "Safilorn", "vocab": 97, "width": 76, "norm": {"eps": 3e-6}, "embedding": {"scale": 1.0},
    "layers": [
        _latent(1, 10, 6, 14, 18, 20, 0.25, 500.0, 6, (3.0, 24, 6.0, 2.0), _moe(20, 1.5, 5, 2)),
        _latent(7, 4, 2, 6, 28, 12, 0.5, 50.0, 2, None, None),
        _gla(2, 12, 20, 9.0, 7, _dense(52)),
    ]}
SAFI_B_INIT = dict(seed=32, std=0.1, embedding_std=0.7, norm_jitter=0.2)

# sizes in multiples of 16 throughout
SAFI_C = {
    "architecture": "Safilorn", "vocab": 128, "width": 96, "norm": {"eps": 1e-6}, "embedding": {"scale": 9.797958971132712},
    "layers": [
        _latent(4, 32, 16, 48, 48, 64, 0.15, 10000.0, 16, (8.0, 64, 16.0, 1.0), _moe(32, 1.25, 8, 2)),
        _gla(2, 64, 64, 8.0, 16, _dense(128)),
        _gla(4, 16, 32, 2.0, 16, _moe(64, 3.0, 4, 4)),
    ]}
SAFI_C_INIT = dict(seed=33, std=0.12, embedding_std=0.3, norm_jitter=0.05)

CASES = {"a": (SAFI_A, SAFI_A_INIT), "b": (SAFI_B, SAFI_B_INIT), "c": (SAFI_C, SAFI_C_INIT)}


def random_case(seed):
    """A configuration drawn from a seed: one to four layers, every size and option drawn on its own."""
    import random
    rng = random.Random(seed)
    layers = []
    for _ in range(rng.choice([1, 2, 3, 4])):
        mlp = rng.choice([None, "dense", "moe", "moe"])
        if mlp == "dense":
            mlp = _dense(rng.choice([8, 20, 48, 72]))
        elif mlp == "moe":
            experts = rng.choice([1, 2, 5, 8, 12])
            mlp = _moe(rng.choice([4, 8, 24, 40]), rng.choice([0.5, 1.0, 7.0]), experts, rng.randint(1, min(experts, 4)))
        if rng.random() < 0.5:
            rot_dim = rng.choice([2, 4, 6, 16, 16, 32, 64])
            dims = rng.choice(range(2, rot_dim + 1, 2))
            stretch = (rng.choice([2.0, 4.0, 40.0]), rng.choice([8, 32, 512]), rng.choice([4.0, 32.0]), rng.choice([0.5, 1.0])) \
                if rng.random() < 0.7 else None
            dim = rng.choice([2, 5, 8, 16, 48])
            layers.append(_latent(rng.choice([1, 2, 3, 6, 9]), dim, rot_dim, rng.choice([3, 8, 16, 40]),
                                  rng.choice([4, 9, 32, 64]), rng.choice([4, 7, 16, 32, 48, 64, 96, 128, 160]),
                                  rng.choice([(dim + rot_dim) ** -0.5, 0.2, 0.5]), rng.choice([10.0, 10000.0, 500000.0]), dims,
                                  stretch, mlp))
        else:
            layers.append(_gla(rng.choice([1, 2, 3, 5]), rng.choice([2, 4, 12, 16, 40, 64]), rng.choice([3, 8, 16, 33, 64]),
                               rng.choice([1.0, 2.5, 16.0]), rng.choice([1, 4, 16]), mlp))
    raw = {"architecture": "Safilorn", "vocab": rng.choice([50, 97, 256]), "width": rng.choice([16, 24, 40, 64, 96, 200]),
           "norm": {"eps": rng.choice([1e-6, 1e-5])}, "embedding": {"scale": rng.choice([1.0, 2.5, 8.0])}, "layers": layers}
    return raw, dict(seed=seed, std=0.15, embedding_std=0.5, norm_jitter=0.1)


def make_folder(tmp_path_factory, name, dtype="bfloat16"):
    from tests.conftest import make_folder as make
    raw, init = random_case(name) if isinstance(name, int) else CASES[name]
    return make(tmp_path_factory, "safilorn_" + str(name), dict(raw, architectures=[raw["architecture"]]), init, dtype)


# ------------------------------------------------------------------ one mixer of the package, piece by piece
def latent_tensors(g, W, m, dtype=torch.float32):
    H, D, R, Dv, Q, C = (m[k] for k in ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank"))
    r = lambda *shape, s=1.0: (s * torch.randn(*shape, generator=g)).to(dtype)
    return {"dq": r(Q, W, s=W ** -0.5), "dq.norm": 1 + 0.2 * r(Q), "uq": r(H * (D + R), Q, s=Q ** -0.5 * 2),
            "dkv": r(C + R, W, s=W ** -0.5 * 2), "dkv.norm": 1 + 0.2 * r(C), "uk": r(H * D, C, s=C ** -0.5 * 2),
            "uv": r(H * Dv, C, s=C ** -0.5), "sink": r(H), "g": r(H, W, s=W ** -0.5), "o": r(W, H * Dv, s=(H * Dv) ** -0.5)}


def gla_tensors(g, W, m, rank, dtype=torch.float32):
    H, D, V = m["heads"], m["dim"], m["vdim"]
    r = lambda *shape, s=1.0: (s * torch.randn(*shape, generator=g)).to(dtype)
    return {"q": r(H * D, W, s=W ** -0.5), "k": r(H * D, W, s=W ** -0.5), "v": r(H * V, W, s=W ** -0.5),
            "g": r(H * V, W, s=W ** -0.5), "o": r(W, H * V, s=(H * V) ** -0.5), "norm": 1 + 0.2 * r(V),
            "a1": r(rank, W, s=W ** -0.5), "a2": r(H * D, rank, s=rank ** -0.5), "a2.b": (2.0 + r(H * D)).to(dtype)}


def build_latent(ops, W, m, w, eps, max_pos, dtype="float32", device="cpu"):
    from return_amd.parts.attention import LatentAttention
    from return_amd.parts.position import RotaryPosition
    from return_amd.parts.runtime import Runtime
    rt = Runtime(device, dtype, ops=ops)
    rot = m["rot"]
    position = RotaryPosition({"head_dim": m["rot_dim"], "rotary_dim": rot["dims"], "theta": rot["base"],
                               "max_position": max_pos, "exact_tables": True, "scaling": rot.get("scaling")}, {}, rt)
    params = {"hidden_size": W, "num_heads": m["heads"], "head_dim": m["dim"], "rot_dim": m["rot_dim"],
              "value_dim": m["vdim"], "q_rank": m["q_rank"], "kv_rank": m["kv_rank"], "scale": m["scale"], "eps": eps,
              "position": "p", "sink": True, "gate": True}
    roles = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv",
             "sink": "sink", "gate": "g", "o": "o"}
    return LatentAttention(params, {role: w[name].to(rt.dtype).to(device) for role, name in roles.items()}, rt, {"p": position})


def build_gla(ops, W, m, w, eps, dtype="float32", device="cpu"):
    from return_amd.parts.delta import GatedLinearAttention
    from return_amd.parts.runtime import Runtime
    rt = Runtime(device, dtype, ops=ops)
    params = {"hidden_size": W, "num_heads": m["heads"], "head_dim": m["dim"], "value_dim": m["vdim"], "tau": m["tau"],
              "eps": eps, "decay_rank": None}
    roles = {"q_proj": "q", "k_proj": "k", "v_proj": "v", "g_proj": "g", "o_proj": "o", "o_norm": "norm",
             "a1_proj": "a1", "a2_proj": "a2", "a2_bias": "a2.b"}
    return GatedLinearAttention(params, {role: w[name].to(rt.dtype).to(device) for role, name in roles.items()}, rt)


def run_mixer_in_pieces(part, x, pieces, P=16, pages=(2, 0, 3, 1), slot=1):
    """part.forward over the rows x [T, W] of one request cut into the given pieces, on pages in a shuffled order
    (a paged mixer) or on a state slot (a mixer with state). Returns [T, W]."""
    from return_amd.cache.spec import PagedKVSpec
    rt = part.rt
    dev, dt = rt.device, rt.dtype
    spec = part.cache_spec()
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    paged = isinstance(spec, PagedKVSpec)
    if paged and len(pages) * P < x.shape[0]:
        raise ValueError("too few pages for these rows")
    if paged:
        cache = types.SimpleNamespace(group=0,
                                      k_pool=torch.zeros(max(pages) + 2, 1, P, spec.head_dim, dtype=dt, device=dev),
                                      v_pool=torch.zeros(max(pages) + 2, 1, P, spec.value_dim, dtype=dt, device=dev))
    else:
        cache = types.SimpleNamespace(tensors={name: torch.zeros(slot + 2, *shape, dtype=getattr(torch, kind), device=dev)
                                               for name, shape, kind in spec.tensors})
    tile_rows = (part.step_needs() if hasattr(part, "step_needs") else {}).get("prefill_tile_rows", ())
    out, at = [], 0
    for n in pieces:
        pos = list(range(at, at + n))
        tiles = {rows: i32([[0, off] for off in range(0, n, rows)]) for rows in tile_rows} if n > 1 else {}
        grp = types.SimpleNamespace(page_table=i32(list(pages)), cu_pages=i32([0, len(pages)]), kv_start=i32([0]),
                                    slot_mapping=i32([pages[p // P] * P + p % P for p in pos]) if paged else None)
        step = types.SimpleNamespace(groups=[grp], n_seqs=1, n_tokens=n, cu_q=i32([0, n]), q_start=i32([at]),
                                     positions=i32(pos), all_decode=n == 1, max_q_len=n, slot_ids=i32([slot]),
                                     cu_q_host=[0, n], slot_ids_host=[slot], n_decode=1 if n == 1 else 0,
                                     n_prefill_tokens=0 if n == 1 else n, decode_segs=None, prefill_toks=None,
                                     prefill_tiles=tiles, q_lens=[n], q_starts=[at], max_decode_seq_len=at + n if n == 1 else 0)
        out.append(part.forward(x[at:at + n].to(dt).to(dev).contiguous(), step, cache))
        at += n
    assert at == x.shape[0]
    return torch.cat(out, dim=0)
