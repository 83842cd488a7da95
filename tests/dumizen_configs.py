"""Tiny Dumizen configurations and weights for tests.  The weights are drawn here, larger than a checkpoint's random init, so
that scores differ between keys and experts, windows, pooled blocks, sinks and decays are felt."""
import json
import os

import numpy as np
import torch


def _rot(dims, base, scaling=None):
    rot = {"base": base, "dims": dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return rot


def _mlp(mlp):
    """None or (ff, experts, top, scale, (groups, kept) or None, shared ff or None)."""
    if mlp is None:
        return None
    ff, experts, top, scale, groups, shared = mlp
    router = {"experts": experts, "top": top, "scale": scale}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def windowed(heads, kv_heads, dim, vdim, size, pool, rot, scale=None, mlp=None):
    return {"type": "attention", "mlp": _mlp(mlp),
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5,
                      "mask": {"size": size, "pool": pool}, "rot": rot}}


def sigmoid(heads, kv_heads, dim, vdim, softcap, coef, every, scale=None, mlp=None):
    return {"type": "attention_2", "mlp": _mlp(mlp),
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5, "softcap": softcap,
                      "q_temp": {"coef": coef, "every": every}}}


def pair(left, right, left_scale, right_scale, mlp=None):
    """left: (heads, kv_heads, dim, rot, scale); right: (heads, dim, vdim, decays, rot)."""
    heads, kv_heads, dim, rot, scale = left
    rh, rd, rv, decay, rrot = right
    return {"type": "parallel", "mlp": _mlp(mlp),
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "rot": rot},
                      "right": {"heads": rh, "dim": rd, "vdim": rv, "decay": list(decay), "rot": rrot},
                      "left_scale": left_scale, "right_scale": right_scale}}


def config(width, vocab, layers, loop=None, eps=1e-5):
    cfg = {"architecture": "Dumizen", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers}
    if loop is not None:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


_YARN = (4.0, 32, 8.0, 1.0)       # a short original context, so that every band of lanes occurs among sixteen
# A: all three mixers, a loop that does not begin at the first layer, three groups of two experts of which two are kept, a shared
# expert, blocks of four behind windows of twelve on pages of eight, values wider and narrower than keys
A = config(64, 96, [
    sigmoid(4, 2, 16, 24, 5.0, 0.4, 8, mlp=(24, 6, 2, 1.5, (3, 2), 40)),
    windowed(4, 1, 32, 16, 12, 4, _rot(16, 100.0, _YARN), scale=0.2, mlp=(24, 6, 2, 1.5, (3, 2), 40)),
    pair((4, 2, 32, _rot(32, 1000.0, _YARN), 0.15), (2, 16, 24, (0.9, 0.97), _rot(8, 50.0)), 0.7, 1.3, mlp=(24, 6, 2, 1.5, (3, 2), 40)),
    windowed(2, 2, 16, 16, 12, 4, _rot(16, 100.0), scale=0.3),
], loop=(1, 3, 2))
# B: no loop, blocks of ONE position (every token behind the window is its own block), a window that is no multiple of the
# page, one group (every expert can be chosen), every expert of the kept group picked, no shared expert, full rotation, as many
# key/value heads as heads, a temperature that steps every four positions, a decay of exactly 1
B = config(96, 120, [
    windowed(3, 3, 32, 32, 5, 1, _rot(32, 10000.0), mlp=(40, 3, 3, 1.0, None, None)),
    sigmoid(3, 3, 32, 32, 40.0, 0.35, 4, mlp=(40, 4, 2, 1.8, (2, 1), 56)),
    pair((3, 3, 32, _rot(32, 10000.0), 0.18), (1, 32, 32, (1.0,), None), 1.0, 1.0, mlp=(40, 4, 2, 1.8, (2, 1), 56)),
], eps=1e-6)
# C: sizes that are multiples of nothing (keys lie lane by lane in the pages), blocks of three on pages of sixteen (blocks
# straddle pages), a window of seven, the whole model looped three times, four groups of one expert
C = config(68, 77, [
    windowed(3, 1, 12, 10, 7, 3, _rot(6, 30.0, _YARN), scale=0.4, mlp=(18, 4, 2, 0.8, (4, 2), 22)),
    pair((2, 1, 20, _rot(10, 77.0), 0.25), (3, 10, 6, (0.7, 0.9, 0.999), _rot(10, 20.0)), 0.5, 2.0, mlp=(18, 4, 2, 0.8, (4, 2), 22)),
    sigmoid(3, 1, 12, 20, 3.0, 1.0, 5, scale=0.5),
], loop=(0, 3, 3))
# D: head sizes the matrix-core attention takes on the left (64), long windows with blocks of a page, eight experts in four
# groups, a loop of one layer twice in the middle
D = config(128, 160, [
    sigmoid(4, 2, 64, 64, 20.0, 0.25, 32, scale=0.125, mlp=(48, 8, 3, 1.7, (4, 2), 64)),
    windowed(8, 2, 64, 32, 48, 16, _rot(32, 20000.0, (8.0, 64, 16.0, 1.0)), scale=0.1, mlp=(48, 8, 3, 1.7, (4, 2), 64)),
    pair((8, 4, 64, _rot(64, 100000.0, (8.0, 64, 16.0, 1.0)), 0.125), (2, 64, 64, (0.95, 0.999), _rot(64, 100000.0)), 0.9, 1.2,
         mlp=(48, 8, 3, 1.7, (4, 2), 64)),
], loop=(1, 2, 2), eps=1e-6)
CONFIGS = {"A": A, "B": B, "C": C, "D": D}
PAGE_SIZES = {"A": 8, "B": 16, "C": 16, "D": 16}


def bf16_round(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float32)).to(torch.bfloat16).to(torch.float32)


def weights(cfg, seed, decided_router=False):
    """name -> float32 torch tensor whose values are exact in bfloat16 (both precisions load the same numbers).

    `decided_router`: for comparisons in bfloat16, where a random router has close calls that rounding flips, which is a
    large error that says nothing about the kernels.  The first two lanes of the stream then carry a direction that depends on
    the token alone (the norms behind the parts weigh them with zero, the matrix of a pass's input hands them on from the
    embedding), every router row looks at those two lanes only, row e along the angle 2 pi e / E, and the tokens' angles lie a
    quarter of the way between two experts: every pick and every group has a margin far above the rounding."""
    rng = np.random.default_rng(seed)
    W = cfg["width"]
    out = {"embed": rng.normal(0, 0.4, (cfg["vocab"], W)), "final.norm": 1 + rng.uniform(-0.3, 0.3, W)}
    counts = {spec["mlp"]["router"]["experts"] for spec in cfg["layers"] if spec["mlp"]}
    if decided_router:
        E = max(counts)
        angle = (np.arange(cfg["vocab"]) % (2 * E) + 0.5) * np.pi / E
        out["embed"][:, 0], out["embed"][:, 1] = 1.2 * np.cos(angle), 1.2 * np.sin(angle)
    if cfg.get("loop"):
        out["loop.in"] = np.concatenate([np.eye(W) * 0.8, np.eye(W) * 0.3], axis=1) + rng.normal(0, 0.3 * W ** -0.5, (W, 2 * W))
        out["loop.step"] = rng.normal(0, 0.2, (cfg["loop"]["times"], W))
        if decided_router:
            out["loop.in"][:2] = 0.0
            out["loop.in"][0, W], out["loop.in"][1, W + 1] = 1.0, 1.0
            out["loop.step"][:, :2] = 0.0

    def attention(p, m, biases, o_bias):
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        out[p + "q"] = rng.normal(0, 2 * W ** -0.5, (H * d, W))
        out[p + "k"] = rng.normal(0, 2 * W ** -0.5, (G * d, W))
        out[p + "o"] = rng.normal(0, (H * dv) ** -0.5, (W, H * dv))
        if biases:
            out[p + "v"] = rng.normal(0, W ** -0.5, (G * dv, W))
            for n, size in (("q", H * d), ("k", G * d), ("v", G * dv)):
                out[p + n + ".b"] = rng.normal(0, 0.3, size)
        if o_bias:
            out[p + "o.b"] = rng.normal(0, 0.3, W)

    for i, spec in enumerate(cfg["layers"]):
        m, p = spec["mixer"], f"l{i}."
        for name in ("norm1", "norm1b"):
            out[p + name] = 1 + rng.uniform(-0.3, 0.3, W)
        if decided_router:
            out[p + "norm1b"][:2] = 0.0
        if spec["type"] == "attention":
            attention(p + "mix.", m, True, False)
            out[p + "mix.q.norm"], out[p + "mix.k.norm"] = 1 + rng.uniform(-0.4, 0.4, m["dim"]), 1 + rng.uniform(-0.4, 0.4, m["dim"])
        elif spec["type"] == "attention_2":
            attention(p + "mix.", m, True, True)
            H = m["heads"]
            out[p + "mix.r1"], out[p + "mix.r2"] = rng.uniform(0.2, 1.0, H), rng.uniform(0.05, 0.5, H)
            out[p + "mix.pb"] = rng.normal(-1.0, 1.0, H)
        else:
            L, R = m["left"], m["right"]
            attention(p + "mix.left.", L, False, False)
            out[p + "mix.left.g"] = rng.normal(0, 2 * W ** -0.5, (L["heads"] * L["dim"], W))
            out[p + "mix.left.q.norm"] = 1 + rng.uniform(-0.4, 0.4, L["heads"] * L["dim"])
            out[p + "mix.left.k.norm"] = 1 + rng.uniform(-0.4, 0.4, L["kv_heads"] * L["dim"])
            H, d, dv = R["heads"], R["dim"], R["vdim"]
            out[p + "mix.right.q"] = rng.normal(0, 2 * W ** -0.5, (H * d, W))
            # keys lean towards their own queries: a token's product with itself then stands well above the rounding of its
            # terms, so the sign of a first token's output (all the norm of a head keeps of it) is no close call
            out[p + "mix.right.k"] = 0.6 * out[p + "mix.right.q"] + 0.8 * rng.normal(0, 2 * W ** -0.5, (H * d, W))
            out[p + "mix.right.v"] = rng.normal(0, W ** -0.5, (H * dv, W))
            out[p + "mix.right.g"] = rng.normal(0, 2 * W ** -0.5, (H * dv, W))
            out[p + "mix.right.o"] = rng.normal(0, (H * dv) ** -0.5, (W, H * dv))
        mlp = spec["mlp"]
        if mlp is None:
            continue
        for name in ("norm2", "norm2b"):
            out[p + name] = 1 + rng.uniform(-0.3, 0.3, W)
        ff, E = mlp["expert"]["ff"], mlp["router"]["experts"]
        out[p + "mlp.router"] = rng.normal(0, 1.5 * W ** -0.5, (E, W))
        out[p + "mlp.correction"] = rng.normal(0, 0.15, E)
        if decided_router:
            out[p + "norm2b"][:2] = 0.0
            out[p + "norm2"][:2] = 1.0
            at = 2 * np.pi * np.arange(E) / E
            out[p + "mlp.router"][:] = 0.0
            out[p + "mlp.router"][:, 0], out[p + "mlp.router"][:, 1] = 0.6 * np.cos(at), 0.6 * np.sin(at)
            out[p + "mlp.correction"] = rng.normal(0, 0.004, E)
        for e in range(E):
            out[f"{p}mlp.e{e}.up"] = rng.normal(0, 2 * W ** -0.5, (ff, W))
            out[f"{p}mlp.e{e}.down"] = rng.normal(0, ff ** -0.5, (W, ff))
        if mlp.get("shared"):
            out[p + "mlp.shared.up"] = rng.normal(0, 2 * W ** -0.5, (mlp["shared"]["ff"], W))
            out[p + "mlp.shared.down"] = rng.normal(0, mlp["shared"]["ff"] ** -0.5, (W, mlp["shared"]["ff"]))
    return {n: bf16_round(a) for n, a in out.items()}


def to_float64(tensors):
    return {n: t.to(torch.float64).numpy() for n, t in tensors.items()}


def write_model(folder, cfg, tensors, dtype=torch.bfloat16):
    from fllm_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    write_safetensors(os.path.join(folder, "model.safetensors"), {n: t.to(dtype) for n, t in tensors.items()})
    return folder


def random_ids(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, size=n).tolist()
