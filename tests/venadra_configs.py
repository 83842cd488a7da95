"""Tiny Venadra configurations and weights for tests.  The weights are drawn here, larger than a checkpoint's random init,
so that scores differ between keys and experts, sinks matter and decays are felt."""
import json
import os

import numpy as np
import torch


def lightning(heads, dim, vdim, decay, mlp=None, weights_of=None):
    out = {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}, "mlp": _mlp(mlp)}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def attention(heads, kv_heads, dim, vdim, chunk=None, scale=None, mlp=None, weights_of=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if chunk is not None:
        mixer["mask"] = {"size": chunk}
    out = {"type": "attention", "mixer": mixer, "mlp": _mlp(mlp)}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def _mlp(mlp):
    """None, ("dense", ff) or ("moe", ff, experts, top, limit, router scale)."""
    if mlp is None:
        return None
    if mlp[0] == "dense":
        return {"kind": "dense", "ff": mlp[1]}
    return {"kind": "moe", "expert": {"ff": mlp[1], "limit": mlp[4]}, "router": {"experts": mlp[2], "top": mlp[3], "scale": mlp[5]}}


def config(width, vocab, layers, taps=None, eps=1e-5, embedding_scale=3.0):
    cfg = {"architecture": "Venadra", "width": width, "vocab": vocab, "embedding": {"scale": embedding_scale}, "norm": {"eps": eps},
           "layers": layers}
    if taps is not None:
        cfg["canon"] = {"taps": taps}
    return cfg


_LA = lightning(2, 16, 24, (0.9, 0.97), mlp=("dense", 80))
_AA = attention(4, 2, 32, 16, chunk=24, scale=0.2, mlp=("moe", 24, 5, 2, 1.5, 2.0))
# A: both mixers, both feed-forwards, layers that run another layer's tensors with a state or cache of their own, a layer
# without feed-forward, keys wider than values, four taps
A = config(64, 96, [_LA, _AA, dict(_LA, weights_of=0), dict(_AA, weights_of=1), lightning(3, 8, 8, (0.5, 0.8, 0.99))], taps=4)
# B: attention alone, as many key/value heads as heads, every expert picked, a router scale of 1, an embedding that is not
# scaled, chunks that are no multiple of the page, two taps
B = config(96, 120, [attention(3, 3, 32, 32, chunk=40, scale=0.11, mlp=("moe", 40, 3, 3, 2.0, 1.0)),
                     attention(3, 3, 32, 32, chunk=40, scale=0.11, mlp=("dense", 112))], taps=2, eps=1e-6, embedding_scale=1.0)
# C: lightning alone (a model without pages), one head, a decay of exactly 1 (nothing is forgotten) beside a fast one,
# head sizes that are multiples of nothing, a single expert, one tap (the convolution keeps no inputs)
C = config(48, 80, [lightning(1, 20, 12, (1.0,), mlp=("moe", 16, 1, 1, 1.0, 0.7)), lightning(2, 6, 10, (0.3, 0.95), mlp=("dense", 64))],
           taps=1)
# D: head sizes the matrix-core attention takes (64 and 64) beside values half as wide (widened in bfloat16), no mask on one
# layer, sixteen experts, no convolution at all
D = config(128, 160, [attention(8, 2, 64, 64, chunk=80, scale=0.125, mlp=("dense", 192)),
                      lightning(2, 64, 64, (0.95, 0.999), mlp=("moe", 48, 16, 4, 1.0, 1.5)),
                      attention(4, 1, 64, 32, scale=0.1, mlp=("moe", 48, 16, 4, 1.0, 1.5)),
                      dict(lightning(2, 64, 64, (0.95, 0.999), mlp=("moe", 48, 16, 4, 1.0, 1.5)), weights_of=1)])
# E: sizes that are multiples of nothing, three heads on one key/value head, values wider than keys, a chunk of 7 positions,
# five taps, two picks of seven experts
E = config(68, 77, [attention(3, 1, 24, 40, chunk=7, scale=0.3, mlp=("moe", 18, 7, 2, 0.8, 1.2)),
                    lightning(3, 10, 6, (0.7, 0.9, 0.999), mlp=("dense", 50))], taps=5, embedding_scale=2.0)
CONFIGS = {"A": A, "B": B, "C": C, "D": D, "E": E}
PAGE_SIZES = {"A": 8, "B": 16, "C": 8, "D": 16, "E": 16}


def bf16_round(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float32)).to(torch.bfloat16).to(torch.float32)


def weights(cfg, seed, decided_router=False):
    """name -> float32 torch tensor whose values are exact in bfloat16 (both precisions load the same numbers).

    `decided_router`: for comparisons in bfloat16, where a random router has close calls that rounding flips, which is a
    large error that says nothing about the kernels.  The first two lanes of the stream then carry a direction that depends
    on the token alone (no output or down projection writes to them), every router row looks at those two lanes only, row e
    along the angle 2 pi e / E, and the tokens' angles lie halfway between the angles at which two experts tie: every pick has
    a margin far above the rounding, and tokens differ in their picks and weights."""
    rng = np.random.default_rng(seed)
    W = cfg["width"]
    out = {"embed": rng.normal(0, 0.4, (cfg["vocab"], W)), "head": rng.normal(0, W ** -0.5, (cfg["vocab"], W)),
           "final.norm": np.array(1 + rng.uniform(-0.3, 0.3))}
    counts = {spec["mlp"]["router"]["experts"] for spec in cfg["layers"] if spec["mlp"] and spec["mlp"]["kind"] == "moe"}
    if decided_router and counts:
        n = max(counts)
        angle = (np.arange(cfg["vocab"]) % (2 * n) + 0.5) * np.pi / n
        out["embed"][:, 0], out["embed"][:, 1] = 1.2 * np.cos(angle), 1.2 * np.sin(angle)
    taps = cfg["canon"]["taps"] if cfg.get("canon") else 0

    def quiet(matrix):             # a projection into the stream that leaves the first two lanes alone
        if decided_router:
            matrix[:2] = 0.0
        return matrix

    for i, spec in enumerate(cfg["layers"]):
        if spec.get("weights_of") is not None:
            continue
        m = spec["mixer"]
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        G = m.get("kv_heads", H)
        p = f"l{i}."
        out[p + "norm1"] = np.array(1 + rng.uniform(-0.3, 0.3))
        if taps:
            out[p + "canon1"] = rng.normal(0, 0.3, (W, taps))
        out[p + "mix.q"] = rng.normal(0, 2 * W ** -0.5, (H * d, W))
        out[p + "mix.k"] = rng.normal(0, 2 * W ** -0.5, (G * d, W))
        if spec["type"] == "lightning":
            # keys lean towards their own queries: a token's product with itself is then well above the rounding of its
            # terms, so the sign of a first token's output (all a norm over the heads keeps of it) is no close call
            out[p + "mix.k"] = 0.6 * out[p + "mix.q"] + 0.8 * out[p + "mix.k"]
        out[p + "mix.v"] = rng.normal(0, W ** -0.5, (G * dv, W))
        out[p + "mix.g"] = rng.normal(0, 2 * W ** -0.5, (H * dv, W))
        out[p + "mix.o"] = quiet(rng.normal(0, (H * dv) ** -0.5, (W, H * dv)))
        if spec["type"] == "lightning":
            out[p + "mix.norm"] = 1 + rng.uniform(-0.3, 0.3, H * dv)
        else:
            out[p + "mix.sink"] = rng.normal(0, 1.5, H)
        mlp = spec["mlp"]
        if mlp is None:
            continue
        out[p + "norm2"] = np.array(1 + rng.uniform(-0.3, 0.3))
        if mlp["kind"] == "dense":
            ff = mlp["ff"]
            out[p + "mlp.up"] = rng.normal(0, 2 * W ** -0.5, (ff, W))
            out[p + "mlp.down"] = quiet(rng.normal(0, ff ** -0.5, (W, ff)))
            out[p + "mlp.act"] = np.array([0.8, 0.5, -0.3, 0.1]) + rng.uniform(-0.1, 0.1, 4)
        else:
            ff, n = mlp["expert"]["ff"], mlp["router"]["experts"]
            out[p + "mlp.router"] = rng.normal(0, 1.5 * W ** -0.5, (n, W))
            if decided_router:
                at = 2 * np.pi * np.arange(n) / n
                out[p + "mlp.router"][:] = 0.0
                out[p + "mlp.router"][:, 0], out[p + "mlp.router"][:, 1] = 5.0 * np.cos(at), 5.0 * np.sin(at)
            for e in range(n):
                out[f"{p}mlp.e{e}.gate"] = rng.normal(0, 2 * W ** -0.5, (ff, W))
                out[f"{p}mlp.e{e}.up"] = rng.normal(0, 2 * W ** -0.5, (ff, W))
                out[f"{p}mlp.e{e}.down"] = quiet(rng.normal(0, ff ** -0.5, (W, ff)))
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
