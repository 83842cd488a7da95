"""A plain, slow implementation of the Dumizen design in float64 numpy, one function per mechanism.

It shares no code with the product: whole sequences at once, no cache, no pages, no state slots.  Weights are a
dictionary name -> float64 array with the checkpoint's names; the configuration is the config.json dictionary.
`forward(cfg, w, tokens)` returns the logits at every position, `layer_outputs` the stream after every layer run.
"""
import math

import numpy as np


# ---- small functions ------------------------------------------------------------------------------------------------
def unit_rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def relu_squared(z):
    return np.maximum(z, 0.0) ** 2


# ---- rotation -------------------------------------------------------------------------------------------------------
def rotary_angles(dims, base, scaling, positions):
    """(angles [positions, dims / 2], magnitude).  `scaling` None or {factor, original, fast, slow}: lanes that turn often
    keep their frequency, lanes that turn rarely get it divided by the factor, a ramp of lanes between mixes the two."""
    lanes = np.arange(dims // 2, dtype=np.float64)
    freq = base ** (-2.0 * lanes / dims)
    magnitude = 1.0
    if scaling is not None:
        factor, original = float(scaling["factor"]), float(scaling["original"])

        def lane_of(turns):
            return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo = max(math.floor(lane_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(lane_of(float(scaling["slow"]))), dims - 1)
        ramp = np.clip((lanes - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        freq = freq / factor * ramp + freq * (1.0 - ramp)
        magnitude = 0.1 * math.log(factor) + 1.0
    return np.asarray(positions, dtype=np.float64)[:, None] * freq[None, :], magnitude


def rotate(x, rot, positions):
    """x [T, heads, dim]: the first rot.dims lanes of every head turn, lane i with lane i + dims / 2."""
    if rot is None or not rot.get("dims"):
        return x
    dims = int(rot["dims"])
    angles, magnitude = rotary_angles(dims, float(rot["base"]), rot.get("scaling"), positions)
    cos, sin = np.cos(angles)[:, None, :] * magnitude, np.sin(angles)[:, None, :] * magnitude
    half = dims // 2
    u, v = x[..., :half], x[..., half:dims]
    out = x.copy()
    out[..., :half] = u * cos - v * sin
    out[..., half:dims] = v * cos + u * sin
    return out


# ---- mixers ---------------------------------------------------------------------------------------------------------
def pooled_window_attention(q, k, v, scale, size, pool):
    """q [T, H, d], k [T, G, d], v [T, G, dv] as a cache would hold them.  Row i sees the tokens i - size + 1 .. i and,
    for every block of `pool` positions that ends at or before i - size, ONE key and value: the block's means.  One softmax
    over both kinds."""
    T, H, d = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    blocks = T // pool
    k_mean = k[:blocks * pool].reshape(blocks, pool, G, -1).mean(axis=1) if blocks else np.zeros((0, G, d))
    v_mean = v[:blocks * pool].reshape(blocks, pool, G, -1).mean(axis=1) if blocks else np.zeros((0, G, v.shape[2]))
    for i in range(T):
        first = max(0, i - size + 1)
        seen = [b for b in range(blocks) if b * pool + pool - 1 <= i - size]
        for h in range(H):
            g = h // (H // G)
            keys = np.concatenate([k_mean[seen, g], k[first:i + 1, g]], axis=0)
            values = np.concatenate([v_mean[seen, g], v[first:i + 1, g]], axis=0)
            s = keys @ q[i, h] * scale
            p = np.exp(s - s.max())
            out[i, h] = (p / p.sum()) @ values
    return out


def attention_mixer(h, w, p, m, eps, positions):
    """Mixer 'attention': biased projections, a weighted RMS norm over every head of q and of k, rotation, windows with
    pooled blocks."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, d)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, d)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, dv)
    q = unit_rms(q, eps) * w[p + "q.norm"]
    k = unit_rms(k, eps) * w[p + "k.norm"]
    q, k = rotate(q, m.get("rot"), positions), rotate(k, m.get("rot"), positions)
    o = pooled_window_attention(q, k, v, m["scale"], m["mask"]["size"], m["mask"]["pool"])
    return o.reshape(T, H * dv) @ w[p + "o"].T


def sigmoid_attention(q, k, v, scale, softcap, r1, r2, pb):
    """No softmax: every earlier key j weighs sigmoid(cap * tanh(q_i . k_j * scale / cap) - r1_h ln(1 + r2_h (i - j)) + pb_h)."""
    T, H, d = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for i in range(T):
        dist = (i - np.arange(i + 1)).astype(np.float64)
        for h in range(H):
            g = h // (H // G)
            s = k[:i + 1, g] @ q[i, h] * scale
            s = softcap * np.tanh(s / softcap)
            s = s - r1[h] * np.log(1.0 + r2[h] * dist)
            out[i, h] = sigmoid(s + pb[h]) @ v[:i + 1, g]
    return out


def attention_2_mixer(h, w, p, m, positions):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, d)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, d)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, dv)
    pos = np.asarray(positions, dtype=np.float64)
    temp = 1.0 + m["q_temp"]["coef"] * np.log(np.floor((pos + 1.0) / m["q_temp"]["every"]) + 1.0)
    q = q * temp[:, None, None]
    o = sigmoid_attention(q, k, v, m["scale"], m["softcap"], w[p + "r1"], w[p + "r2"], w[p + "pb"])
    return o.reshape(T, H * dv) @ w[p + "o"].T + w[p + "o.b"]


def sink_attention(q, k, v, scale):
    """Causal attention whose softmax has one more term of score 0 that carries no value."""
    T, H, d = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for i in range(T):
        for h in range(H):
            g = h // (H // G)
            s = k[:i + 1, g] @ q[i, h] * scale
            top = max(s.max(), 0.0)
            e = np.exp(s - top)
            out[i, h] = (e / (np.exp(-top) + e.sum())) @ v[:i + 1, g]
    return out


def retention(q, k, v, decay):
    """S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, from S = 0.  q, k [T, H, d], v [T, H, dv]."""
    T, H, d = q.shape
    S = np.zeros((H, d, v.shape[2]))
    out = np.zeros((T, H, v.shape[2]))
    for t in range(T):
        for h in range(H):
            S[h] = decay[h] * S[h] + np.outer(k[t, h], v[t, h])
            out[t, h] = S[h].T @ q[t, h]
    return out


def parallel_mixer(h, w, p, m, eps, positions):
    T = h.shape[0]
    # left: keys double as values, norms over whole projections, a sink, an output gate
    L, lp = m["left"], p + "left."
    H, G, d = L["heads"], L["kv_heads"], L["dim"]
    q_flat, k_flat = h @ w[lp + "q"].T, h @ w[lp + "k"].T
    v = k_flat.reshape(T, G, d)                                 # as projected
    q = (unit_rms(q_flat, eps) * w[lp + "q.norm"]).reshape(T, H, d)
    k = (unit_rms(k_flat, eps) * w[lp + "k.norm"]).reshape(T, G, d)
    q, k = rotate(q, L.get("rot"), positions), rotate(k, L.get("rot"), positions)
    o = sink_attention(q, k, v, L["scale"]).reshape(T, H * d)
    left = (o * sigmoid(h @ w[lp + "g"].T)) @ w[lp + "o"].T
    # right: retention
    R, rp = m["right"], p + "right."
    Hr, dr, dvr = R["heads"], R["dim"], R["vdim"]
    q = rotate((h @ w[rp + "q"].T).reshape(T, Hr, dr), R.get("rot"), positions)
    k = rotate((h @ w[rp + "k"].T).reshape(T, Hr, dr), R.get("rot"), positions) * dr ** -0.5
    v = (h @ w[rp + "v"].T).reshape(T, Hr, dvr)
    o = unit_rms(retention(q, k, v, R["decay"]), eps).reshape(T, Hr * dvr)
    right = (o * silu(h @ w[rp + "g"].T)) @ w[rp + "o"].T
    return m["left_scale"] * left + m["right_scale"] * right


# ---- feed-forward ---------------------------------------------------------------------------------------------------
def route(h, w_router, correction, router):
    """(chosen experts [T, top], their weights [T, top]).  The choice looks at sigmoid scores plus a correction and only
    inside the groups whose two best corrected scores sum highest; the weights are the plain scores of the chosen,
    divided by their sum, times a constant."""
    E, top = router["experts"], router["top"]
    s = sigmoid(h @ w_router.T)
    choice = s + correction
    groups = router.get("groups")
    if groups is not None:
        count, keep = groups["count"], groups["keep"]
        per = E // count
        by_group = choice.reshape(-1, count, per)
        best_two = np.sort(by_group, axis=-1)[..., -2:].sum(-1)
        order = np.argsort(-best_two, axis=-1, kind="stable")[:, :keep]
        allowed = np.zeros((h.shape[0], count), dtype=bool)
        np.put_along_axis(allowed, order, True, axis=1)
        choice = np.where(np.repeat(allowed, per, axis=1), choice, -np.inf)
    ids = np.argsort(-choice, axis=-1, kind="stable")[:, :top]
    picked = np.take_along_axis(s, ids, axis=1)
    weights = picked / (picked.sum(-1, keepdims=True) + 1e-20) * router["scale"]
    return ids, weights


def expert(h, up, down):
    return relu_squared(h @ up.T) @ down.T


def feed_forward(h, w, p, mlp):
    ids, weights = route(h, w[p + "router"], w[p + "correction"], mlp["router"])
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(ids[t], weights[t]):
            out[t] += a * expert(h[t], w[f"{p}e{e}.up"], w[f"{p}e{e}.down"])
    if mlp.get("shared") is not None:
        out = out + expert(h, w[p + "shared.up"], w[p + "shared.down"])
    return out


# ---- the model ------------------------------------------------------------------------------------------------------
def run_order(cfg):
    """(layer, pass or None when the layer starts no pass) for every layer run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if loop is None:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return order + [(i, None) for i in range(loop["stop"], n)]


def layer(x, cfg, w, i, positions):
    spec, eps, p = cfg["layers"][i], cfg["norm"]["eps"], f"l{i}."
    norm = lambda name, t: unit_rms(t, eps) * w[p + name]
    h = norm("norm1", x)
    kind = spec["type"]
    if kind == "attention":
        y = attention_mixer(h, w, p + "mix.", spec["mixer"], eps, positions)
    elif kind == "attention_2":
        y = attention_2_mixer(h, w, p + "mix.", spec["mixer"], positions)
    elif kind == "parallel":
        y = parallel_mixer(h, w, p + "mix.", spec["mixer"], eps, positions)
    else:
        raise ValueError(kind)
    x = x + norm("norm1b", y)
    if spec.get("mlp") is not None:
        x = x + norm("norm2b", feed_forward(norm("norm2", x), w, p + "mlp.", spec["mlp"]))
    return x


def layer_outputs(cfg, w, tokens):
    """The stream after every layer run, [runs, T, width], and the logits [T, vocab]."""
    tokens = np.asarray(tokens)
    positions = np.arange(len(tokens))
    x0 = w["embed"][tokens]
    x = x0.copy()
    after = []
    for i, begins in run_order(cfg):
        if begins is not None:
            x = np.concatenate([x, x0], axis=1) @ w["loop.in"].T + w["loop.step"][begins]
        x = layer(x, cfg, w, i, positions)
        after.append(x.copy())
    logits = (unit_rms(x, cfg["norm"]["eps"]) * w["final.norm"]) @ w["embed"].T
    return np.stack(after), logits


def forward(cfg, w, tokens):
    return layer_outputs(cfg, w, tokens)[1]
