"""Venadra, written out plainly: one function per mechanism, float64 NumPy, token by token where a recurrence is
defined that way.  It reads the configuration dictionary and a name -> array dictionary of weights directly and shares
no code with the engine; the tests compare the engine with it.

Notation: x the residual stream [T, width]; h what a mixer or feed-forward reads; positions count from 0.
"""
import math

import numpy as np


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    x = np.asarray(x, dtype=np.float64)
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def scalar_norm(x, g, eps):
    """RMS norm whose weight is one number for all coordinates."""
    return rms(x, eps) * float(np.asarray(g, dtype=np.float64).reshape(-1)[0])


def input_convolution(h, w):
    """h + conv(h): conv(h)_t = sum_j w[:, j] * h_(t - taps + 1 + j), zeros before the sequence's start.  h [T, width],
    w [width, taps]."""
    T, width = h.shape
    taps = w.shape[1]
    out = h.copy()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def lightning(h, wq, wk, wv, wg, wo, norm_w, decay, heads, dim, vdim, eps):
    """Linear attention with a decay a head, one token after the other: S <- decay * S + k v^T, o = S^T q."""
    T = h.shape[0]
    q = silu(h @ wq.T).reshape(T, heads, dim)
    k = silu(h @ wk.T).reshape(T, heads, dim)
    v = silu(h @ wv.T).reshape(T, heads, vdim)
    o = np.zeros((T, heads, vdim))
    for a in range(heads):
        S = np.zeros((dim, vdim))
        for t in range(T):
            S = float(decay[a]) * S + np.outer(k[t, a], v[t, a])
            o[t, a] = S.T @ q[t, a]
    o = rms(o.reshape(T, heads * vdim), eps) * norm_w
    return (o * sigmoid(h @ wg.T)) @ wo.T


def chunk_attention(h, wq, wk, wv, wg, wo, sink, heads, kv_heads, dim, vdim, scale, chunk, eps):
    """Grouped-query attention without positions: q and k normed over a head's lanes, keys of the row's own chunk of
    positions up to the row, a sink in the softmax's denominator, a gate lane by lane on the output."""
    T = h.shape[0]
    q = rms((h @ wq.T).reshape(T, heads, dim), eps)
    k = rms((h @ wk.T).reshape(T, kv_heads, dim), eps)
    v = (h @ wv.T).reshape(T, kv_heads, vdim)
    per = heads // kv_heads
    out = np.zeros((T, heads, vdim))
    for i in range(T):
        lo = (i // chunk) * chunk if chunk else 0
        for a in range(heads):
            b = a // per
            s = (k[lo:i + 1, b] @ q[i, a]) * scale
            top = max(s.max(), float(sink[a]))
            e = np.exp(s - top)
            out[i, a] = (e @ v[lo:i + 1, b]) / (e.sum() + math.exp(float(sink[a]) - top))
    return (out.reshape(T, heads * vdim) * sigmoid(h @ wg.T)) @ wo.T


def polynorm_ff(h, w_up, w_down, act, eps):
    """W_down (a N(z) + b N(z^2) + c N(z^3) + e), z = W_up h, N = division by the root mean square over ff."""
    z = h @ w_up.T
    a, b, c, e = (float(t) for t in act)
    y = a * rms(z, eps) + b * rms(z * z, eps) + c * rms(z * z * z, eps) + e
    return y @ w_down.T


def expert(h, w_gate, w_up, w_down, limit):
    g = np.minimum(h @ w_gate.T, limit)
    u = np.clip(h @ w_up.T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w_down.T


def routed_ff(h, w_router, experts, top, limit, router_scale):
    """Softmax router over all experts, the `top` largest, their scores over their sum times a constant."""
    T = h.shape[0]
    z = h @ w_router.T
    z = z - z.max(-1, keepdims=True)
    s = np.exp(z)
    s = s / s.sum(-1, keepdims=True)
    out = np.zeros((T, experts[0][2].shape[0]))
    for t in range(T):
        picks = np.argsort(-s[t], kind="stable")[:top]
        w = s[t, picks] / (s[t, picks].sum() + 1e-20) * router_scale
        for p, e in enumerate(picks):
            out[t] += w[p] * expert(h[t:t + 1], *experts[e], limit)[0]
    return out


def forward(config, weights, tokens, collect_layers=False):
    """Logits [T, vocab] of one sequence (and the residual stream after every layer run)."""
    W = {n: np.asarray(t, dtype=np.float64) for n, t in weights.items()}
    eps = float(config["norm"]["eps"])
    taps = int(config["canon"]["taps"]) if config.get("canon") else 0
    x = W["embed"][np.asarray(tokens)] * float(config["embedding"]["scale"])
    streams = []
    for i, layer in enumerate(config["layers"]):
        p = "l%d." % layer.get("weights_of", i)
        m = layer["mixer"]
        h = scalar_norm(x, W[p + "norm1"], eps)
        if taps:
            h = input_convolution(h, W[p + "canon1"])
        mx = p + "mix."
        if layer["type"] == "lightning":
            x = x + lightning(h, W[mx + "q"], W[mx + "k"], W[mx + "v"], W[mx + "g"], W[mx + "o"], W[mx + "norm"], m["decay"],
                              m["heads"], m["dim"], m["vdim"], eps)
        elif layer["type"] == "attention":
            mask = m.get("mask")
            x = x + chunk_attention(h, W[mx + "q"], W[mx + "k"], W[mx + "v"], W[mx + "g"], W[mx + "o"], W[mx + "sink"],
                                    m["heads"], m["kv_heads"], m["dim"], m["vdim"], float(m["scale"]),
                                    int(mask["size"]) if mask else 0, eps)
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp is not None:
            h = scalar_norm(x, W[p + "norm2"], eps)
            f = p + "mlp."
            if mlp["kind"] == "dense":
                x = x + polynorm_ff(h, W[f + "up"], W[f + "down"], W[f + "act"], eps)
            else:
                r = mlp["router"]
                experts = [(W[f + "e%d.gate" % e], W[f + "e%d.up" % e], W[f + "e%d.down" % e]) for e in range(r["experts"])]
                x = x + routed_ff(h, W[f + "router"], experts, r["top"], float(mlp["expert"]["limit"]), float(r["scale"]))
        streams.append(x.copy())
    logits = scalar_norm(x, W["final.norm"], eps) @ W["head"].T
    return (logits, np.stack(streams)) if collect_layers else logits


def greedy(config, weights, prompt, count):
    tokens = list(prompt)
    for _ in range(count):
        tokens.append(int(np.argmax(forward(config, weights, tokens)[-1])))
    return tokens[len(prompt):]
