"""Dumizen: the description of the architecture in terms of parts.

x = E[token].  A layer norms each part's input and its output: x += rms_1b(mixer(rms_1(x))), then x += rms_2b(ff(rms_2(x)))
(`parts/block.py: SandwichBlock`, no layer scale, no constant).  Three mixers.  "attention": grouped-query attention with
biased projections, every head of q and of k normed with one weight vector, rotary with band-wise frequency scaling
(`parts/rope.py`, "yarn"), and a window of tokens with pooled blocks of older tokens behind it
(`parts/normed_attention.py`).  "attention_2": sigmoid attention without positions but a query temperature, a capped score
and a bias by distance (`parts/sigmoid_attention.py`).  "parallel": two mixers on the same input, their outputs added with
a constant each (`parts/pair.py`): on the left attention whose keys are its values, normed over whole projections, rotated,
with a zero sink and an output gate (`parts/normed_attention.py`); on the right retention, linear attention with a decay a
head over rotated queries and scaled keys, every head divided by its root mean square and gated with a silu
(`parts/lightning.py`).  The feed-forward is a set of small experts W_down relu(W_up n)^2 picked by a sigmoid router with
corrections and groups, beside one shared expert (`parts/experts.py`).  The layers loop.start .. loop.stop - 1 run
loop.times times in a row with the same weights and a cache and state of their own each pass; every pass begins with
x <- W_in [x; E[token]] + step_t (`parts/stream.py: PassMix`).  logits = E rms(x) with the embedding table itself.

Tensor names: `embed`, `loop.in`, `loop.step`, `final.norm`, and per layer `l<i>.norm1`, `l<i>.norm1b`, `l<i>.norm2`,
`l<i>.norm2b`, `l<i>.mix.*` (q, k, v, o with `.b` biases, `q.norm`, `k.norm`, `r1`, `r2`, `pb`, or `left.*` and `right.*`) and
`l<i>.mlp.{router,correction}`, `l<i>.mlp.e<j>.{up,down}`, `l<i>.mlp.shared.{up,down}`.
"""
from __future__ import annotations

from ..config.dumizen import DumizenConfig
from ..config.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from ..registry import Architecture, register_architecture


def _position(rot, max_position):
    if rot is None:
        return None
    position = {"kind": "rotary", "dims": rot.dims, "theta": rot.base, "pairing": "half", "scaling": "none",
                "max_position": max_position, "precise": True}
    if rot.scaling is not None:
        s = rot.scaling
        position.update(scaling="yarn", factor=s.factor, original_max_position=s.original, beta_fast=s.fast, beta_slow=s.slow)
    return position


def _attention_sizes(cfg, a):
    return {"hidden_size": cfg.width, "num_heads": a.heads, "num_kv_heads": a.kv_heads, "head_dim": a.dim,
            "value_head_dim": a.vdim, "scale": a.scale}


def _mixer(cfg: DumizenConfig, m, p: str) -> PartSpec:
    a = m.attention
    if m.kind == "attention":
        names = {"q": f"{p}q", "k": f"{p}k", "v": f"{p}v", "o": f"{p}o", "q_bias": f"{p}q.b", "k_bias": f"{p}k.b", "v_bias": f"{p}v.b",
                 "q_norm": f"{p}q.norm", "k_norm": f"{p}k.norm"}
        return PartSpec("normed_attention",
                        dict(_attention_sizes(cfg, a), qk_norm="head", qk_norm_eps=cfg.eps, window=a.window, pool=a.pool,
                             position=_position(a.rot, cfg.max_position)), names)
    if m.kind == "attention_2":
        names = {"q": f"{p}q", "k": f"{p}k", "v": f"{p}v", "o": f"{p}o", "q_bias": f"{p}q.b", "k_bias": f"{p}k.b", "v_bias": f"{p}v.b",
                 "o_bias": f"{p}o.b", "r1": f"{p}r1", "r2": f"{p}r2", "pb": f"{p}pb"}
        return PartSpec("sigmoid_attention",
                        dict(_attention_sizes(cfg, a), softcap=a.softcap, temp_coef=a.temp_coef, temp_every=a.temp_every), names)
    r = m.retention
    left = PartSpec("normed_attention",
                    dict(_attention_sizes(cfg, a), qk_norm="projection", qk_norm_eps=cfg.eps, values="keys", sink="zero",
                         output_gate=True, position=_position(a.rot, cfg.max_position)),
                    {"q": f"{p}left.q", "k": f"{p}left.k", "g": f"{p}left.g", "o": f"{p}left.o", "q_norm": f"{p}left.q.norm",
                     "k_norm": f"{p}left.k.norm"})
    right = PartSpec("lightning_attention",
                     {"hidden_size": cfg.width, "num_heads": r.heads, "head_dim": r.dim, "value_head_dim": r.vdim, "decay": r.decay,
                      "eps": cfg.eps, "activation": "none", "head_norm": True, "gate_activation": "silu",
                      "key_scale": r.dim ** -0.5, "position": _position(r.rot, cfg.max_position)},
                     {n: f"{p}right.{n}" for n in ("q", "k", "v", "g", "o")})
    tensors = {"left." + n: t for n, t in left.tensors.items()}
    tensors.update({"right." + n: t for n, t in right.tensors.items()})
    return PartSpec("mixer_pair", {"size": cfg.width, "left": left, "right": right, "left_scale": m.left_scale,
                                   "right_scale": m.right_scale}, tensors)


def build_spec(cfg: DumizenConfig) -> ModelSpec:
    layers = []
    ignorable = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        norm = lambda name: PartSpec("rms", {"size": cfg.width, "eps": cfg.eps}, {"weight": f"{p}.{name}"})
        mixer = _mixer(cfg, layer.mixer, f"{p}.mix.")
        norms = {"mixer": norm("norm1"), "mixer_out": norm("norm1b")}
        ffn = None
        if layer.mlp is None:
            ignorable += [f"{p}.norm2", f"{p}.norm2b"]
        else:
            mlp = layer.mlp
            norms.update(feed_forward=norm("norm2"), feed_forward_out=norm("norm2b"))
            names = {"router": f"{p}.mlp.router", "correction": f"{p}.mlp.correction"}
            for e in range(mlp.experts):
                names.update({f"up_{e}": f"{p}.mlp.e{e}.up", f"down_{e}": f"{p}.mlp.e{e}.down"})
            if mlp.shared_ff:
                names.update(shared_up=f"{p}.mlp.shared.up", shared_down=f"{p}.mlp.shared.down")
            ffn = PartSpec("routed_experts",
                           {"hidden_size": cfg.width, "intermediate_size": mlp.ff, "experts": mlp.experts, "top": mlp.top,
                            "score": "sigmoid", "renormalize": True, "route_scale": mlp.route_scale, "weight_on": "output",
                            "gated": False, "groups": mlp.groups, "groups_kept": mlp.groups_kept, "shared": mlp.shared_ff}, names)
        block = PartSpec("sandwich", {"size": cfg.width, "residual_mult": 1.0})
        layers.append(LayerSpec(block=block, mixer=mixer, feed_forward=ffn, norms=norms))
    n = len(cfg.layers)
    if cfg.loop is None:
        order = [RunEntry(layer=i) for i in range(n)]
        ignorable += ["loop.in", "loop.step"]
    else:
        start, stop, times = cfg.loop
        order = [RunEntry(layer=i) for i in range(start)]
        for t in range(times):
            enter = PartSpec("pass_mix", {"size": cfg.width, "row": t, "rows": times}, {"mix": "loop.in", "steps": "loop.step"})
            order += [RunEntry(layer=i, before=enter if i == start else None) for i in range(start, stop)]
        order += [RunEntry(layer=i) for i in range(stop, n)]
    table = {"weight": "embed"}
    return ModelSpec(
        architecture="dumizen",
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_position=cfg.max_position,
        embedding=PartSpec("table", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "scale": 1.0}, table),
        layers=tuple(layers),
        run_order=tuple(order),
        final_norm=PartSpec("rms", {"size": cfg.width, "eps": cfg.eps}, {"weight": "final.norm"}),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": cfg.width}, table),
        ignorable_tensors=tuple(ignorable),
    )


register_architecture(Architecture(
    model_type="dumizen",
    hf_architectures=(),
    parse_config=DumizenConfig.from_dict,
    build_spec=build_spec,
))
