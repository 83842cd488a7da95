"""Venadra: the description of the architecture in terms of parts.

x = E[token] * embedding.scale.  A layer is pre-norm: x += mixer(n1(x)), then x += ff(n2(x)), every norm an RMS norm with ONE
learned number for all coordinates (`parts/norm.py: ScalarRMSNorm`).  What a mixer reads is first replaced by h + conv(h), a
causal convolution of `canon.taps` taps over time on every channel (`parts/conv_input.py`, which wraps the mixer and keeps
the last taps - 1 inputs of every sequence).  Two mixers: "lightning", linear attention with a decay a head carried as a
float32 matrix a head and sequence, its heads normed together and gated (`parts/lightning.py`); and "attention",
grouped-query attention without positions whose q and k heads are divided by their root mean square, with a score scale from
the file, keys visible inside the row's own chunk of positions, a learned sink a head in the softmax's denominator and an
output gate sigmoid(W_g h) (`parts/attention.py`).  Two feed-forwards: dense, W_down PolyNorm(W_up h)
(`parts/mlp.py: PolyNormMLP`), or routed: small clamped gated experts, a softmax router over all experts, the `top` largest
scores renormalized and scaled, weights on the experts' outputs (`parts/experts.py`).  A layer with `weights_of`: j runs
layer j's tensors with a cache and state of its own: the run order names layer j again.  logits = head rms(x).

Tensor names: `embed`, `head`, `final.norm`, and per layer `l<i>.norm1`, `l<i>.norm2`, `l<i>.canon1`, `l<i>.mix.{q,k,v,g,o}`
with `l<i>.mix.norm` (lightning) or `l<i>.mix.sink` (attention), and `l<i>.mlp.{up,down,act}` or `l<i>.mlp.router` with
`l<i>.mlp.e<j>.{gate,up,down}`.
"""
from __future__ import annotations

from ..config.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from ..config.venadra import VenadraConfig
from ..registry import Architecture, register_architecture

EXPERT_ALPHA = 1.702       # an expert's activation: g * sigmoid(1.702 g) * (u + 1)
EXPERT_UP_OFFSET = 1.0


def build_spec(cfg: VenadraConfig) -> ModelSpec:
    layers = []
    index_of = {}          # layer of the file -> its place among the layers that hold tensors
    ignorable = []
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        p, m = f"l{i}", layer.mixer
        norm = lambda name: PartSpec("rms_scalar", {"size": cfg.width, "eps": cfg.eps}, {"weight": f"{p}.{name}"})
        names = {n: f"{p}.mix.{n}" for n in ("q", "k", "v", "g", "o")}
        if m.kind == "lightning":
            mixer = PartSpec("lightning_attention",
                             {"hidden_size": cfg.width, "num_heads": m.heads, "head_dim": m.dim, "value_head_dim": m.vdim,
                              "decay": m.decay, "eps": cfg.eps, "activation": "silu"},
                             dict(names, norm=f"{p}.mix.norm"))
        else:
            mixer = PartSpec("attention",
                             {"hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                              "value_head_dim": m.vdim, "scale": m.scale, "chunk": m.chunk, "position": None,
                              "qk_norm_eps": cfg.eps, "sink": True, "output_gate": True, "widen_heads": True},
                             dict(names, sink=f"{p}.mix.sink"))
        if cfg.taps:
            mixer = PartSpec("conv_input", {"size": cfg.width, "taps": cfg.taps, "inner": mixer},
                             dict({"inner." + n: t for n, t in mixer.tensors.items()}, conv=f"{p}.canon1"))
        ffn = None
        norms = {"mixer": norm("norm1")}
        if layer.mlp is None:
            ignorable.append(f"{p}.norm2")
        else:
            norms["feed_forward"] = norm("norm2")
            if layer.mlp.kind == "dense":
                ffn = PartSpec("polynorm_mlp", {"hidden_size": cfg.width, "intermediate_size": layer.mlp.ff, "eps": cfg.eps},
                               {"up": f"{p}.mlp.up", "down": f"{p}.mlp.down", "act": f"{p}.mlp.act"})
            else:
                tensors = {"router": f"{p}.mlp.router"}
                for e in range(layer.mlp.experts):
                    tensors.update({f"gate_{e}": f"{p}.mlp.e{e}.gate", f"up_{e}": f"{p}.mlp.e{e}.up", f"down_{e}": f"{p}.mlp.e{e}.down"})
                ffn = PartSpec("routed_experts",
                               {"hidden_size": cfg.width, "intermediate_size": layer.mlp.ff, "experts": layer.mlp.experts,
                                "top": layer.mlp.top, "score": "softmax", "renormalize": True, "route_scale": layer.mlp.router_scale,
                                "weight_on": "output", "limit": layer.mlp.limit, "alpha": EXPERT_ALPHA, "up_offset": EXPERT_UP_OFFSET},
                               tensors)
        index_of[i] = len(layers)
        layers.append(LayerSpec(block=PartSpec("prenorm"), mixer=mixer, feed_forward=ffn, norms=norms))
    order = tuple(RunEntry(layer=index_of[i if layer.weights_of is None else layer.weights_of]) for i, layer in enumerate(cfg.layers))
    return ModelSpec(
        architecture="venadra",
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_position=cfg.max_position,
        embedding=PartSpec("table", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "scale": cfg.embedding_scale}, {"weight": "embed"}),
        layers=tuple(layers),
        run_order=order,
        final_norm=PartSpec("rms_scalar", {"size": cfg.width, "eps": cfg.eps}, {"weight": "final.norm"}),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": cfg.width}, {"weight": "head"}),
        ignorable_tensors=tuple(ignorable),
    )


register_architecture(Architecture(
    model_type="venadra",
    hf_architectures=(),
    parse_config=VenadraConfig.from_dict,
    build_spec=build_spec,
))
