"""Typed configuration of the Venadra architecture, read from a checkpoint's config.json.

The file names the design under `architecture`; sizes and constants are nested by what they belong to: `width`, `vocab`,
`embedding.scale`, `norm.eps`, `canon.taps` (the causal convolution on every mixer's input; absent: none) and `layers`,
a list whose entries give the mixer's `type` ("lightning" or "attention"), its sizes under `mixer` (lightning: heads,
dim, vdim, `decay` with one number a head; attention: heads, kv_heads, dim, vdim, scale, `mask` {size}) and the
feed-forward under `mlp`: null for none, `kind` "dense" with ff, or `kind` "moe" with `expert` {ff, limit} and `router`
{experts, top, scale}.  An entry with `weights_of`: j runs layer j's tensors with a cache or state of its own.
Everything is checked here, before any weight is read.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .menitar import DEFAULT_MAX_POSITION, _need, _positive
from .spec import ConfigError


@dataclass(frozen=True)
class VenadraMixer:
    kind: str                      # "lightning" or "attention"
    heads: int
    dim: int
    vdim: int
    kv_heads: int = 0              # attention
    scale: float = 1.0             # attention
    chunk: Optional[int] = None    # attention: positions see their own chunk of this many positions; None: all before them
    decay: Tuple[float, ...] = ()  # lightning: one number a head


@dataclass(frozen=True)
class VenadraMLP:
    kind: str                      # "dense" or "moe"
    ff: int                        # lanes of the dense layer, or of one expert
    limit: float = 0.0             # moe: what an expert's gate and up are clamped to
    experts: int = 0
    top: int = 0
    router_scale: float = 1.0


@dataclass(frozen=True)
class VenadraLayer:
    mixer: VenadraMixer
    mlp: Optional[VenadraMLP]
    weights_of: Optional[int]      # the layer whose tensors this one runs; None: its own


@dataclass(frozen=True)
class VenadraConfig:
    width: int
    vocab: int
    embedding_scale: float
    eps: float
    taps: int                      # 0: no convolution on the mixers' inputs
    layers: Tuple[VenadraLayer, ...]
    max_position: int

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @staticmethod
    def from_dict(cfg: Dict[str, Any]) -> "VenadraConfig":
        width = _positive(cfg, "width", "")
        vocab = _positive(cfg, "vocab", "")
        eps = _need(_need(cfg, "norm", dict, ""), "eps", float, "norm.")
        if not eps > 0.0:
            raise ConfigError(f"norm.eps must be positive, is {eps}")
        taps = 0
        if cfg.get("canon") is not None:
            taps = _positive(_need(cfg, "canon", dict, ""), "taps", "canon.")
        raw_layers = _need(cfg, "layers", list, "")
        if not raw_layers:
            raise ConfigError("layers must list at least one layer")
        layers = []
        for i, raw in enumerate(raw_layers):
            layer = _layer(raw, f"layers[{i}].")
            j = layer.weights_of
            if j is not None:
                if not 0 <= j < len(raw_layers) or j == i or (isinstance(raw_layers[j], dict) and raw_layers[j].get("weights_of") is not None):
                    raise ConfigError(f"layers[{i}].weights_of {j} must name another layer that holds tensors of its own")
            layers.append(layer)
        for i, layer in enumerate(layers):
            if layer.weights_of is not None:
                owner = layers[layer.weights_of]
                if (layer.mixer, layer.mlp) != (owner.mixer, owner.mlp):
                    raise ConfigError(f"layers[{i}] runs the tensors of layers[{layer.weights_of}] but names other sizes")
        max_position = cfg.get("max_position", DEFAULT_MAX_POSITION)
        if isinstance(max_position, bool) or not isinstance(max_position, int) or max_position <= 0:
            raise ConfigError(f"max_position must be a positive integer, is {max_position!r}")
        return VenadraConfig(width, vocab, _need(_need(cfg, "embedding", dict, ""), "scale", float, "embedding."), eps, taps,
                             tuple(layers), max_position)


def _layer(raw, where: str) -> VenadraLayer:
    kind = _need(raw, "type", str, where)
    m = _need(raw, "mixer", dict, where)
    mw = where + "mixer."
    heads, dim, vdim = _positive(m, "heads", mw), _positive(m, "dim", mw), _positive(m, "vdim", mw)
    if kind == "lightning":
        decay = _need(m, "decay", list, mw)
        if len(decay) != heads or any(isinstance(d, bool) or not isinstance(d, (int, float)) for d in decay):
            raise ConfigError(f"{mw}decay must hold one number for each of the {heads} heads, is {decay!r}")
        mixer = VenadraMixer("lightning", heads, dim, vdim, decay=tuple(float(d) for d in decay))
    elif kind == "attention":
        kv_heads = _positive(m, "kv_heads", mw)
        if heads % kv_heads != 0:
            raise ConfigError(f"{mw}heads {heads} is not a multiple of kv_heads {kv_heads}")
        mask = m.get("mask")
        chunk = None if mask is None else _positive(mask, "size", mw + "mask.")
        mixer = VenadraMixer("attention", heads, dim, vdim, kv_heads=kv_heads, scale=_need(m, "scale", float, mw), chunk=chunk)
    else:
        raise ConfigError(f"{where}type {kind!r} is no mixer of this design (known: 'lightning', 'attention')")
    raw_mlp = raw.get("mlp")
    mlp = None
    if raw_mlp is not None:
        pw = where + "mlp."
        mlp_kind = _need(raw_mlp, "kind", str, pw)
        if mlp_kind == "dense":
            mlp = VenadraMLP("dense", _positive(raw_mlp, "ff", pw))
        elif mlp_kind == "moe":
            router = _need(raw_mlp, "router", dict, pw)
            experts, top = _positive(router, "experts", pw + "router."), _positive(router, "top", pw + "router.")
            if top > experts:
                raise ConfigError(f"{pw}router.top {top} is more than router.experts {experts}")
            one = _need(raw_mlp, "expert", dict, pw)
            limit = _need(one, "limit", float, pw + "expert.")
            if not limit > 0.0:
                raise ConfigError(f"{pw}expert.limit must be positive, is {limit}")
            mlp = VenadraMLP("moe", _positive(one, "ff", pw + "expert."), limit=limit, experts=experts, top=top,
                             router_scale=_need(router, "scale", float, pw + "router."))
        else:
            raise ConfigError(f"{pw}kind {mlp_kind!r} is no feed-forward of this design (known: 'dense', 'moe')")
    weights_of = raw.get("weights_of")
    if weights_of is not None and (isinstance(weights_of, bool) or not isinstance(weights_of, int)):
        raise ConfigError(f"{where}weights_of must be an integer, is {weights_of!r}")
    return VenadraLayer(mixer, mlp, weights_of)
