"""Typed configuration of the Dumizen architecture, read from a checkpoint's config.json.

The file names the design under `architecture`; sizes and constants are nested by what they belong to: `width`, `vocab`,
`norm.eps`, `loop` (start, stop, times; absent: no layer runs twice) and `layers`, a list whose entries give the mixer's
`type` ("attention", "attention_2" or "parallel"), its sizes under `mixer`, and the feed-forward under `mlp` (null: none):
`kind` "moe" with `expert.ff`, `router` {experts, top, scale, `groups` {count, keep}} and `shared` {ff} (absent: no shared
expert).  Mixer sizes: heads, kv_heads, dim, vdim, scale; `rot` {base, dims, `scaling` {factor, original, fast, slow}};
"attention" adds `mask` {size, pool}; "attention_2" adds `softcap` and `q_temp` {coef, every}; "parallel" holds `left`
(an attention's sizes), `right` {heads, dim, vdim, decay, rot} and the two scales.  Everything is checked here, before any
weight is read.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .menitar import DEFAULT_MAX_POSITION, _need, _positive
from .spec import ConfigError


@dataclass(frozen=True)
class BandScaling:
    """Rotary frequencies of lanes that turn more than `fast` times over `original` positions stay, those of lanes that turn
    fewer than `slow` times are divided by `factor`, the lanes between are mixed along a ramp; cos and sin grow by
    0.1 ln(factor) + 1."""
    factor: float
    original: int
    fast: float
    slow: float


@dataclass(frozen=True)
class Rotation:
    dims: int
    base: float
    scaling: Optional[BandScaling]


@dataclass(frozen=True)
class AttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[Rotation] = None
    window: Optional[int] = None       # "attention": tokens a row sees, itself included
    pool: Optional[int] = None         # "attention": positions of a block that is seen as one key behind the window
    softcap: Optional[float] = None    # "attention_2"
    temp_coef: float = 0.0             # "attention_2": q *= 1 + coef * ln(floor((p + 1) / every) + 1)
    temp_every: int = 1


@dataclass(frozen=True)
class RetentionSizes:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot: Optional[Rotation]


@dataclass(frozen=True)
class DumizenMixer:
    kind: str                                  # "attention", "attention_2" or "parallel"
    attention: AttentionSizes                  # the mixer itself, or the left one of a parallel pair
    retention: Optional[RetentionSizes] = None
    left_scale: float = 1.0
    right_scale: float = 1.0


@dataclass(frozen=True)
class DumizenMLP:
    ff: int
    experts: int
    top: int
    route_scale: float
    groups: int                  # 1: every expert can be chosen
    groups_kept: int
    shared_ff: int               # 0: no shared expert


@dataclass(frozen=True)
class DumizenLayer:
    mixer: DumizenMixer
    mlp: Optional[DumizenMLP]


@dataclass(frozen=True)
class DumizenConfig:
    width: int
    vocab: int
    eps: float
    layers: Tuple[DumizenLayer, ...]
    loop: Optional[Tuple[int, int, int]]      # (start, stop, times)
    max_position: int

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @staticmethod
    def from_dict(cfg: Dict[str, Any]) -> "DumizenConfig":
        width = _positive(cfg, "width", "")
        vocab = _positive(cfg, "vocab", "")
        eps = _need(_need(cfg, "norm", dict, ""), "eps", float, "norm.")
        if not eps > 0.0:
            raise ConfigError(f"norm.eps must be positive, is {eps}")
        raw_layers = _need(cfg, "layers", list, "")
        if not raw_layers:
            raise ConfigError("layers must list at least one layer")
        layers = tuple(_layer(raw, f"layers[{i}].") for i, raw in enumerate(raw_layers))
        loop = None
        if cfg.get("loop") is not None:
            raw = cfg["loop"]
            start, stop, times = _need(raw, "start", int, "loop."), _need(raw, "stop", int, "loop."), _positive(raw, "times", "loop.")
            if not 0 <= start < stop <= len(layers):
                raise ConfigError(f"loop.start {start} and loop.stop {stop} must name a run of the {len(layers)} layers")
            loop = (start, stop, times)
        max_position = cfg.get("max_position", DEFAULT_MAX_POSITION)
        if isinstance(max_position, bool) or not isinstance(max_position, int) or max_position <= 0:
            raise ConfigError(f"max_position must be a positive integer, is {max_position!r}")
        return DumizenConfig(width, vocab, eps, layers, loop, max_position)


def _rotation(m, where: str, dim: int) -> Optional[Rotation]:
    rot = m.get("rot")
    if rot is None:
        return None
    rw = where + "rot."
    dims, base = _need(rot, "dims", int, rw), _need(rot, "base", float, rw)
    if dims < 0 or dims % 2 != 0 or dims > dim:
        raise ConfigError(f"{rw}dims must be even and at most dim {dim}, is {dims}")
    if dims == 0:
        return None
    if not base > 1.0:
        raise ConfigError(f"{rw}base must be above 1, is {base}")
    scaling = None
    if rot.get("scaling") is not None:
        sc, sw = rot["scaling"], rw + "scaling."
        scaling = BandScaling(_need(sc, "factor", float, sw), _positive(sc, "original", sw), _need(sc, "fast", float, sw),
                              _need(sc, "slow", float, sw))
        if not (scaling.factor > 0.0 and scaling.fast > 0.0 and scaling.slow > 0.0):
            raise ConfigError(f"{sw}factor, fast and slow must be positive, is {sc!r}")
    return Rotation(dims, base, scaling)


def _attention(m, where: str, kind: str) -> AttentionSizes:
    heads, kv_heads = _positive(m, "heads", where), _positive(m, "kv_heads", where)
    if heads % kv_heads != 0:
        raise ConfigError(f"{where}heads {heads} is not a multiple of kv_heads {kv_heads}")
    dim, vdim = _positive(m, "dim", where), _positive(m, "vdim", where)
    extra = {}
    if kind == "attention":
        mask = _need(m, "mask", dict, where)
        extra.update(window=_positive(mask, "size", where + "mask."), pool=_positive(mask, "pool", where + "mask."))
    elif kind == "attention_2":
        softcap = _need(m, "softcap", float, where)
        if not softcap > 0.0:
            raise ConfigError(f"{where}softcap must be positive, is {softcap}")
        extra.update(softcap=softcap)
        if m.get("q_temp") is not None:       # absent: the queries keep their temperature of 1
            temp = _need(m, "q_temp", dict, where)
            extra.update(temp_coef=_need(temp, "coef", float, where + "q_temp."), temp_every=_positive(temp, "every", where + "q_temp."))
    elif vdim != dim:          # the left mixer of a pair: its keys are its values
        raise ConfigError(f"{where}vdim {vdim} must equal dim {dim}: the values of this mixer are its keys")
    rot = None if kind == "attention_2" else _rotation(m, where, dim)
    return AttentionSizes(heads, kv_heads, dim, vdim, _need(m, "scale", float, where), rot, **extra)


def _layer(raw, where: str) -> DumizenLayer:
    kind = _need(raw, "type", str, where)
    m, mw = _need(raw, "mixer", dict, where), where + "mixer."
    if kind in ("attention", "attention_2"):
        mixer = DumizenMixer(kind, _attention(m, mw, kind))
    elif kind == "parallel":
        right, rw = _need(m, "right", dict, mw), mw + "right."
        heads, dim, vdim = _positive(right, "heads", rw), _positive(right, "dim", rw), _positive(right, "vdim", rw)
        decay = _need(right, "decay", list, rw)
        if len(decay) != heads or not all(isinstance(d, (int, float)) and not isinstance(d, bool) and 0.0 < d <= 1.0 for d in decay):
            raise ConfigError(f"{rw}decay must list a number in (0, 1] for each of the {heads} heads, is {decay!r}")
        retention = RetentionSizes(heads, dim, vdim, tuple(float(d) for d in decay), _rotation(right, rw, dim))
        mixer = DumizenMixer(kind, _attention(_need(m, "left", dict, mw), mw + "left.", "left"), retention,
                             _need(m, "left_scale", float, mw), _need(m, "right_scale", float, mw))
    else:
        raise ConfigError(f"{where}type {kind!r} is no mixer of this design (known: 'attention', 'attention_2', 'parallel')")
    raw_mlp = raw.get("mlp")
    mlp = None
    if raw_mlp is not None:
        pw = where + "mlp."
        mlp_kind = _need(raw_mlp, "kind", str, pw)
        if mlp_kind != "moe":
            raise ConfigError(f"{pw}kind {mlp_kind!r} is no feed-forward of this design (known: 'moe')")
        router, rw = _need(raw_mlp, "router", dict, pw), pw + "router."
        experts, top = _positive(router, "experts", rw), _positive(router, "top", rw)
        groups, kept = 1, 1
        if router.get("groups") is not None:
            groups, kept = _positive(router["groups"], "count", rw + "groups."), _positive(router["groups"], "keep", rw + "groups.")
        if experts % groups != 0 or kept > groups:
            raise ConfigError(f"{rw}groups: {experts} experts do not form {groups} equal groups of which {kept} are kept")
        if top > kept * (experts // groups):
            raise ConfigError(f"{rw}top {top} is more than the {kept * (experts // groups)} experts of the kept groups")
        shared = raw_mlp.get("shared")
        mlp = DumizenMLP(_positive(_need(raw_mlp, "expert", dict, pw), "ff", pw + "expert."), experts, top,
                         _need(router, "scale", float, rw), groups, kept,
                         0 if shared is None else _positive(shared, "ff", pw + "shared."))
    return DumizenLayer(mixer, mlp)
