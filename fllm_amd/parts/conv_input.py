"""A causal convolution over time on a mixer's input: the mixer reads h + conv(h) instead of h,
conv(h)_t = sum_j w[:, j] * h_(t - taps + 1 + j) on every channel, zeros before a sequence's start.

`ConvInput` wraps any mixer (`inner`: the wrapped mixer's PartSpec): it keeps the last taps - 1 inputs of every live request
in a state of its own beside whatever the wrapped mixer keeps, convolves, and hands the result on.  Cache, state, portions
and graphs are the wrapped mixer's; its tensors are listed under `inner.<name>`.
"""
from __future__ import annotations

from types import SimpleNamespace

import torch

from ..registry import part_class, register_part
from .base import INIT_MATRIX, Mixer, StateNeed, take_prepared

_TAIL = "conv_inputs"      # the name of the wrapper's own state


class ConvInput(Mixer):
    @classmethod
    def tensor_shapes(cls, spec):
        inner = spec["inner"]
        shapes = {"conv": ((spec["size"], spec["taps"]), INIT_MATRIX)}
        for name, shape in part_class("mixer", inner.kind).tensor_shapes(inner).items():
            shapes["inner." + name] = shape
        return shapes

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.size = int(spec["size"])
        self.taps = int(spec["taps"])
        if not 1 <= self.taps <= 16:
            raise ValueError(f"a convolution of {self.taps} taps is outside 1..16")
        self.w = rt.vector(weights["conv"])                   # float32 [size, taps]
        inner = spec["inner"]
        own = {name[len("inner."):]: t for name, t in weights.items() if name.startswith("inner.")}
        self.inner = part_class("mixer", inner.kind)(inner, own, rt)
        self.graph_safe = bool(getattr(self.inner, "graph_safe", False))
        need = self.inner.state_need()
        self._inner_names = None if need is None else (list(need) if isinstance(need, dict) else "")
        if isinstance(need, dict) and _TAIL in need:
            raise ValueError(f"the wrapped mixer names a state {_TAIL!r} itself")

    def cache_need(self):
        return self.inner.cache_need()

    def portion_multiple(self) -> int:
        return self.inner.portion_multiple()

    def state_need(self):
        need = self.inner.state_need()
        out = {} if need is None else (dict(need) if isinstance(need, dict) else {"": need})
        if self.taps > 1:
            out[_TAIL] = StateNeed((self.taps - 1, self.size), self.rt.dtype)
        return out or None

    def _inner_binding(self, binding):
        """The binding as the wrapped mixer expects it: its own state alone, named as it named it."""
        if self._inner_names is None:
            state = None
        elif self._inner_names == "":
            state = binding.state[""]
        else:
            state = {name: binding.state[name] for name in self._inner_names}
        return SimpleNamespace(group=binding.group, k_pages=binding.k_pages, v_pages=binding.v_pages, page_size=binding.page_size,
                               writes=binding.writes, state=state)

    def _tail(self, binding):
        return binding.state[_TAIL] if self.taps > 1 else None

    def forward(self, ctx, h, residual, binding, **kw) -> None:
        out = self.rt.empty(tuple(h.shape))
        self.rt.ops.short_conv(h, self.w, self._tail(binding), ctx.row_seg, ctx.seg_start, ctx.slots, out)
        self.inner.forward(ctx, out, residual, self._inner_binding(binding), **kw)

    def forward_from_residual(self, ctx, residual, norm, binding, **kw) -> bool:
        """Steps of one row a request: the norm before the mixer and the convolution are one kernel."""
        ops = self.rt.ops
        fused = getattr(ops, "norm_short_conv", None)
        prologue = getattr(norm, "fused_prologue", lambda: None)()
        if fused is None or prologue is None or not ctx.uniform_rows:
            return False
        take_prepared(ctx, norm, residual)          # whatever was prepared for this norm is not used here
        out = self.rt.empty(tuple(residual.shape))
        fused(residual, prologue[0], prologue[1], self.w, self._tail(binding), ctx.row_seg, ctx.slots, out)
        self.inner.forward(ctx, out, residual, self._inner_binding(binding), **kw)
        return True

    @property
    def stores_branch(self):
        return bool(getattr(self.inner, "stores_branch", False))

    @property
    def branch_parts(self):
        return int(getattr(self.inner, "branch_parts", 1))


register_part("mixer", "conv_input", ConvInput)
