"""Two mixers side by side: both read the same input, and the result is left_scale * left + right_scale * right.

`MixerPair` wraps two mixers (`left`, `right`: their PartSpecs; their tensors are listed under `left.<name>` and
`right.<name>`).  Either may keep pages (at most one of them: a run entry has one place in a cache group) and either may
keep state, which the pair names `left.<name>` / `right.<name>` beside each other.  Both must be able to store their output
as a branch; the sum is taken in float32.
"""
from __future__ import annotations

from types import SimpleNamespace

import torch

from ..registry import part_class, register_part
from .base import Mixer, StateNeed, fused_form


class MixerPair(Mixer):
    stores_branch = True

    @classmethod
    def tensor_shapes(cls, spec):
        shapes = {}
        for side in ("left", "right"):
            inner = spec[side]
            for name, shape in part_class("mixer", inner.kind).tensor_shapes(inner).items():
                shapes[f"{side}.{name}"] = shape
        return shapes

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.size = int(spec["size"])
        self.scales = (float(spec.get("left_scale", 1.0)), float(spec.get("right_scale", 1.0)))
        self.sides = []
        for side in ("left", "right"):
            inner = spec[side]
            own = {}
            for name, t in weights.items():
                if name.startswith(side + "."):
                    own[name[len(side) + 1:]] = t
            part = part_class("mixer", inner.kind)(inner, own, rt)
            if not getattr(part, "stores_branch", False):
                raise ValueError(f"the {side} mixer of a pair cannot hand its output over as a branch")
            self.sides.append((side, part))
        if sum(1 for _, p in self.sides if p.cache_need() is not None) > 1:
            raise ValueError("only one mixer of a pair can keep pages")
        self.graph_safe = all(getattr(p, "graph_safe", False) for _, p in self.sides)

    def cache_need(self):
        for _, part in self.sides:
            need = part.cache_need()
            if need is not None:
                return need
        return None

    def portion_multiple(self) -> int:
        a, b = (int(p.portion_multiple()) for _, p in self.sides)
        g = a
        while b:
            g, b = b, g % b
        return a * int(self.sides[1][1].portion_multiple()) // g

    def state_need(self):
        out = {}
        for side, part in self.sides:
            need = part.state_need()
            if need is None:
                continue
            for name, n in (need.items() if isinstance(need, dict) else [("", need)]):
                out[f"{side}.{name}"] = n
        return out or None

    def _binding(self, binding, side, part):
        need = part.state_need()
        if need is None:
            state = None
        elif isinstance(need, dict):
            state = {name: binding.state[f"{side}.{name}"] for name in need}
        else:
            state = binding.state[f"{side}."]
        keeps = part.cache_need() is not None
        return SimpleNamespace(group=binding.group if keeps else -1, k_pages=binding.k_pages if keeps else None,
                               v_pages=binding.v_pages if keeps else None, page_size=binding.page_size, writes=binding.writes,
                               state=state, pool_k=getattr(binding, "pool_k", None) if keeps else None,
                               pool_v=getattr(binding, "pool_v", None) if keeps else None)

    def forward(self, ctx, h, residual, binding, branch=None) -> None:
        rt = self.rt
        outs = []
        for side, part in self.sides:
            out = rt.empty((h.shape[0], self.size), torch.float32)
            part.forward(ctx, h, None, self._binding(binding, side, part), branch=out)
            outs.append(out)
        self._sum(outs, residual, branch)

    def forward_from_residual(self, ctx, residual, norm, binding, branch=None) -> bool:
        """Decode-sized steps: each side reads the residual stream through the norm in the kernel of its own first product,
        where both sides have such a form (the norm's few operations are done twice, its launch and its pass not at all).
        False: not taken."""
        joint = [getattr(part, "forward_from_residual", None) or getattr(part, "project_norm", None) for _, part in self.sides]
        if any(j is None for j in joint) or self.rt.dtype != torch.bfloat16:
            return False
        # both sides must take it: a side that declines after the other has stored its keys would run that side twice
        rows = residual.shape[0]
        if any(fused_form(self.rt.ops, rows, self.size, getattr(part, "w_qkv", getattr(part, "w_qkvg", None))) != "resident"
               for _, part in self.sides) or getattr(norm, "fused_prologue", lambda: None)() is None:
            return False
        outs = []
        for side, part in self.sides:
            out = self.rt.empty((rows, self.size), torch.float32)
            inner = self._binding(binding, side, part)
            if hasattr(part, "forward_from_residual"):
                if not part.forward_from_residual(ctx, residual, norm, inner, branch=out):
                    raise RuntimeError(f"the {side} mixer of a pair declined a step its sizes fit")
            else:
                part.forward_from_projection(ctx, part.project_norm(ctx, residual, norm), None, inner, branch=out)
            outs.append(out)
        self._sum(outs, residual, branch)
        return True

    def _sum(self, outs, residual, branch) -> None:
        ops = self.rt.ops
        if branch is not None:
            ops.weighted_sum(branch, outs[0], self.scales[0], outs[1], self.scales[1])
        else:
            ops.weighted_sum(residual, outs[0], self.scales[0], outs[1], self.scales[1], accumulate=True)


register_part("mixer", "mixer_pair", MixerPair)
