"""Parts of role `stream`: what a run entry does to the residual stream before its layer runs.

`pass_input`: the input of a pass of looped layers.  x += E[token] * scale for every pass but the first (the output of
the embedding as the model began with, which the embedding part recomputes from the step's token ids: no copy of it
is kept), then x += steps[row], one learned vector a pass, where the design has such vectors (`rows` in the spec).

`pass_mix`: x <- W [x; x0] + steps[row] before every pass (the first too): the stream and the embedding's output x0 side by
side through one matrix [size, 2 * size] (x first), then the pass's vector, which rides as the product's bias."""
from __future__ import annotations

from ..registry import register_part
import torch

from .base import INIT_BIAS, INIT_MATRIX, Part


class PassInput(Part):
    role = "stream"
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, spec):
        return {"steps": ((spec["rows"], spec["size"]), INIT_BIAS)} if spec.get("rows") else {}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.vector = None
        if spec.get("rows"):
            row, rows = int(spec["row"]), int(spec["rows"])
            if not 0 <= row < rows:
                raise ValueError(f"pass {row} of {rows}")
            self.vector = rt.vector(weights["steps"])[row]    # a view of the shared table: one row, contiguous
        self.add_embedding = bool(spec.get("add_embedding", False))
        if self.vector is None and not self.add_embedding:
            raise ValueError("a pass input that adds nothing")

    def forward(self, ctx, x, embedding) -> None:
        """`embedding`: the model's embedding part (its table and scale are what the stream began with)."""
        if self.add_embedding:
            self.rt.ops.stream_add(x, ids=ctx.ids, table=embedding.table, scale=embedding.scale, vec=self.vector)
        elif self.vector is not None:
            self.rt.ops.stream_add(x, vec=self.vector)


class PassMix(Part):
    role = "stream"
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, spec):
        shapes = {"mix": ((spec["size"], 2 * spec["size"]), INIT_MATRIX)}
        if spec.get("rows"):
            shapes["steps"] = ((spec["rows"], spec["size"]), INIT_BIAS)
        return shapes

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.size = int(spec["size"])
        self.w = rt.matrix(weights["mix"])
        self.vector = None
        if spec.get("rows"):
            row, rows = int(spec["row"]), int(spec["rows"])
            if not 0 <= row < rows:
                raise ValueError(f"pass {row} of {rows}")
            self.vector = rt.vector(weights["steps"])[row]

    def forward(self, ctx, x, embedding) -> None:
        rt, ops = self.rt, self.rt.ops
        both = rt.empty((x.shape[0], 2 * self.size))
        ops.stream_concat(x, ctx.ids, embedding.table, embedding.scale, both)
        mixed = rt.empty(tuple(x.shape), torch.float32)
        ops.linear(both, self.w, mixed, bias=self.vector)
        x.copy_(mixed)


register_part("stream", "pass_input", PassInput)
register_part("stream", "pass_mix", PassMix)
