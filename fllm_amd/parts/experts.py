"""A feed-forward of many small gated layers of which every token uses a few.

Router: z = W_router n in float32, score = sigmoid(z); the `top` experts with the largest scores are a token's picks (the
lower index among equal scores) and the scores themselves are their weights, not renormalized.  A pick's weight multiplies
the expert's INPUT: y = sum over the picks of W_down_e (a(W_gate_e (s_e n)) * (W_up_e (s_e n) + up_offset)) with
a(g) = g * sigmoid(alpha g), operands clamped to `limit` where there is one (the constants of `ClampedGLU`; the defaults
are SwiGLU).  The experts' matrices are stacked at load: [experts, 2 * inter, width] (gate rows, then up rows) and
[experts, width, inter], so that a kernel finds an expert by its index.

What a design may choose otherwise: `score` "softmax" (the scores are the softmax of the router's logits over ALL experts),
`renormalize` (the picks' scores are divided by their sum + 1e-20), `route_scale` (a constant on the weights), and
`weight_on` "output": y = sum over the picks of weight_e * expert_e(n), the weight on what the expert gives, not on what it reads.
"""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import INIT_MATRIX, FeedForward


class RoutedExperts(FeedForward):
    graph_safe = True      # the picks stay on the device: no per-step decision on the host

    @classmethod
    def tensor_shapes(cls, spec):
        h, i, n = spec["hidden_size"], spec["intermediate_size"], spec["experts"]
        shapes = {"router": ((n, h), INIT_MATRIX)}
        for e in range(n):
            shapes[f"gate_{e}"] = ((i, h), INIT_MATRIX)
            shapes[f"up_{e}"] = ((i, h), INIT_MATRIX)
            shapes[f"down_{e}"] = ((h, i), INIT_MATRIX)
        return shapes

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.experts = int(spec["experts"])
        self.top = int(spec["top"])
        if not 1 <= self.top <= self.experts:
            raise ValueError(f"{self.top} picks among {self.experts} experts")
        self.score = spec.get("score", "sigmoid")
        if self.score not in ("sigmoid", "softmax"):
            raise ValueError(f"router score {self.score!r}: the router's kernel scores with a sigmoid or a softmax over all experts")
        self.renormalize = bool(spec.get("renormalize", False))
        self.route_scale = float(spec.get("route_scale", 1.0))
        self.weight_on = spec.get("weight_on", "input")
        if self.weight_on not in ("input", "output"):
            raise ValueError(f"a pick's weight goes on the expert's input or output, not on {self.weight_on!r}")
        # forward(..., branch=t) stores the picks' outputs in t; with the weights on the outputs the sum needs the weights,
        # so this part then adds to the stream itself (an arrangement hands it a stand-in)
        self.stores_branch = self.weight_on == "input"
        self.limit = float(spec.get("limit") or 0.0)          # 0: nothing is clamped
        self.alpha = float(spec.get("alpha", 1.0))
        self.up_offset = float(spec.get("up_offset", 0.0))
        self.w_router = rt.matrix(weights["router"])
        n = self.experts
        self.w_gate_up = torch.stack([torch.cat([rt.matrix(weights[f"gate_{e}"]), rt.matrix(weights[f"up_{e}"])], dim=0)
                                      for e in range(n)]).contiguous()
        self.w_down = torch.stack([rt.matrix(weights[f"down_{e}"]) for e in range(n)]).contiguous()

    @property
    def branch_parts(self) -> int:
        """Rows of a stored branch that make up one token's output: a token's picks leave their outputs one after the
        other, and whoever adds the branch to the stream sums them in pick order."""
        return self.top

    def forward(self, ctx, h, residual, branch=None):
        """`branch`: float32 [rows * top, width], row r's picks at r * top ..; None: the sum goes into `residual`."""
        rt, ops = self.rt, self.rt.ops
        rows = h.shape[0]
        ids = rt.empty((rows, self.top), torch.int32)
        weights = rt.empty((rows, self.top), torch.float32)
        if self.score == "sigmoid" and not self.renormalize and self.route_scale == 1.0:
            ops.route_topk(h, self.w_router, self.top, ids, weights)
        else:
            ops.route_topk(h, self.w_router, self.top, ids, weights, score=self.score, renormalize=self.renormalize,
                           route_scale=self.route_scale)
        on_output = None
        if self.weight_on == "output" and branch is not None:
            raise ValueError("experts whose weights lie on their outputs add to the stream themselves: no stored branch")
        if self.weight_on == "output":          # the experts read the rows as they are; the weights wait for the sum
            on_output, weights = weights, self._ones(("ones", rows, self.top), (rows, self.top))
        parts = branch if branch is not None else rt.empty((rows * self.top, self.hidden), torch.float32)
        grouped = getattr(ops, "experts_grouped", None)
        if grouped is None or not grouped(h, ids, weights, self.w_gate_up, self.w_down, parts, self.limit, self.alpha, self.up_offset):
            act = rt.empty((rows * self.top, self.inter))
            ops.experts_gate_up(h, ids, weights, self.w_gate_up, act, self.limit, self.alpha, self.up_offset)
            ops.experts_down(act, ids, self.w_down, parts)
        if branch is None:
            ones = self._ones(("ones", self.hidden), (self.hidden,))
            if on_output is not None:
                ops.postnorm_add(residual, parts, ones, None, parts=self.top, part_weights=on_output)
            else:
                ops.postnorm_add(residual, parts, ones, None, parts=self.top)

    def _ones(self, key, shape):
        ones = self.rt.shared.get(key)
        if ones is None:
            ones = self.rt.shared[key] = torch.ones(shape, dtype=torch.float32, device=self.rt.device)
        return ones


register_part("feed_forward", "routed_experts", RoutedExperts)
