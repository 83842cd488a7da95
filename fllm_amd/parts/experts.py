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
`correction` (a tensor, one number an expert): the picks are made by score + correction, the weights stay the scores
themselves; `groups` and `groups_kept`: the experts form that many equal groups of neighbours, a group counts the sum of its
two largest corrected scores, and only experts of the best `groups_kept` groups can be picked (such a router scores with a
sigmoid and renormalizes).  `gated` False: an expert is W_down a(W_up n) with a(z) = relu(z)^2 and has no gate matrix
(stacked [experts, inter, width]); its weight lies on its output.  `shared`: lanes of one more expert of the same form that
every token uses with weight 1 (`shared_up`, `shared_down`); its output joins the sum.
"""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import INIT_BIAS, INIT_MATRIX, FeedForward


class RoutedExperts(FeedForward):
    graph_safe = True      # the picks stay on the device: no per-step decision on the host

    @classmethod
    def tensor_shapes(cls, spec):
        h, i, n = spec["hidden_size"], spec["intermediate_size"], spec["experts"]
        shapes = {"router": ((n, h), INIT_MATRIX), "correction": ((n,), INIT_BIAS)}
        for e in range(n):
            shapes[f"gate_{e}"] = ((i, h), INIT_MATRIX)
            shapes[f"up_{e}"] = ((i, h), INIT_MATRIX)
            shapes[f"down_{e}"] = ((h, i), INIT_MATRIX)
        if spec.get("shared"):
            shapes["shared_up"] = ((spec["shared"], h), INIT_MATRIX)
            shapes["shared_down"] = ((h, spec["shared"]), INIT_MATRIX)
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
        self.gated = bool(spec.get("gated", True))
        self.groups = int(spec.get("groups", 1))
        self.groups_kept = int(spec.get("groups_kept", self.groups))
        self.correction = rt.vector(weights["correction"]) if weights.get("correction") is not None else None
        if self.groups <= 0 or n % self.groups != 0 or not 1 <= self.groups_kept <= self.groups:
            raise ValueError(f"{n} experts in {self.groups} groups of which {self.groups_kept} are kept")
        self.grouped_router = self.correction is not None or self.groups > 1
        if self.grouped_router:
            if self.score != "sigmoid" or not self.renormalize:
                raise ValueError("a router with corrections or groups scores with a sigmoid and renormalizes the picks' scores")
            if self.top > self.groups_kept * (n // self.groups):
                raise ValueError(f"{self.top} picks do not fit into {self.groups_kept} groups of {n // self.groups} experts")
            if self.correction is None:
                self.correction = torch.zeros(n, dtype=torch.float32, device=rt.device)
        if self.gated:
            self.w_gate_up = torch.stack([torch.cat([rt.matrix(weights[f"gate_{e}"]), rt.matrix(weights[f"up_{e}"])], dim=0)
                                          for e in range(n)]).contiguous()
        else:
            if self.weight_on != "output" or self.limit or self.up_offset:
                raise ValueError("experts without a gate carry their weight on the output and clamp nothing")
            self.w_up = torch.stack([rt.matrix(weights[f"up_{e}"]) for e in range(n)]).contiguous()
        self.w_down = torch.stack([rt.matrix(weights[f"down_{e}"]) for e in range(n)]).contiguous()
        self.shared = int(spec.get("shared") or 0)
        if self.shared:
            if self.gated:
                raise ValueError("a shared expert comes with experts without a gate")
            self.w_shared_up = rt.matrix(weights["shared_up"])
            self.w_shared_down = rt.matrix(weights["shared_down"])
            rt.tile_for_decode(self.w_shared_down)

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
        if self.grouped_router:
            ops.route_grouped(h, self.w_router, self.correction, self.top, self.groups, self.groups_kept, ids, weights,
                              route_scale=self.route_scale)
        elif self.score == "sigmoid" and not self.renormalize and self.route_scale == 1.0:
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
        if not self.gated:
            ungrouped = getattr(ops, "experts_grouped_ungated", None)
            if ungrouped is None or not ungrouped(h, ids, self.w_up, self.w_down, parts):
                act = rt.empty((rows * self.top, self.inter))
                ops.experts_up(h, ids, self.w_up, act, activation="relu2")
                ops.experts_down(act, ids, self.w_down, parts)
        elif grouped is None or not grouped(h, ids, weights, self.w_gate_up, self.w_down, parts, self.limit, self.alpha, self.up_offset):
            act = rt.empty((rows * self.top, self.inter))
            ops.experts_gate_up(h, ids, weights, self.w_gate_up, act, self.limit, self.alpha, self.up_offset)
            ops.experts_down(act, ids, self.w_down, parts)
        if branch is None:
            ones = self._ones(("ones", self.hidden), (self.hidden,))
            if on_output is not None:
                ops.postnorm_add(residual, parts, ones, None, parts=self.top, part_weights=on_output)
            else:
                ops.postnorm_add(residual, parts, ones, None, parts=self.top)
        if self.shared:          # one more expert that every row uses, its weight 1: its sum joins the picks' in the stream
            wide = rt.empty((rows, self.shared))
            ops.linear(h, self.w_shared_up, wide)
            ops.activation(wide, wide, "relu2")
            ops.linear(wide, self.w_shared_down, residual, accumulate=True)

    def _ones(self, key, shape):
        ones = self.rt.shared.get(key)
        if ones is None:
            ones = self.rt.shared[key] = torch.ones(shape, dtype=torch.float32, device=self.rt.device)
        return ones


register_part("feed_forward", "routed_experts", RoutedExperts)
