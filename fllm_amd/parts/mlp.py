"""Gated feed-forward: x += W_down (silu(W_gate n) * W_up n), silu(g) = g / (1 + exp(-g))
(rust/engine/src/rust_decoder.rs:8328-8352, :1645; rust/engine/src/cpu_elementwise.rs:3-43).
Gate and up are one product with the concatenated matrix."""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import INIT_BIAS, INIT_MATRIX, INIT_NORM, FeedForward, add_and_prepare, fused_form, take_prepared


class GatedMLP(FeedForward):
    graph_safe = True      # forward launches kernels only: no per-step decision on the host

    @classmethod
    def tensor_shapes(cls, spec):
        h, i = spec["hidden_size"], spec["intermediate_size"]
        return {"gate": ((i, h), INIT_MATRIX), "up": ((i, h), INIT_MATRIX), "down": ((h, i), INIT_MATRIX),
                "gate_bias": ((i,), INIT_BIAS), "up_bias": ((i,), INIT_BIAS), "down_bias": ((h,), INIT_BIAS)}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        if spec.get("activation", "silu") not in ("silu", "swish"):
            raise ValueError(f"unsupported activation {spec.get('activation')!r}; the gated feed-forward uses silu")
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.w_gate_up = torch.cat([rt.matrix(weights["gate"]), rt.matrix(weights["up"])], dim=0).contiguous()
        self.w_down = rt.matrix(weights["down"])
        rt.tile_for_decode(self.w_down)
        rt.tile_for_decode(self.w_gate_up, gate_up=True, priority=1)
        gb, ub = weights.get("gate_bias"), weights.get("up_bias")
        self.b_gate_up = None
        if gb is not None or ub is not None:
            zeros = lambda: torch.zeros(self.inter, dtype=torch.float32, device=rt.device)
            self.b_gate_up = torch.cat([rt.vector(gb) if gb is not None else zeros(),
                                        rt.vector(ub) if ub is not None else zeros()]).contiguous()
        self.b_down = rt.vector(weights["down_bias"]) if weights.get("down_bias") is not None else None

    def forward_from_residual(self, ctx, residual, norm) -> bool:
        """Decode-sized steps in bfloat16: norm, gate/up product and activation are one kernel.
        False: not taken, the block runs norm and `forward`."""
        rt, ops = self.rt, self.rt.ops
        rows = residual.shape[0]
        prologue = getattr(norm, "fused_prologue", lambda: None)()
        form = fused_form(ops, rows, self.hidden, self.w_gate_up, gate_up=True) if hasattr(ops, "norm_gate_up_swiglu") else None
        if rt.dtype != torch.bfloat16 or prologue is None or form is None:
            return False
        norm_scale, norm_eps = prologue
        act = rt.empty((rows, self.inter))
        prepared = take_prepared(ctx, norm, residual)      # the sum before this norm may have computed its first steps
        if prepared is None and form == "chunks":
            prepared = ops.prepare_norm(residual, norm_scale)
        ops.norm_gate_up_swiglu(residual, norm_scale, norm_eps, self.w_gate_up, act, bias=self.b_gate_up,
                                **({"prepared": prepared} if prepared is not None else {}))
        if not add_and_prepare(ctx, ops, act, self.w_down, residual, self.b_down):
            ops.linear(act, self.w_down, residual, bias=self.b_down, accumulate=True)
        return True

    def _own_products(self, rows: int) -> bool:
        """17 to 128 rows: the kernel library may prefer its own products to the GEMM library's (it does when both matrices
        have their tile-major copies)."""
        own = getattr(self.rt.ops, "own_feed_forward", None)
        return own is not None and self.rt.dtype == torch.bfloat16 and own(rows, self.w_gate_up, self.w_down)

    def forward_branch(self, ctx, h):
        """The output as a tensor of its own instead of a sum into the residual stream (large bfloat16
        steps whose products go to the GEMM library, which has no residual epilogue): the block lets
        the sum ride on the next norm.  None: not taken."""
        rt, ops = self.rt, self.rt.ops
        rows = h.shape[0]
        start = getattr(ops, "library_gemm_from", None)
        if rt.dtype != torch.bfloat16 or start is None or rows < start or self.b_down is not None:
            return None
        if self._own_products(rows):
            return None          # `forward` runs the own products, which add into the residual stream themselves
        act = rt.empty((rows, self.inter))
        if (getattr(ops, "prefers_own_gate_up", None) is not None and ops.prefers_own_gate_up(rows, self.w_gate_up)
                and self.hidden % 8 == 0 and h.stride(0) % 8 == 0):
            ops.gate_up_swiglu(h, self.w_gate_up, act, bias=self.b_gate_up)     # the activation as the product's epilogue
        else:
            gate_up = rt.empty((rows, 2 * self.inter))
            ops.linear(h, self.w_gate_up, gate_up, bias=self.b_gate_up)
            ops.swiglu(gate_up, act)
        out = rt.empty((rows, self.hidden))
        ops.linear(act, self.w_down, out)
        return out

    def forward(self, ctx, h, residual):
        rt, ops = self.rt, self.rt.ops
        rows = h.shape[0]
        start = getattr(ops, "library_gemm_from", None)
        if (rt.dtype == torch.bfloat16 and self.hidden % 8 == 0 and h.stride(0) % 8 == 0
                and (self._own_products(rows) or (rows <= getattr(ops, "GATE_UP_SWIGLU_ROWS", 0) and (start is None or rows < start)))):
            # decode batches that the hand-written products serve: the activation is the epilogue of the gate/up product
            act = rt.empty((rows, self.inter))
            ops.gate_up_swiglu(h, self.w_gate_up, act, bias=self.b_gate_up)
            ops.linear(act, self.w_down, residual, bias=self.b_down, accumulate=True)
            return
        gate_up = rt.empty((rows, 2 * self.inter))
        ops.linear(h, self.w_gate_up, gate_up, bias=self.b_gate_up)
        act = rt.empty((rows, self.inter))
        ops.swiglu(gate_up, act)
        ops.linear(act, self.w_down, residual, bias=self.b_down, accumulate=True)


class ClampedGLU(FeedForward):
    """x += W_down (a(g) * (u + up_offset)) with g = min(W_gate n, limit), u = clamp(W_up n, -limit, limit) and
    a(g) = g * sigmoid(alpha * g).  Gate and up are one product with the concatenated matrix."""
    graph_safe = True
    stores_branch = True   # forward(..., branch=t) stores the down projection in t instead of adding it to the stream

    @classmethod
    def tensor_shapes(cls, spec):
        h, i = spec["hidden_size"], spec["intermediate_size"]
        return {"gate": ((i, h), INIT_MATRIX), "up": ((i, h), INIT_MATRIX), "down": ((h, i), INIT_MATRIX)}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.limit = float(spec.get("limit") or 0.0)          # 0: nothing is clamped
        self.alpha = float(spec.get("alpha", 1.0))
        self.up_offset = float(spec.get("up_offset", 0.0))
        self.w_gate_up = torch.cat([rt.matrix(weights["gate"]), rt.matrix(weights["up"])], dim=0).contiguous()
        self.w_down = rt.matrix(weights["down"])
        rt.tile_for_decode(self.w_down)
        rt.tile_for_decode(self.w_gate_up, gate_up=True, priority=1)

    def begins_from_residual(self, rows: int) -> bool:
        """Whether `begin_from_residual` would take a step of `rows` rows (an arrangement that can fold this part's
        norm into another kernel asks first)."""
        ops = self.rt.ops
        return (self.rt.dtype == torch.bfloat16 and hasattr(ops, "norm_gate_up_glu")
                and fused_form(ops, rows, self.hidden, self.w_gate_up, gate_up=True) == "resident")

    def begin_from_residual(self, ctx, residual, norm):
        """Decode-sized steps in bfloat16: the norm before this part, the gate/up product and the activation are one
        kernel that reads the residual stream; the activations come back and `finish` adds the down projection, which
        lets an arrangement run other readers of the same stream in between.  None: not taken."""
        rt, ops = self.rt, self.rt.ops
        rows = residual.shape[0]
        prologue = getattr(norm, "fused_prologue", lambda: None)()
        if rt.dtype != torch.bfloat16 or prologue is None or not hasattr(ops, "norm_gate_up_glu"):
            return None
        if fused_form(ops, rows, self.hidden, self.w_gate_up, gate_up=True) != "resident":
            return None
        act = rt.empty((rows, self.inter))
        ops.norm_gate_up_glu(residual, prologue[0], prologue[1], self.w_gate_up, act, self.limit, self.alpha, self.up_offset)
        return act

    def finish(self, ctx, act, residual, branch=None):
        if branch is not None:
            self.rt.ops.linear(act, self.w_down, branch)
        else:
            self.rt.ops.linear(act, self.w_down, residual, accumulate=True)

    def forward(self, ctx, h, residual, branch=None):
        rt, ops = self.rt, self.rt.ops
        rows = h.shape[0]
        act = rt.empty((rows, self.inter))
        start = getattr(ops, "library_gemm_from", None)
        own = getattr(ops, "own_feed_forward", None)
        if (rt.dtype == torch.bfloat16 and hasattr(ops, "gate_up_glu") and self.hidden % 8 == 0 and h.stride(0) % 8 == 0
                and ((own is not None and own(rows, self.w_gate_up, self.w_down))
                     or (rows <= getattr(ops, "GATE_UP_SWIGLU_ROWS", 0) and (start is None or rows < start)))):
            # steps that the hand-written products serve: the activation is the epilogue of the gate/up product
            ops.gate_up_glu(h, self.w_gate_up, act, self.limit, self.alpha, self.up_offset)
        else:
            gate_up = rt.empty((rows, 2 * self.inter))
            ops.linear(h, self.w_gate_up, gate_up)
            ops.glu_clamped(gate_up, act, self.limit, self.alpha, self.up_offset)
        self.finish(ctx, act, residual, branch)


class PolyNormMLP(FeedForward):
    """x += W_down act(W_up n) with act(z) = a N(z) + b N(z^2) + c N(z^3) + e: powers lane by lane, N the division of a token's
    vector of intermediate values by its root mean square (eps inside the root), and (a, b, c, e) the four learned numbers of
    the tensor `act`.  The sums of squares and the division are float32."""
    graph_safe = True
    stores_branch = True

    @classmethod
    def tensor_shapes(cls, spec):
        h, i = spec["hidden_size"], spec["intermediate_size"]
        return {"up": ((i, h), INIT_MATRIX), "down": ((h, i), INIT_MATRIX), "act": ((4,), INIT_NORM)}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.eps = float(spec["eps"])
        self.w_up = rt.matrix(weights["up"])
        self.w_down = rt.matrix(weights["down"])
        self.coeffs = rt.vector(weights["act"])
        rt.tile_for_decode(self.w_down)
        rt.tile_for_decode(self.w_up, priority=1)

    def forward(self, ctx, h, residual, branch=None):
        rt, ops = self.rt, self.rt.ops
        rows = h.shape[0]
        z = rt.empty((rows, self.inter))
        ops.linear(h, self.w_up, z)
        act = rt.empty((rows, self.inter))
        ops.polynorm(z, self.coeffs, self.eps, act)
        if branch is not None:
            ops.linear(act, self.w_down, branch)
        elif not add_and_prepare(ctx, ops, act, self.w_down, residual, None):
            ops.linear(act, self.w_down, residual, accumulate=True)

    def forward_from_residual(self, ctx, residual, norm) -> bool:
        """Decode-sized steps in bfloat16: the norm before this part rides in the up product.  False: not taken."""
        rt, ops = self.rt, self.rt.ops
        rows = residual.shape[0]
        prologue = getattr(norm, "fused_prologue", lambda: None)()
        if rt.dtype != torch.bfloat16 or prologue is None or not hasattr(ops, "norm_linear"):
            return False
        if fused_form(ops, rows, self.hidden, self.w_up) != "resident":
            return False
        take_prepared(ctx, norm, residual)
        z = rt.empty((rows, self.inter))
        ops.norm_linear(residual, prologue[0], prologue[1], self.w_up, z)
        act = rt.empty((rows, self.inter))
        ops.polynorm(z, self.coeffs, self.eps, act)
        if not add_and_prepare(ctx, ops, act, self.w_down, residual, None):
            ops.linear(act, self.w_down, residual, accumulate=True)
        return True


register_part("feed_forward", "gated_mlp", GatedMLP)
register_part("feed_forward", "polynorm_mlp", PolyNormMLP)
register_part("feed_forward", "clamped_glu", ClampedGLU)
