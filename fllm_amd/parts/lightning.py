"""Linear attention with a decay a head, carried from token to token as a matrix.

q = act(W_q h), k = act(W_k h) (heads x dim), v = act(W_v h) (heads x vdim), act = silu; per head
S_t = decay_h * S_(t-1) + k_t v_t^T and o_t = S_t^T q_t, with no other scale.  The heads side by side are RMS-normed together
(weight `norm`), multiplied lane by lane with sigmoid(W_g h), and projected by W_o into the residual stream.  S starts at zero,
is float32 [heads, dim, vdim] for every live request, and is all this mixer keeps: it has no pages, and a prompt may be cut
anywhere.  q, k, v and the gate are one product with the concatenated matrix.

What a design may choose otherwise: `position` (rotary on the first lanes of every head of q and of k, in float32 behind the
product, lane i with lane i + dims / 2), `key_scale` (a constant on k behind the rotation), `head_norm` (every head's output
is divided by its own root mean square, no weight, instead of the weighted norm over all heads) and `gate_activation`
"silu" (the gate is silu(W_g h) instead of a sigmoid).  With rotation or a key scale the operands of the recurrence are
float32 in both precisions: nothing that enters the recurrence is rounded behind the projection.
"""
from __future__ import annotations

import numpy as np
import torch

from ..config.spec import PartSpec
from ..registry import part_class, register_part
from .base import INIT_MATRIX, INIT_NORM, Mixer, StateNeed, add_and_prepare, fused_form, take_prepared


class LightningAttention(Mixer):
    graph_safe = True      # forward launches kernels only: no per-step decision on the host
    stores_branch = True

    @classmethod
    def tensor_shapes(cls, spec):
        h, nh, d, dv = spec["hidden_size"], spec["num_heads"], spec["head_dim"], spec["value_head_dim"]
        return {"q": ((nh * d, h), INIT_MATRIX), "k": ((nh * d, h), INIT_MATRIX), "v": ((nh * dv, h), INIT_MATRIX),
                "g": ((nh * dv, h), INIT_MATRIX), "o": ((h, nh * dv), INIT_MATRIX), "norm": ((nh * dv,), INIT_NORM)}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.dim = int(spec["head_dim"])
        self.v_dim = int(spec["value_head_dim"])
        self.eps = float(spec["eps"])
        self.activation = spec.get("activation", "silu")
        if self.activation not in ("silu", "none"):
            raise ValueError(f"activation {self.activation!r}: linear attention applies silu or nothing to q, k and v")
        decay = [float(d) for d in spec["decay"]]
        if len(decay) != self.heads:
            raise ValueError(f"{len(decay)} decays for {self.heads} heads")
        # a decay as a float32 pair: the sum of the two is the number itself to 48 bits, so its power over thousands of
        # tokens does not drift from that of the number the file gives
        hi = np.asarray(decay, dtype=np.float64).astype(np.float32)
        lo = (np.asarray(decay, dtype=np.float64) - hi.astype(np.float64)).astype(np.float32)
        self.decay_hi = torch.from_numpy(hi).to(rt.device)
        self.decay_lo = torch.from_numpy(lo).to(rt.device)
        self.w_qkvg = torch.cat([rt.matrix(weights[n]) for n in ("q", "k", "v", "g")], dim=0).contiguous()
        self.w_o = rt.matrix(weights["o"])
        self.head_norm = bool(spec.get("head_norm", False))
        self.norm_weight = None if self.head_norm else rt.vector(weights["norm"])
        self.gate_activation = spec.get("gate_activation", "sigmoid")
        if self.gate_activation not in ("sigmoid", "silu") or (self.gate_activation == "silu" and not self.head_norm):
            raise ValueError("the gate is a sigmoid, or with `head_norm` a silu")
        self.key_scale = float(spec.get("key_scale", 1.0))
        self.position = None
        position = spec.get("position")
        if position is not None:
            position = dict(position)
            kind = position.pop("kind")
            self.position = part_class("position", kind)(PartSpec(kind, position), {}, rt)
            if self.position.pairing != 0 or self.position.dims > self.dim:
                raise ValueError("linear attention turns lane i with lane i + dims / 2 inside a head")
        if (self.position is not None or self.key_scale != 1.0) and self.activation != "none":
            raise ValueError("rotated or scaled operands come without an activation")
        rt.tile_for_decode(self.w_o)
        rt.tile_for_decode(self.w_qkvg, priority=1)

    def state_need(self):
        return StateNeed((self.heads, self.dim, self.v_dim), torch.float32)

    def forward(self, ctx, h, residual, binding, branch=None) -> None:
        qkvg = self.rt.empty((h.shape[0], self.w_qkvg.shape[0]))
        self.rt.ops.linear(h, self.w_qkvg, qkvg)
        self.forward_from_projection(ctx, qkvg, residual, binding, branch)

    def project_norm(self, ctx, residual, norm):
        """Decode-sized steps in bfloat16: the joint product straight from the residual stream, the norm before the mixer
        folded in, for whoever arranges this mixer and goes on with `forward_from_projection`.  None: not taken."""
        rt, ops = self.rt, self.rt.ops
        prologue = getattr(norm, "fused_prologue", lambda: None)()
        if rt.dtype != torch.bfloat16 or prologue is None or not hasattr(ops, "norm_linear"):
            return None
        if fused_form(ops, residual.shape[0], self.hidden, self.w_qkvg) != "resident":
            return None
        qkvg = rt.empty((residual.shape[0], self.w_qkvg.shape[0]))
        ops.norm_linear(residual, prologue[0], prologue[1], self.w_qkvg, qkvg)
        return qkvg

    def forward_from_projection(self, ctx, qkvg, residual, binding, branch=None) -> None:
        """From the joint product [q | k | v | gate] of the step's rows to the output projection."""
        rt, ops = self.rt, self.rt.ops
        rows = qkvg.shape[0]
        nq, nv = self.heads * self.dim, self.heads * self.v_dim
        o = rt.empty((rows, nv), torch.float32)
        operands = qkvg
        if self.position is not None or self.key_scale != 1.0:
            operands = rt.empty((rows, 2 * nq + nv), torch.float32)
            if self.position is not None:
                cos, sin, dims = self.position.cos, self.position.sin, self.position.dims
            else:
                cos, sin, dims, _ = ctx.no_rotation(rt)
            ops.rotate_scale(qkvg, operands, ctx.row_pos, cos, sin, self.heads, self.dim, self.v_dim, dims, self.key_scale)
        ops.linear_attention(operands, self.decay_hi, self.decay_lo, binding.state, ctx.row_seg, ctx.seg_start, ctx.slots, o,
                             self.heads, self.dim, self.v_dim, activation=self.activation)
        gated = rt.empty((rows, nv))
        if self.head_norm:
            ops.group_norm_gate(o, self.eps, self.v_dim, qkvg[:, 2 * nq + nv:], gated, activation=self.gate_activation)
        else:
            ops.gated_norm(o, self.norm_weight, self.eps, qkvg[:, 2 * nq + nv:], gated)
        if branch is not None:
            ops.linear(gated, self.w_o, branch)
        elif not add_and_prepare(ctx, ops, gated, self.w_o, residual, None):
            ops.linear(gated, self.w_o, residual, accumulate=True)


register_part("mixer", "lightning_attention", LightningAttention)
