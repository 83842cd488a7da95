"""Linear attention with a decay a head, carried from token to token as a matrix.

q = act(W_q h), k = act(W_k h) (heads x dim), v = act(W_v h) (heads x vdim), act = silu; per head
S_t = decay_h * S_(t-1) + k_t v_t^T and o_t = S_t^T q_t, with no other scale.  The heads side by side are RMS-normed together
(weight `norm`), multiplied lane by lane with sigmoid(W_g h), and projected by W_o into the residual stream.  S starts at zero,
is float32 [heads, dim, vdim] for every live request, and is all this mixer keeps: it has no pages, and a prompt may be cut
anywhere.  q, k, v and the gate are one product with the concatenated matrix.
"""
from __future__ import annotations

import numpy as np
import torch

from ..registry import register_part
from .base import INIT_MATRIX, INIT_NORM, Mixer, StateNeed, add_and_prepare


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
        self.norm_weight = rt.vector(weights["norm"])
        rt.tile_for_decode(self.w_o)
        rt.tile_for_decode(self.w_qkvg, priority=1)

    def state_need(self):
        return StateNeed((self.heads, self.dim, self.v_dim), torch.float32)

    def forward(self, ctx, h, residual, binding, branch=None) -> None:
        rt, ops = self.rt, self.rt.ops
        rows = h.shape[0]
        nq, nv = self.heads * self.dim, self.heads * self.v_dim
        qkvg = rt.empty((rows, 2 * nq + 2 * nv))
        ops.linear(h, self.w_qkvg, qkvg)
        o = rt.empty((rows, nv), torch.float32)
        ops.linear_attention(qkvg, self.decay_hi, self.decay_lo, binding.state, ctx.row_seg, ctx.seg_start, ctx.slots, o,
                             self.heads, self.dim, self.v_dim, activation=self.activation)
        gated = rt.empty((rows, nv))
        ops.gated_norm(o, self.norm_weight, self.eps, qkvg[:, 2 * nq + nv:], gated)
        if branch is not None:
            ops.linear(gated, self.w_o, branch)
        elif not add_and_prepare(ctx, ops, gated, self.w_o, residual, None):
            ops.linear(gated, self.w_o, residual, accumulate=True)


register_part("mixer", "lightning_attention", LightningAttention)
