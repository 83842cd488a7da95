"""Attention without a softmax over the paged cache: every key up to the row weighs on its own.

q, k, v = one product with the concatenated matrix (biases allowed), no rotation.  For row i at position p and key j:
s = (q_i . k_j) * scale * temp(p), temp(p) = 1 + temp_coef * ln(floor((p + 1) / temp_every) + 1) (a query temperature that
grows with the position); s <- softcap * tanh(s / softcap); s <- s - r1_h * ln(1 + r2_h * (p - j)) (a bias by distance, two
learned numbers a head); the key's weight is sigmoid(s + pb_h) (one more learned number a head) and the output is the plain
sum of weight * value: weights are not normalized over the keys.  Output projection with an optional bias.
"""
from __future__ import annotations

import torch

from ..registry import register_part
from .base import INIT_BIAS, INIT_MATRIX, INIT_NORM, KVNeed, Mixer, add_and_prepare, fused_form, take_prepared


class SigmoidAttention(Mixer):
    graph_safe = True
    stores_branch = True
    KEY_CHUNK = 8

    @classmethod
    def tensor_shapes(cls, spec):
        h, nh, nkv, d = spec["hidden_size"], spec["num_heads"], spec["num_kv_heads"], spec["head_dim"]
        dv = spec.get("value_head_dim") or d
        return {
            "q": ((nh * d, h), INIT_MATRIX), "k": ((nkv * d, h), INIT_MATRIX), "v": ((nkv * dv, h), INIT_MATRIX),
            "o": ((h, nh * dv), INIT_MATRIX),
            "q_bias": ((nh * d,), INIT_BIAS), "k_bias": ((nkv * d,), INIT_BIAS), "v_bias": ((nkv * dv,), INIT_BIAS),
            "o_bias": ((h,), INIT_BIAS),
            "r1": ((nh,), INIT_NORM), "r2": ((nh,), INIT_NORM), "pb": ((nh,), INIT_BIAS),
        }

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.kv_heads = int(spec["num_kv_heads"])
        self.head_dim = int(spec["head_dim"])
        self.v_dim = int(spec.get("value_head_dim") or self.head_dim)
        self.scale = float(spec["scale"])
        self.softcap = float(spec["softcap"])
        self.temp_coef = float(spec.get("temp_coef", 0.0))
        self.temp_every = int(spec.get("temp_every", 1))
        if self.heads % self.kv_heads != 0:
            raise ValueError(f"head count {self.heads} is not a multiple of key/value head count {self.kv_heads}")
        if not self.softcap > 0.0 or self.temp_every <= 0:
            raise ValueError("softcap and temp_every must be positive")
        self.key_chunk = self.KEY_CHUNK if self.head_dim % self.KEY_CHUNK == 0 else 1
        self.w_qkv = torch.cat([rt.matrix(weights[n]) for n in ("q", "k", "v")], dim=0).contiguous()
        self.w_o = rt.matrix(weights["o"])
        rt.tile_for_decode(self.w_o)
        rt.tile_for_decode(self.w_qkv, priority=1)
        sizes = (self.heads * self.head_dim, self.kv_heads * self.head_dim, self.kv_heads * self.v_dim)
        biases = [weights.get(n) for n in ("q_bias", "k_bias", "v_bias")]
        self.b_qkv = None
        if any(b is not None for b in biases):
            self.b_qkv = torch.cat([rt.vector(b) if b is not None else torch.zeros(n, dtype=torch.float32, device=rt.device)
                                    for b, n in zip(biases, sizes)]).contiguous()
        self.b_o = rt.vector(weights["o_bias"]) if weights.get("o_bias") is not None else None
        self.r1, self.r2, self.pb = (rt.vector(weights[n]) for n in ("r1", "r2", "pb"))

    def cache_need(self):
        return KVNeed(self.kv_heads, self.head_dim, self.v_dim, None, key_chunk=self.key_chunk)

    def forward(self, ctx, h, residual, binding, branch=None):
        qkv = self.rt.empty((h.shape[0], self.w_qkv.shape[0]))
        self.rt.ops.linear(h, self.w_qkv, qkv, bias=self.b_qkv)
        self._attend(ctx, qkv, residual, binding, branch)

    def forward_from_residual(self, ctx, residual, norm, binding, branch=None) -> bool:
        """Decode-sized steps in bfloat16: the norm before the mixer and the joint product are one kernel that reads the
        residual stream.  False: not taken, the block runs the norm and `forward`."""
        rt, ops = self.rt, self.rt.ops
        prologue = getattr(norm, "fused_prologue", lambda: None)()
        if rt.dtype != torch.bfloat16 or prologue is None or not hasattr(ops, "norm_linear"):
            return False
        if fused_form(ops, residual.shape[0], self.hidden, self.w_qkv) != "resident":
            return False
        take_prepared(ctx, norm, residual)
        qkv = rt.empty((residual.shape[0], self.w_qkv.shape[0]))
        ops.norm_linear(residual, prologue[0], prologue[1], self.w_qkv, qkv, bias=self.b_qkv)
        self._attend(ctx, qkv, residual, binding, branch)
        return True

    def _attend(self, ctx, qkv, residual, binding, branch=None):
        rt, ops = self.rt, self.rt.ops
        rows = qkv.shape[0]
        nh, nkv, d, dv = self.heads, self.kv_heads, self.head_dim, self.v_dim
        tables = ctx.tables[binding.group]
        cos, sin, dims, pairing = ctx.no_rotation(rt)
        shape_args = {}
        if dv != d:
            shape_args["v_dim"] = dv
        if self.key_chunk != self.KEY_CHUNK:
            shape_args["key_chunk"] = self.key_chunk
        ops.rope_kv_store(qkv, ctx.row_pos, ctx.row_seg, tables, cos, sin, binding.k_pages if binding.writes else None,
                          binding.v_pages if binding.writes else None, nh, nkv, d, dims, pairing, binding.page_size, **shape_args)
        out = rt.empty((rows, nh * dv))
        ops.sigmoid_attention(qkv[:, : nh * d], binding.k_pages, binding.v_pages, tables, ctx.row_pos, ctx.row_seg, ctx.seg_start, out,
                              nh, nkv, d, dv, binding.page_size, self.scale, self.softcap, self.r1, self.r2, self.pb, self.temp_coef,
                              self.temp_every, self.key_chunk, max_context=ctx.max_context)
        if branch is not None:
            ops.linear(out, self.w_o, branch, bias=self.b_o)
        elif not add_and_prepare(ctx, ops, out, self.w_o, residual, self.b_o):
            ops.linear(out, self.w_o, residual, bias=self.b_o, accumulate=True)


register_part("mixer", "sigmoid_attention", SigmoidAttention)
