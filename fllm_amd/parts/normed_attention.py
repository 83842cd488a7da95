"""Attention whose queries and keys pass a weighted RMS norm before they are rotated, over the paged cache.

q, k, v (and the gate) are one product with the concatenated matrix.  `qk_norm`: "head" norms every head of q and of k over
its own lanes with ONE weight vector of a head's size for all heads (`q_norm`, `k_norm`), "projection" norms the whole
query projection and the whole key projection at once with weights of those sizes, None norms nothing.  Rotary then turns
the first lanes of every head (lane i with lane i + dims / 2; any table the position part builds).  `values`: "projected"
(W_v h) or "keys": the values are the keys as projected, before norm and rotation, and there is no W_v.

What a row sees: with `window` and `pool`, the last `window` tokens and, for every block of `pool` positions that lies
wholly before them, one key and one value, the means of the block's keys and values as the pages hold them; tokens and
blocks share one softmax.  The means are kept beside the pages (float32, `KVNeed.pooled`), made once when a block's last
token is stored.  Without: every token up to the row.  `sink` "zero": the softmax's denominator holds one more term
exp(0), which has no value.  `output_gate`: the heads' outputs times sigmoid(W_g h) before the output projection.
"""
from __future__ import annotations

import torch

from ..config.spec import PartSpec
from ..registry import part_class, register_part
from .base import INIT_BIAS, INIT_MATRIX, INIT_NORM, KVNeed, Mixer, add_and_prepare, fused_form, take_prepared

NORM_MODES = {None: 0, "head": 1, "projection": 2}


class NormedAttention(Mixer):
    graph_safe = True
    stores_branch = True
    KEY_CHUNK = 8

    @classmethod
    def tensor_shapes(cls, spec):
        h, nh, nkv, d = spec["hidden_size"], spec["num_heads"], spec["num_kv_heads"], spec["head_dim"]
        dv = spec.get("value_head_dim") or d
        whole = spec.get("qk_norm") == "projection"
        return {
            "q": ((nh * d, h), INIT_MATRIX), "k": ((nkv * d, h), INIT_MATRIX), "v": ((nkv * dv, h), INIT_MATRIX),
            "o": ((h, nh * dv), INIT_MATRIX), "g": ((nh * dv, h), INIT_MATRIX),
            "q_bias": ((nh * d,), INIT_BIAS), "k_bias": ((nkv * d,), INIT_BIAS), "v_bias": ((nkv * dv,), INIT_BIAS),
            "o_bias": ((h,), INIT_BIAS),
            "q_norm": ((nh * d if whole else d,), INIT_NORM), "k_norm": ((nkv * d if whole else d,), INIT_NORM),
        }

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.kv_heads = int(spec["num_kv_heads"])
        self.head_dim = int(spec["head_dim"])
        self.v_dim = int(spec.get("value_head_dim") or self.head_dim)
        self.scale = float(spec["scale"])
        if self.heads % self.kv_heads != 0:
            raise ValueError(f"head count {self.heads} is not a multiple of key/value head count {self.kv_heads}")
        self.norm_mode = spec.get("qk_norm")
        if self.norm_mode not in NORM_MODES:
            raise ValueError(f"qk_norm {self.norm_mode!r}: 'head', 'projection' or None")
        self.eps = float(spec.get("qk_norm_eps") or 0.0)
        if self.norm_mode is not None and not self.eps > 0.0:
            raise ValueError("a norm of queries and keys needs a positive qk_norm_eps")
        self.values_from_keys = spec.get("values", "projected") == "keys"
        if spec.get("values", "projected") not in ("projected", "keys"):
            raise ValueError(f"values {spec.get('values')!r}: 'projected' or 'keys'")
        if self.values_from_keys and self.v_dim != self.head_dim:
            raise ValueError("keys that double as values have the keys' width")
        self.window, self.pool = spec.get("window"), spec.get("pool")
        if (self.window is None) != (self.pool is None):
            raise ValueError("a window with pooled blocks behind it names both `window` and `pool`")
        if self.window is not None and (int(self.window) <= 0 or int(self.pool) <= 0):
            raise ValueError("window and pool must be positive")
        sink = spec.get("sink")
        if sink not in (None, "zero"):
            raise ValueError(f"sink {sink!r}: 'zero' or None")
        if sink is not None and self.window is not None:
            raise ValueError("the kernel of windows with pooled blocks knows no sink")
        self.sinks = torch.zeros(self.heads, dtype=torch.float32, device=rt.device) if sink == "zero" else None
        self.gated = bool(spec.get("output_gate", False))
        self.key_chunk = self.KEY_CHUNK if self.head_dim % self.KEY_CHUNK == 0 else 1
        position = spec.get("position")
        self.position = None
        if position is not None:
            position = dict(position)
            kind = position.pop("kind")
            self.position = part_class("position", kind)(PartSpec(kind, position), {}, rt)
            if self.position.pairing != 0:
                raise ValueError("this mixer's kernel turns lane i with lane i + dims / 2")
        pieces = [rt.matrix(weights["q"]), rt.matrix(weights["k"])]
        if not self.values_from_keys:
            pieces.append(rt.matrix(weights["v"]))
        if self.gated:
            pieces.append(rt.matrix(weights["g"]))
        self.w_qkv = torch.cat(pieces, dim=0).contiguous()
        self.w_o = rt.matrix(weights["o"])
        rt.tile_for_decode(self.w_o)
        rt.tile_for_decode(self.w_qkv, priority=1)
        nq, nk, nv = self.heads * self.head_dim, self.kv_heads * self.head_dim, self.kv_heads * self.v_dim
        self.gate_at = nq + nk + (0 if self.values_from_keys else nv)
        biases = [weights.get("q_bias"), weights.get("k_bias"), None if self.values_from_keys else weights.get("v_bias")]
        self.b_qkv = None
        if any(b is not None for b in biases):
            sizes = [nq, nk] + ([] if self.values_from_keys else [nv]) + ([self.heads * self.v_dim] if self.gated else [])
            given = biases[:2] + ([] if self.values_from_keys else [biases[2]]) + ([None] if self.gated else [])
            self.b_qkv = torch.cat([rt.vector(b) if b is not None else torch.zeros(n, dtype=torch.float32, device=rt.device)
                                    for b, n in zip(given, sizes)]).contiguous()
        self.b_o = rt.vector(weights["o_bias"]) if weights.get("o_bias") is not None else None
        self.q_weight = rt.vector(weights["q_norm"]) if self.norm_mode is not None else None
        self.k_weight = rt.vector(weights["k_norm"]) if self.norm_mode is not None else None

    def cache_need(self):
        return KVNeed(self.kv_heads, self.head_dim, self.v_dim, None, key_chunk=self.key_chunk, pooled=int(self.pool or 0))

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
        take_prepared(ctx, norm, residual)          # whatever was prepared for this norm is not used here
        qkv = rt.empty((residual.shape[0], self.w_qkv.shape[0]))
        ops.norm_linear(residual, prologue[0], prologue[1], self.w_qkv, qkv, bias=self.b_qkv)
        self._attend(ctx, qkv, residual, binding, branch)
        return True

    def _attend(self, ctx, qkv, residual, binding, branch=None):
        """From the joint product [q | k | v | gate] of the step's rows to the output projection."""
        rt, ops = self.rt, self.rt.ops
        rows = qkv.shape[0]
        nh, nkv, d, dv = self.heads, self.kv_heads, self.head_dim, self.v_dim
        tables = ctx.tables[binding.group]
        if self.position is not None:
            cos, sin, dims = self.position.cos, self.position.sin, self.position.dims
        else:
            cos, sin, dims, _ = ctx.no_rotation(rt)
        q = rt.empty((rows, nh * d))
        writes = binding.writes
        ops.normed_rope_store(qkv, NORM_MODES[self.norm_mode], self.q_weight, self.k_weight, self.eps, q, ctx.row_pos, ctx.row_seg,
                              tables, cos, sin, binding.k_pages if writes else None, binding.v_pages if writes else None,
                              nh, nkv, d, dv, dims, binding.page_size, self.key_chunk, values_from_keys=self.values_from_keys)
        out = rt.empty((rows, nh * dv))
        if self.window is not None:
            if writes:
                ops.pool_blocks(binding.k_pages, binding.v_pages, binding.pool_k, binding.pool_v, tables, ctx.row_pos, ctx.row_seg,
                                nkv, d, dv, binding.page_size, self.key_chunk, int(self.pool))
            ops.pooled_window_attention(q, binding.k_pages, binding.v_pages, binding.pool_k, binding.pool_v, tables, ctx.row_pos,
                                        ctx.row_seg, ctx.seg_start, out, nh, nkv, d, dv, binding.page_size, self.scale,
                                        int(self.window), int(self.pool), self.key_chunk, max_context=ctx.max_context)
        else:
            extra = {}
            if dv != d:
                extra["v_dim"] = dv
            if self.key_chunk != self.KEY_CHUNK:
                extra["key_chunk"] = self.key_chunk
            if self.sinks is not None:
                extra["sinks"] = self.sinks
            single_from = ctx.single_rows_from()
            if 0 < single_from < ctx.num_segments:
                single_from = ctx.num_segments
            ops.attention(q, binding.k_pages, binding.v_pages, tables, ctx.row_pos, ctx.row_seg, ctx.seg_start, out, nh, nkv, d,
                          binding.page_size, self.scale, None, ctx.max_context, single_from=single_from,
                          workspace=ctx.attention_workspace(rt, rows, nh, nkv, d), **extra)
        if self.gated:
            gated = rt.empty((rows, nh * dv))
            out = ops.gated_norm(out, None, 0.0, qkv[:, self.gate_at:], gated)
        if branch is not None:
            ops.linear(out, self.w_o, branch, bias=self.b_o)
        elif not add_and_prepare(ctx, ops, out, self.w_o, residual, self.b_o):
            ops.linear(out, self.w_o, residual, bias=self.b_o, accumulate=True)


register_part("mixer", "normed_attention", NormedAttention)
