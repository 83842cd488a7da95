"""Attention over the paged cache.

q, k, v = one product with the concatenated projection matrix; rotary on q and k; k and v stored
in the pages of the row's request; every row attends to the keys of its request at positions
[pos - window + 1, pos] (all from 0 without a window) and, with `chunk`, to none before the start of its
own chunk of that many positions (chunks counted from the request's first position), heads grouped over
the key/value heads (h -> h / (heads / kv_heads)); values may have a width of their own (`value_head_dim`);
output projection added to the residual stream, or stored as a branch for a block that norms it first.
Options a design may ask for: `qk_norm_eps` (every head of q and of k is divided by its root mean square over the head's
lanes, no weight; such a layer has no rotary), `sink` (a learned number a head whose exponential joins the softmax's
denominator: a term without key or value, neither scaled nor masked), `output_gate` (the heads' outputs are multiplied lane
by lane with sigmoid(W_g h) before the output projection; W_g rides in the q/k/v product)
(rust/engine/src/rust_decoder.rs:8827-8835 projections, :8895-8898 rotary, :8955-8963 cache write,
:6065-6166 scores, mask, softmax and output, :9025 and :9059 projection and residual).
"""
from __future__ import annotations

import torch

from ..config.spec import PartSpec
from ..registry import part_class, register_part
from .base import INIT_BIAS, INIT_MATRIX, KVNeed, Mixer, add_and_prepare, fused_form, take_prepared


class PagedAttention(Mixer):
    graph_safe = True      # forward launches kernels only: no per-step decision on the host
    stores_branch = True   # forward(..., branch=t) stores the output projection in t instead of adding it to the stream
    KEY_CHUNK = 8          # values of a key that lie together in a page (csrc/common.h, key_offset)
    MATRIX_CORE_WIDTHS = (32, 64, 128)      # head sizes the matrix-core attention kernels take

    @classmethod
    def tensor_shapes(cls, spec):
        h, nh, nkv, d = spec["hidden_size"], spec["num_heads"], spec["num_kv_heads"], spec["head_dim"]
        dv = spec.get("value_head_dim") or d
        return {
            "q": ((nh * d, h), INIT_MATRIX), "k": ((nkv * d, h), INIT_MATRIX), "v": ((nkv * dv, h), INIT_MATRIX),
            "o": ((h, nh * dv), INIT_MATRIX),
            "q_bias": ((nh * d,), INIT_BIAS), "k_bias": ((nkv * d,), INIT_BIAS), "v_bias": ((nkv * dv,), INIT_BIAS),
            "o_bias": ((h,), INIT_BIAS),
            "g": ((nh * dv, h), INIT_MATRIX), "sink": ((nh,), INIT_BIAS),
        }

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.kv_heads = int(spec["num_kv_heads"])
        self.head_dim = int(spec["head_dim"])
        self.scale = float(spec["scale"])
        self.window = spec.get("window")
        self.chunk = spec.get("chunk")
        self.v_dim = int(spec.get("value_head_dim") or self.head_dim)
        if self.heads % self.kv_heads != 0:
            raise ValueError(f"head count {self.heads} is not a multiple of key/value head count {self.kv_heads}")
        if self.window is not None and self.window <= 0:
            raise ValueError("an attention window must be positive")
        if self.chunk is not None and self.chunk <= 0:
            raise ValueError("a chunk of positions must be positive")
        # The matrix-core kernels (bfloat16) read keys and values of ONE width of 32, 64 or 128 lanes.  A layer whose two
        # widths differ, or fit none of the three, runs them all the same: heads are widened to the next such width with
        # lanes that are zero (zero rows of the q, k and v projections, zero columns of the output projection).  A zero lane
        # adds exactly nothing to a score or an output, and rotary only touches the first lanes, so the results are the
        # layer's own; the pages are wider than the layer needs, which is the price.  An architecture asks for it
        # with `widen_heads` in the mixer's spec.
        self.checkpoint_dims = (self.head_dim, self.v_dim)
        widest = max(self.head_dim, self.v_dim)
        fits = next((w for w in self.MATRIX_CORE_WIDTHS if w >= widest), None)
        if (spec.get("widen_heads", False) and rt.dtype == torch.bfloat16 and fits is not None and hasattr(rt.ops, "tile_for_decode")
                and (self.head_dim, self.v_dim) != (fits, fits)):
            self.head_dim = self.v_dim = fits
        # keys lie in chunks of 8 values inside a page where the head size allows it (what the matrix-core kernels read);
        # other head sizes store a head's lanes one by one and run the plain kernels
        self.key_chunk = self.KEY_CHUNK if self.head_dim % self.KEY_CHUNK == 0 else 1
        # what only the plain kernels take (values of another width than the keys, a chunk of positions in the fused
        # store, key lanes one by one): named once, so that every call hands over the same arguments
        self.shape_args = {}
        if self.v_dim != self.head_dim:
            self.shape_args["v_dim"] = self.v_dim
        if self.key_chunk != self.KEY_CHUNK:
            self.shape_args["key_chunk"] = self.key_chunk
        self.qk_norm_eps = spec.get("qk_norm_eps")
        if self.qk_norm_eps is not None:
            self.qk_norm_eps = float(self.qk_norm_eps)
            if not self.qk_norm_eps > 0.0:
                raise ValueError("the norm over a head's lanes needs a positive eps")
            if spec.get("position") is not None:
                raise ValueError("heads normed over their lanes come without rotary here: no kernel does both")
        self.gated = bool(spec.get("output_gate", False))
        if self.gated and self.qk_norm_eps is None:
            raise ValueError("an output gate rides in the product of a layer with normed heads: ask for qk_norm_eps too")
        self.sink = rt.vector(weights["sink"]) if spec.get("sink", False) else None
        position = spec.get("position")
        self.position = None
        if position is not None:
            position = dict(position)
            kind = position.pop("kind")
            self.position = part_class("position", kind)(PartSpec(kind, position), {}, rt)
        # Rotary with the checkpoint's pairing (l, l + dims/2): the rows of the q and k projections are
        # reordered inside every head so that the partners sit next to each other (2l, 2l + 1), the
        # pairing the kernels rotate.  q . k does not change when both are reordered alike
        # (the reference's importer does the same: rust/checkpoint/src/convert.rs:2713-2745).
        self.pairing = 1
        order_q = order_k = None
        d0, dv0 = self.checkpoint_dims
        if self.position is not None and self.position.pairing == 0:
            order_q = self._pair_order(self.heads, d0, self.position.dims).to(rt.device)
            order_k = self._pair_order(self.kv_heads, d0, self.position.dims).to(rt.device)
        elif self.position is not None:
            self.pairing = self.position.pairing
        reorder = lambda t, order: t if order is None or t is None else t.index_select(0, order)

        def widen(t, heads, have, want):
            """Rows of `heads` heads of `have` lanes -> heads of `want` lanes, the new lanes zero."""
            if t is None or have == want:
                return t
            wide = torch.zeros((heads, want) + tuple(t.shape[1:]), dtype=t.dtype, device=t.device)
            wide[:, :have] = t.view(heads, have, *t.shape[1:])
            return wide.view(heads * want, *t.shape[1:])

        # one matrix for q, k and v: the normed input is read once
        pieces = [widen(reorder(rt.matrix(weights["q"]), order_q), self.heads, d0, self.head_dim),
                  widen(reorder(rt.matrix(weights["k"]), order_k), self.kv_heads, d0, self.head_dim),
                  widen(rt.matrix(weights["v"]), self.kv_heads, dv0, self.v_dim)]
        if self.gated:         # the gate's rows behind q, k and v: a zero lane of a widened head is gated by 1/2 and stays zero
            pieces.append(widen(rt.matrix(weights["g"]), self.heads, dv0, self.v_dim))
        self.w_qkv = torch.cat(pieces, dim=0).contiguous()
        self.w_o = rt.matrix(weights["o"])
        if dv0 != self.v_dim:
            self.w_o = widen(self.w_o.t().contiguous(), self.heads, dv0, self.v_dim).t().contiguous()
        rt.tile_for_decode(self.w_o)
        rt.tile_for_decode(self.w_qkv, priority=1)
        biases = [widen(reorder(None if weights.get("q_bias") is None else rt.vector(weights["q_bias"]), order_q), self.heads, d0, self.head_dim),
                  widen(reorder(None if weights.get("k_bias") is None else rt.vector(weights["k_bias"]), order_k), self.kv_heads, d0, self.head_dim),
                  widen(None if weights.get("v_bias") is None else rt.vector(weights["v_bias"]), self.kv_heads, dv0, self.v_dim)]
        self.b_qkv = None
        if any(b is not None for b in biases):
            sizes = (self.heads * self.head_dim, self.kv_heads * self.head_dim, self.kv_heads * self.v_dim)
            self.b_qkv = torch.cat([b if b is not None else torch.zeros(n, dtype=torch.float32, device=rt.device)
                                    for b, n in zip(biases, sizes)]).contiguous()
        self.b_o = rt.vector(weights["o_bias"]) if weights.get("o_bias") is not None else None

    @staticmethod
    def _pair_order(heads: int, head_dim: int, rope_dims: int) -> torch.Tensor:
        """New row -> old row: inside every head, row 2l comes from l and row 2l + 1 from l + rope_dims/2."""
        half = rope_dims // 2
        one = []
        for l in range(half):
            one += [l, l + half]
        one += list(range(rope_dims, head_dim))
        return torch.tensor([h * head_dim + j for h in range(heads) for j in one], dtype=torch.long)

    def cache_need(self):
        # keys in chunks of 8 values (16 bytes in bfloat16) where the head size allows it.  A chunk of positions is a mask,
        # not a window: earlier chunks keep their pages until the request ends.
        return KVNeed(self.kv_heads, self.head_dim, self.v_dim, self.window, key_chunk=self.key_chunk)

    def forward(self, ctx, h, residual, binding, branch=None):
        rt, ops = self.rt, self.rt.ops
        rows = h.shape[0]
        nh, nkv, d = self.heads, self.kv_heads, self.head_dim
        qkv = rt.empty((rows, self.w_qkv.shape[0]))
        ops.linear(h, self.w_qkv, qkv, bias=self.b_qkv)
        tables = ctx.tables[binding.group]
        if self.qk_norm_eps is not None:
            ops.head_norm_kv_store(qkv, self.qk_norm_eps, self.checkpoint_dims[0], ctx.row_pos, ctx.row_seg, tables,
                                   binding.k_pages if binding.writes else None, binding.v_pages if binding.writes else None,
                                   nh, nkv, d, binding.page_size, v_dim=self.v_dim, key_chunk=self.key_chunk)
            gate = qkv[:, (nh + nkv) * d + nkv * self.v_dim:] if self.gated else None
            self._attend_and_project(ctx, qkv[:, : nh * d], residual, binding, branch=branch, gate=gate)
            return
        if self.position is not None:
            cos, sin, dims, pairing = self.position.cos, self.position.sin, self.position.dims, self.pairing
        else:
            cos, sin, dims, pairing = ctx.no_rotation(rt)
        ops.rope_kv_store(qkv, ctx.row_pos, ctx.row_seg, tables, cos, sin,
                          binding.k_pages if binding.writes else None, binding.v_pages if binding.writes else None,
                          nh, nkv, d, dims, pairing, binding.page_size, **self.shape_args)
        self._attend_and_project(ctx, qkv[:, : nh * d], residual, binding, branch=branch)

    def forward_from_residual(self, ctx, residual, norm, binding, branch=None) -> bool:
        """Decode-sized steps in bfloat16: the norm before the mixer, the q/k/v product, rotary and the
        cache store are one kernel.  False: not taken, the block runs norm and `forward`."""
        rt, ops = self.rt, self.rt.ops
        rows = residual.shape[0]
        prologue = getattr(norm, "fused_prologue", lambda: None)()
        form = fused_form(ops, rows, self.hidden, self.w_qkv) if hasattr(ops, "norm_qkv_rope_store") else None
        if rt.dtype != torch.bfloat16 or self.pairing != 1 or prologue is None or form is None or self.head_dim % 4 != 0:
            return False
        if self.shape_args or self.qk_norm_eps is not None or self.sink is not None:
            return False         # the fused store takes keys and values of one width, keys in chunks of 8, and rotates
        norm_scale, norm_eps = prologue
        nh, nkv, d = self.heads, self.kv_heads, self.head_dim
        if self.position is not None:
            cos, sin, dims = self.position.cos, self.position.sin, self.position.dims
        else:
            cos, sin, dims, _ = ctx.no_rotation(rt)
        q = rt.empty((rows, nh * d))
        prepared = take_prepared(ctx, norm, residual)      # the sum before this norm may have computed its first steps
        if prepared is None and form == "chunks":
            prepared = ops.prepare_norm(residual, norm_scale)
        ops.norm_qkv_rope_store(residual, norm_scale, norm_eps, self.w_qkv, q, ctx.row_pos, ctx.row_seg,
                                ctx.tables[binding.group], cos, sin, binding.k_pages if binding.writes else None,
                                binding.v_pages if binding.writes else None, nh, nkv, d, dims, binding.page_size,
                                bias=self.b_qkv, **({"prepared": prepared} if prepared is not None else {}))
        self._attend_and_project(ctx, q, residual, binding, branch=branch)
        return True

    def forward_branch(self, ctx, h, binding):
        """The mixer's output as a tensor of its own instead of a sum into the residual stream, when
        that lets the block fold the residual add into the next norm (large bfloat16 steps whose
        products go to the GEMM library, which has no residual epilogue).  None: not taken."""
        rt, ops = self.rt, self.rt.ops
        rows = h.shape[0]
        start = getattr(ops, "library_gemm_from", None)
        if rt.dtype != torch.bfloat16 or start is None or rows < start or self.b_o is not None:
            return None
        branch = rt.empty((rows, self.hidden))
        self.forward(ctx, h, None, binding, branch=branch)
        return branch

    SPLIT_SINGLE_ROWS_FROM = 3072      # context length (measured: equal cost at about 4,000 keys)

    def _attend_and_project(self, ctx, q, residual, binding, branch=None, gate=None):
        rt, ops = self.rt, self.rt.ops
        rows = q.shape[0]
        nh, nkv, d = self.heads, self.kv_heads, self.head_dim
        tables = ctx.tables[binding.group]
        out = rt.empty((rows, nh * self.v_dim))
        shape_args = dict(self.shape_args, chunk=self.chunk) if self.chunk else self.shape_args
        if self.sink is not None:
            shape_args = dict(shape_args, sinks=self.sink)
        # Single rows behind portions of prompts: with long contexts they go to the kernel that splits a context over
        # workgroups (a second launch); with short ones they ride along in the portions' launch, which is faster then.
        single_from = ctx.single_rows_from()
        if 0 < single_from < ctx.num_segments and ctx.single_max_context < self.SPLIT_SINGLE_ROWS_FROM:
            single_from = ctx.num_segments
        slopes = getattr(self.position, "score_slopes", None)      # a position encoding may bias scores by distance
        if slopes is not None:
            ops.attention(q, binding.k_pages, binding.v_pages, tables, ctx.row_pos, ctx.row_seg, ctx.seg_start,
                          out, nh, nkv, d, binding.page_size, self.scale, self.window, ctx.max_context, head_slopes=slopes,
                          **shape_args)
        else:
            ops.attention(q, binding.k_pages, binding.v_pages, tables, ctx.row_pos, ctx.row_seg, ctx.seg_start,
                          out, nh, nkv, d, binding.page_size, self.scale, self.window, ctx.max_context,
                          single_from=single_from,
                          workspace=ctx.attention_workspace(rt, rows, nh, nkv, d), **shape_args)
        if gate is not None:
            gated = rt.empty((rows, nh * self.v_dim))
            out = ops.gated_norm(out, None, 0.0, gate, gated)
        if branch is not None:
            ops.linear(out, self.w_o, branch, bias=self.b_o)
        elif not add_and_prepare(ctx, ops, out, self.w_o, residual, self.b_o):
            ops.linear(out, self.w_o, residual, bias=self.b_o, accumulate=True)


register_part("mixer", "attention", PagedAttention)
