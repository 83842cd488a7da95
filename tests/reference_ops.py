"""Plain PyTorch versions of every kernel of the library, one function per kernel, with the
kernels' own signatures.  They compute in float64 on whatever device the tensors are on and
round once to the output type.

Two uses: the GPU tests compare each HIP kernel with its function here, and the CPU tests hand
a `ReferenceOps` to the engine in place of the kernel library, so that the step function, the
cache and the scheduler can be exercised without a GPU.  The product never imports this file.
"""
import math

import numpy as np
import torch

import plain_llama


class ReferenceOps:
    def embed(self, ids, table, out, scale=1.0):
        out.copy_((table[ids.long()].double() * scale).to(out.dtype))
        return out

    def rmsnorm(self, x, weight, eps, out, rows=None):
        src = x if rows is None else x[rows.long()]
        src = src.double()
        inv = 1.0 / torch.sqrt((src * src).sum(-1, keepdim=True) / src.shape[-1] + eps)
        out.copy_((src * (inv * weight.double())).to(out.dtype))
        return out

    def linear(self, x, w, out, bias=None, accumulate=False):
        y = x.double() @ w.double().T
        if bias is not None:
            y = y + bias.double()
        if accumulate:
            out.add_(y.to(out.dtype))
        else:
            out.copy_(y.to(out.dtype))
        return out

    # fused forms of decode steps: the same formulas, composed
    def fused_decode_supported(self, rows, width):
        return 1 <= rows <= 16 and width % 8 == 0

    def _normed(self, x, norm_weight, eps):
        x = x.double()
        return x * (torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * norm_weight.double())

    def norm_linear(self, x, norm_weight, eps, w, out, bias=None):
        y = self._normed(x, norm_weight, eps) @ w.double().T
        out.copy_((y if bias is None else y + bias.double()).to(out.dtype))
        return out

    def gate_up_swiglu(self, x, w_gate_up, out, bias=None):
        y = x.double() @ w_gate_up.double().T
        if bias is not None:
            y = y + bias.double()
        inter = y.shape[1] // 2
        g, u = y[:, :inter], y[:, inter:]
        out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))
        return out

    def norm_gate_up_swiglu(self, x, norm_weight, eps, w_gate_up, out, bias=None):
        y = self._normed(x, norm_weight, eps) @ w_gate_up.double().T
        if bias is not None:
            y = y + bias.double()
        inter = y.shape[1] // 2
        g, u = y[:, :inter], y[:, inter:]
        out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))
        return out

    def norm_qkv_rope_store(self, x, norm_weight, eps, w_qkv, q_out, row_pos, row_seg, tables, cos, sin, k_pages, v_pages,
                            heads, kv_heads, head_dim, rope_dims, page_size, bias=None):
        y = self._normed(x, norm_weight, eps) @ w_qkv.double().T
        if bias is not None:
            y = y + bias.double()
        qkv = y.clone()                 # rotated in float64, rounded once when stored
        kp = None if k_pages is None else k_pages.double()
        vp = None if v_pages is None else v_pages.double()
        self.rope_kv_store(qkv, row_pos, row_seg, tables, cos, sin, kp, vp, heads, kv_heads, head_dim, rope_dims, 1, page_size)
        q_out.copy_(qkv[:, : heads * head_dim].to(q_out.dtype))
        if k_pages is not None:
            k_pages.copy_(kp.to(k_pages.dtype))
            v_pages.copy_(vp.to(v_pages.dtype))
        return q_out

    def add_rmsnorm(self, x, branch, weight, eps, out):
        x.add_(branch.to(x.dtype))
        return self.rmsnorm(x, weight, eps, out)

    def add_residual(self, residual, branch):
        residual.add_(branch.to(residual.dtype))
        return residual

    def swiglu(self, gate_up, out):
        inter = gate_up.shape[1] // 2
        g, u = gate_up[:, :inter].double(), gate_up[:, inter:].double()
        out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))
        return out

    def rope_kv_store(self, qkv, row_pos, row_seg, tables, cos, sin, k_pages, v_pages, heads, kv_heads, head_dim,
                      rope_dims, pairing, page_size, v_dim=None, key_chunk=8):
        rows = qkv.shape[0]
        half = rope_dims // 2
        v_dim = head_dim if v_dim is None else v_dim
        rotated = (heads + kv_heads) * head_dim
        view = qkv[:, :rotated].view(rows, heads + kv_heads, head_dim)
        for r in range(rows):
            seg = int(row_seg[r])
            if seg < 0:
                continue
            pos = int(row_pos[r])
            c, s = (cos[pos].double(), sin[pos].double()) if half else (None, None)
            if pairing == 0:
                ia, ib = torch.arange(half), torch.arange(half) + half
            else:
                ia, ib = torch.arange(half) * 2, torch.arange(half) * 2 + 1
            ia, ib = ia.to(qkv.device), ib.to(qkv.device)
            for h in range(heads + kv_heads if half else 0):
                a, b = view[r, h, ia].double(), view[r, h, ib].double()
                view[r, h, ia] = (a * c - b * s).to(qkv.dtype)
                view[r, h, ib] = (b * c + a * s).to(qkv.dtype)
            if k_pages is None:
                continue
            page = int(tables[seg, pos // page_size])
            off = pos % page_size
            # keys lie chunk by chunk in a page: [page][kv_head][head_dim / key_chunk][token][key_chunk]
            k_pages[page, :, :, off, :] = view[r, heads:heads + kv_heads, :].reshape(kv_heads, head_dim // key_chunk, key_chunk)
            v_pages[page, :, :, off] = qkv[r, rotated:].view(kv_heads, v_dim)

    def attention_workspace_bytes(self, rows, heads, kv_heads, head_dim, max_context):
        return 0

    def attention(self, q, k_pages, v_pages, tables, row_pos, row_seg, seg_start, out, heads, kv_heads, head_dim, page_size, scale,
                  window, max_context, uniform_rows=0, workspace=None, single_from=None, head_slopes=None, v_dim=None, chunk=None,
                  key_chunk=8, sinks=None):
        rows = q.shape[0]
        group = heads // kv_heads
        v_dim = head_dim if v_dim is None else v_dim
        for r in range(rows):
            seg = int(row_seg[r])
            if seg < 0:
                out[r] = 0
                continue
            pos = int(row_pos[r])
            n = pos + 1
            lo = max(0, n - window) if window else 0
            if chunk:
                lo = max(lo, pos - pos % chunk)
            keys = torch.arange(lo, n, device=q.device)
            pages = tables[seg, (keys // page_size).long()].long()
            offs = (keys % page_size).long()
            k = k_pages[pages, :, :, offs, :].double().reshape(len(keys), kv_heads, head_dim)     # [n, kv_heads, d]
            v = v_pages[pages, :, :, offs].double()          # [n, kv_heads, d]
            qr = q[r].double().view(heads, head_dim)
            for h in range(heads):
                s = (k[:, h // group, :] @ qr[h]) * scale
                if head_slopes is not None:
                    s = s + float(head_slopes[h]) * (keys - pos).double()
                if sinks is not None:         # one more term in the denominator, without a value
                    p = torch.softmax(torch.cat([s, sinks[h].double().reshape(1)]), dim=0)[:-1]
                else:
                    p = torch.softmax(s, dim=0)
                out[r, h * v_dim:(h + 1) * v_dim] = (p @ v[:, h // group, :]).to(out.dtype)
        return out

    # ---- a branch normed on its way into the stream; routed experts ----
    def postnorm_add(self, x, branch, gain, eps, parts=1, next_weight=None, next_eps=0.0, next_out=None, part_weights=None):
        rows, width = x.shape
        v = branch.double().view(rows, parts, width)
        if part_weights is not None:
            v = v * part_weights.double().view(rows, parts, 1)
        v = v.sum(1)
        if eps is not None:
            v = v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)
        x.copy_((x.double() + v * gain.double()).to(x.dtype))
        if next_weight is not None:
            self.rmsnorm(x, next_weight, next_eps, next_out)
        return x

    def route_topk(self, h, w_router, top, ids, weights, score="sigmoid", renormalize=False, route_scale=1.0):
        z = (h.double() @ w_router.double().T).float()
        score = torch.sigmoid(z) if score == "sigmoid" else torch.softmax(z, dim=1)
        order = torch.sort(score, dim=1, descending=True, stable=True)[1][:, :top]
        ids.copy_(order.to(ids.dtype))
        picked = torch.gather(score, 1, order)
        if renormalize:
            picked = picked / (picked.sum(1, keepdim=True) + 1e-20)
        weights.copy_(picked * route_scale)
        return ids, weights

    # ---- what a sequence carries outside the pages: a short convolution's inputs, a linear attention's matrix ----
    def short_conv(self, x, w, state, row_seg, seg_start, slots, out):
        rows, width = x.shape
        taps = w.shape[1]
        keep = taps - 1
        res = torch.zeros_like(out)
        starts = [int(v) for v in seg_start]
        for s in range(len(starts) - 1):
            r0, r1 = starts[s], starts[s + 1]
            if r1 <= r0 or int(row_seg[r0]) < 0:
                continue
            slot = int(slots[s])
            old = state[slot].double() if keep else x.new_zeros((0, width)).double()
            seq = torch.cat([old, x[r0:r1].double()])                      # inputs at t - keep .. t + n - 1
            for t in range(r1 - r0):
                acc = (seq[t:t + taps] * w.double().T).sum(0)              # w[:, j] meets the input taps - 1 - j back
                res[r0 + t] = (x[r0 + t].double() + acc).to(out.dtype)
            if keep:
                state[slot] = seq[-keep:].to(state.dtype)
        out.copy_(res)
        return out

    def linear_attention(self, qkv, decay_hi, decay_lo, state, row_seg, seg_start, slots, out, heads, dim, vdim, activation="silu"):
        act = (lambda z: z / (1.0 + torch.exp(-z))) if activation == "silu" else (lambda z: z)
        decay = decay_hi.double() + decay_lo.double()
        starts = [int(v) for v in seg_start]
        out.zero_()
        for s in range(len(starts) - 1):
            r0, r1 = starts[s], starts[s + 1]
            if r1 <= r0 or int(row_seg[r0]) < 0:
                continue
            S = state[int(slots[s])].double()
            for r in range(r0, r1):
                row = qkv[r].double()
                q = act(row[:heads * dim]).view(heads, dim)
                k = act(row[heads * dim:2 * heads * dim]).view(heads, dim)
                v = act(row[2 * heads * dim:2 * heads * dim + heads * vdim]).view(heads, vdim)
                S = decay.view(heads, 1, 1) * S + k.unsqueeze(2) * v.unsqueeze(1)
                out[r] = torch.einsum("hdv,hd->hv", S, q).reshape(-1).to(out.dtype)
            state[int(slots[s])] = S.to(state.dtype)
        return out

    def gated_norm(self, x, weight, eps, gate, out):
        v = x.double()
        if weight is not None:
            v = v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * weight.double()
        out.copy_((v * torch.sigmoid(gate.double())).to(out.dtype))
        return out

    def polynorm(self, z, coeffs, eps, out):
        z = z.double()
        c = coeffs.double()
        n = lambda t: t / torch.sqrt((t * t).mean(-1, keepdim=True) + eps)
        out.copy_((c[0] * n(z) + c[1] * n(z * z) + c[2] * n(z * z * z) + c[3]).to(out.dtype))
        return out

    def head_norm_kv_store(self, qkv, eps, norm_dim, row_pos, row_seg, tables, k_pages, v_pages, heads, kv_heads, head_dim,
                           page_size, v_dim=None, key_chunk=8):
        rows = qkv.shape[0]
        v_dim = head_dim if v_dim is None else v_dim
        normed = (heads + kv_heads) * head_dim
        view = qkv[:, :normed].view(rows, heads + kv_heads, head_dim)
        for r in range(rows):
            seg = int(row_seg[r])
            if seg < 0:
                continue
            a = view[r].double()
            y = (a / torch.sqrt((a * a).sum(-1, keepdim=True) / norm_dim + eps)).to(qkv.dtype)
            view[r, :heads] = y[:heads]
            if k_pages is None:
                continue
            pos = int(row_pos[r])
            page, off = int(tables[seg, pos // page_size]), pos % page_size
            k_pages[page, :, :, off, :] = y[heads:].reshape(kv_heads, head_dim // key_chunk, key_chunk)
            v_pages[page, :, :, off] = qkv[r, normed:normed + kv_heads * v_dim].view(kv_heads, v_dim)

    def experts_gate_up(self, h, ids, weights, w_gate_up, act, limit=0.0, alpha=1.0, up_offset=0.0):
        rows, top = ids.shape
        inter = w_gate_up.shape[1] // 2
        for r in range(rows):
            for k in range(top):
                x = (h[r].float() * weights[r, k]).to(h.dtype).double()
                y = w_gate_up[int(ids[r, k])].double() @ x
                g, u = y[:inter], y[inter:]
                if limit > 0:
                    g, u = torch.clamp(g, max=limit), torch.clamp(u, -limit, limit)
                act[r * top + k] = (g / (1.0 + torch.exp(-alpha * g)) * (u + up_offset)).to(act.dtype)
        return act

    def experts_down(self, act, ids, w_down, out):
        flat = ids.reshape(-1)
        for p in range(act.shape[0]):
            out[p] = (w_down[int(flat[p])].double() @ act[p].double()).to(out.dtype)
        return out

    # ---- parts of other layer designs: two norms of one row, clamped gated activation, what a pass of looped layers
    # adds to the stream, logits times a constant, attention whose heads' scores are mixed before the softmax ----
    def rmsnorm_pair(self, x, w1, eps1, out1, w2=None, eps2=None, out2=None):
        self.rmsnorm(x, w1, eps1, out1)
        if w2 is not None:
            self.rmsnorm(x, w2, eps1 if eps2 is None else eps2, out2)
        return out1, out2

    def glu_clamped(self, gate_up, out, limit, alpha, up_offset):
        inter = gate_up.shape[1] // 2
        g, u = gate_up[:, :inter].double(), gate_up[:, inter:].double()
        if limit > 0:
            g, u = torch.clamp(g, max=limit), torch.clamp(u, -limit, limit)
        out.copy_((g / (1.0 + torch.exp(-alpha * g)) * (u + up_offset)).to(out.dtype))
        return out

    def scale_(self, x, scale):
        x.mul_(scale)
        return x

    def stream_add(self, x, ids=None, table=None, scale=1.0, vec=None):
        y = x.double()
        if table is not None:
            y = y + table[ids.long()].double() * scale
        if vec is not None:
            y = y + vec.double()
        x.copy_(y.to(x.dtype))
        return x

    def qk_norm_rope_store(self, qkv, q_weight, k_weight, eps, q_out, row_pos, row_seg, tables, cos, sin, k_pages, v_pages,
                           heads, kv_heads, k_dim, v_dim, rope_dims, page_size, key_chunk):
        nq, nk, nv = heads * k_dim, kv_heads * k_dim, kv_heads * v_dim
        half = rope_dims // 2
        for r in range(qkv.shape[0]):
            seg = int(row_seg[r])
            if seg < 0:
                continue
            pos = int(row_pos[r])
            q, k = qkv[r, :nq].double(), qkv[r, nq:nq + nk].double()
            q = (q / torch.sqrt((q * q).mean() + eps) * q_weight.double()).view(heads, k_dim).clone()
            k = (k / torch.sqrt((k * k).mean() + eps) * k_weight.double()).view(kv_heads, k_dim).clone()
            if half:
                c, s = cos[pos].double(), sin[pos].double()
                for t in (q, k):
                    a, b = t[:, :half].clone(), t[:, half:rope_dims].clone()
                    t[:, :half] = a * c - b * s
                    t[:, half:rope_dims] = b * c + a * s
            q_out[r] = q.reshape(-1).to(q_out.dtype)
            if k_pages is None:
                continue
            page, off = int(tables[seg, pos // page_size]), pos % page_size
            k_pages[page, :, :, off, :] = k.view(kv_heads, k_dim // key_chunk, key_chunk).to(k_pages.dtype)
            v_pages[page, :, :, off] = qkv[r, nq + nk:nq + nk + nv].view(kv_heads, v_dim)
        return q_out

    def talking_attention(self, q, gate, k_pages, v_pages, tables, row_pos, row_seg, seg_start, talk, temp, out, heads, kv_heads,
                          k_dim, v_dim, page_size, scale, chunk, key_chunk, max_context):
        group = heads // kv_heads
        for r in range(q.shape[0]):
            seg = int(row_seg[r])
            if seg < 0:
                out[r] = 0
                continue
            pos = int(row_pos[r])
            lo = pos - pos % chunk if chunk else 0
            keys = torch.arange(lo, pos + 1, device=q.device)
            pages = tables[seg, (keys // page_size).long()].long()
            offs = (keys % page_size).long()
            k = k_pages[pages, :, :, offs, :].double().reshape(len(keys), kv_heads, k_dim)
            v = v_pages[pages, :, :, offs].double()                                    # [n, kv_heads, v_dim]
            qr = q[r].double().view(heads, k_dim)
            raw = torch.stack([(k[:, h // group, :] @ qr[h]) * scale * float(temp[h]) for h in range(heads)])    # [heads, n]
            p = torch.softmax(talk.double() @ raw, dim=1)
            for h in range(heads):
                o = p[h] @ v[:, h // group, :]
                if gate is not None:
                    o = o / (1.0 + torch.exp(-gate[r, h].double()))
                out[r, h * v_dim:(h + 1) * v_dim] = o.to(out.dtype)
        return out

    # ---- attention with normed heads or projections, pooled blocks behind a window, sigmoid weights; retention's operands;
    # routers with groups; experts without a gate; what a pass of looped layers mixes into the stream ----
    def normed_rope_store(self, qkv, norm_mode, q_weight, k_weight, eps, q_out, row_pos, row_seg, tables, cos, sin, k_pages, v_pages,
                          heads, kv_heads, k_dim, v_dim, rope_dims, page_size, key_chunk, values_from_keys=False):
        nq, nk, nv = heads * k_dim, kv_heads * k_dim, kv_heads * v_dim
        half = rope_dims // 2
        for r in range(qkv.shape[0]):
            seg = int(row_seg[r])
            if seg < 0:
                continue
            pos = int(row_pos[r])
            q, k = qkv[r, :nq].double(), qkv[r, nq:nq + nk].double()
            raw_k = qkv[r, nq:nq + nk]
            if norm_mode == 2:        # one mean over the whole projection
                q = q / torch.sqrt((q * q).mean() + eps) * q_weight.double()
                k = k / torch.sqrt((k * k).mean() + eps) * k_weight.double()
            q, k = q.view(heads, k_dim).clone(), k.view(kv_heads, k_dim).clone()
            if norm_mode == 1:        # a mean a head, one weight vector for all heads
                q = q / torch.sqrt((q * q).mean(-1, keepdim=True) + eps) * q_weight.double()
                k = k / torch.sqrt((k * k).mean(-1, keepdim=True) + eps) * k_weight.double()
            if half:
                c, s = cos[pos].double(), sin[pos].double()
                for t in (q, k):
                    a, b = t[:, :half].clone(), t[:, half:rope_dims].clone()
                    t[:, :half] = a * c - b * s
                    t[:, half:rope_dims] = b * c + a * s
            q_out[r] = q.reshape(-1).to(q_out.dtype)
            if k_pages is None:
                continue
            page, off = int(tables[seg, pos // page_size]), pos % page_size
            k_pages[page, :, :, off, :] = k.view(kv_heads, k_dim // key_chunk, key_chunk).to(k_pages.dtype)
            v = raw_k if values_from_keys else qkv[r, nq + nk:nq + nk + nv]
            v_pages[page, :, :, off] = v.view(kv_heads, v_dim)
        return q_out

    def pool_blocks(self, k_pages, v_pages, pool_k, pool_v, tables, row_pos, row_seg, kv_heads, k_dim, v_dim, page_size, key_chunk, pool):
        for r in range(row_pos.shape[0]):
            seg, pos = int(row_seg[r]), int(row_pos[r])
            if seg < 0 or (pos + 1) % pool != 0:
                continue
            keys = torch.arange(pos - pool + 1, pos + 1)
            pages, offs = tables[seg, (keys // page_size).long()].long(), (keys % page_size).long()
            k = k_pages[pages, :, :, offs, :].double().reshape(pool, kv_heads, k_dim).mean(0)
            v = v_pages[pages, :, :, offs].double().mean(0)
            page, slot = int(tables[seg, pos // page_size]), (pos % page_size) // pool
            pool_k[page, :, slot] = k.to(pool_k.dtype)
            pool_v[page, :, slot] = v.to(pool_v.dtype)

    def pooled_window_attention(self, q, k_pages, v_pages, pool_k, pool_v, tables, row_pos, row_seg, seg_start, out, heads, kv_heads,
                                k_dim, v_dim, page_size, scale, window, pool, key_chunk, max_context=0):
        group = heads // kv_heads
        for r in range(q.shape[0]):
            seg = int(row_seg[r])
            if seg < 0:
                out[r] = 0
                continue
            pos = int(row_pos[r])
            keys = torch.arange(max(0, pos - window + 1), pos + 1)
            pages, offs = tables[seg, (keys // page_size).long()].long(), (keys % page_size).long()
            k = k_pages[pages, :, :, offs, :].double().reshape(len(keys), kv_heads, k_dim)
            v = v_pages[pages, :, :, offs].double()
            blocks = max(0, (pos - window + 1) // pool)
            if blocks:
                ends = torch.arange(blocks) * pool + pool - 1
                bp, slot = tables[seg, (ends // page_size).long()].long(), ((ends % page_size) // pool).long()
                k = torch.cat([pool_k[bp, :, slot].double(), k], 0)
                v = torch.cat([pool_v[bp, :, slot].double(), v], 0)
            qr = q[r].double().view(heads, k_dim)
            for h in range(heads):
                p = torch.softmax((k[:, h // group, :] @ qr[h]) * scale, dim=0)
                out[r, h * v_dim:(h + 1) * v_dim] = (p @ v[:, h // group, :]).to(out.dtype)
        return out

    def sigmoid_attention(self, q, k_pages, v_pages, tables, row_pos, row_seg, seg_start, out, heads, kv_heads, k_dim, v_dim, page_size,
                          scale, softcap, r1, r2, pb, temp_coef, temp_every, key_chunk, max_context=0):
        group = heads // kv_heads
        for r in range(q.shape[0]):
            seg = int(row_seg[r])
            if seg < 0:
                out[r] = 0
                continue
            pos = int(row_pos[r])
            keys = torch.arange(0, pos + 1)
            pages, offs = tables[seg, (keys // page_size).long()].long(), (keys % page_size).long()
            k = k_pages[pages, :, :, offs, :].double().reshape(len(keys), kv_heads, k_dim)
            v = v_pages[pages, :, :, offs].double()
            temp = 1.0 + temp_coef * math.log(math.floor((pos + 1) / temp_every) + 1.0)
            qr = q[r].double().view(heads, k_dim)
            for h in range(heads):
                s = (k[:, h // group, :] @ qr[h]) * (scale * temp)
                s = softcap * torch.tanh(s / softcap) - r1[h].double() * torch.log1p(r2[h].double() * (pos - keys).double())
                out[r, h * v_dim:(h + 1) * v_dim] = (torch.sigmoid(s + pb[h].double()) @ v[:, h // group, :]).to(out.dtype)
        return out

    def rotate_scale(self, qkv, out, row_pos, cos, sin, heads, dim, vdim, rope_dims, key_scale):
        nq, half = heads * dim, rope_dims // 2
        for r in range(qkv.shape[0]):
            pos = int(row_pos[r])
            q, k = qkv[r, :nq].double().view(heads, dim).clone(), qkv[r, nq:2 * nq].double().view(heads, dim).clone()
            if half:
                c, s = cos[pos].double(), sin[pos].double()
                for t in (q, k):
                    a, b = t[:, :half].clone(), t[:, half:rope_dims].clone()
                    t[:, :half] = a * c - b * s
                    t[:, half:rope_dims] = b * c + a * s
            out[r, :nq] = q.reshape(-1).to(out.dtype)
            out[r, nq:2 * nq] = (k * key_scale).reshape(-1).to(out.dtype)
            out[r, 2 * nq:] = qkv[r, 2 * nq:2 * nq + heads * vdim].to(out.dtype)
        return out

    def group_norm_gate(self, x, eps, group, gate, out, activation="silu"):
        rows, width = x.shape
        v = x.double().view(rows, width // group, group)
        v = (v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)).view(rows, width)
        g = gate.double()
        g = g / (1.0 + torch.exp(-g)) if activation == "silu" else torch.sigmoid(g)
        out.copy_((v * g).to(out.dtype))
        return out

    def route_grouped(self, h, w_router, correction, top, groups, groups_kept, ids, weights, route_scale=1.0):
        z = (h.double() @ w_router.double().T).float()
        score = torch.sigmoid(z)
        choice = score + correction.float()
        rows, E = choice.shape
        if groups > 1:
            per = E // groups
            best = torch.sort(choice.view(rows, groups, per), dim=-1, descending=True)[0][..., :2].sum(-1)
            kept = torch.sort(best, dim=1, descending=True, stable=True)[1][:, :groups_kept]
            allowed = torch.zeros((rows, groups), dtype=torch.bool)
            allowed.scatter_(1, kept, True)
            choice = torch.where(allowed.repeat_interleave(per, dim=1), choice, torch.full_like(choice, -math.inf))
        order = torch.sort(choice, dim=1, descending=True, stable=True)[1][:, :top]
        ids.copy_(order.to(ids.dtype))
        picked = torch.gather(score, 1, order)
        weights.copy_(picked / (picked.sum(1, keepdim=True) + 1e-20) * route_scale)
        return ids, weights

    def experts_up(self, h, ids, w_up, act, activation="relu2"):
        rows, top = ids.shape
        for r in range(rows):
            for k in range(top):
                y = w_up[int(ids[r, k])].double() @ h[r].double()
                act[r * top + k] = (torch.clamp(y, min=0.0) ** 2).to(act.dtype)
        return act

    def activation(self, x, out, kind="relu2"):
        out.copy_((torch.clamp(x.double(), min=0.0) ** 2).to(out.dtype))
        return out

    def stream_concat(self, x, ids, table, scale, out):
        width = x.shape[1]
        out[:, :width] = x.to(out.dtype)
        out[:, width:] = (table[ids.long()].double() * scale).to(out.dtype)
        return out

    def weighted_sum(self, out, x, a, y, b, accumulate=False):
        v = a * x.double() + b * y.double()
        out.copy_(((out.double() + v) if accumulate else v).to(out.dtype))
        return out

    def carry_ids(self, ids, source, previous):
        for r in range(ids.numel()):
            if int(source[r]) >= 0:
                ids[r] = previous[int(source[r])]
        return ids

    def argmax(self, logits, out):
        for r in range(logits.shape[0]):
            row = logits[r].float().cpu().numpy()
            row = np.where(np.isfinite(row), row, -np.inf)
            out[r] = 0 if not np.isfinite(row).any() else plain_llama.greedy(row)
        return out

    def adjust_logits(self, logits, packed, sections, last_tokens=None):
        """The packed lists of `Ops.adjust_logits`, taken apart here and applied with the plain functions."""
        rows, vocab = logits.shape
        seen, bias, blocked, allowed, pairs = (int(n) for n in sections)
        words = packed.cpu().numpy().astype(np.int32)
        at = rows * 14
        lists = []
        for count in (seen, seen, bias, bias, blocked, allowed, pairs, pairs):
            lists.append(words[at:at + count])
            at += count
        seen_ids, seen_counts, bias_ids, bias_values, blocked_ids, allowed_ids, if_last, then_blocked = lists
        bias_values = bias_values.view(np.float32)
        for r in range(rows):
            rec = words[r * 14:(r + 1) * 14]
            rep, pres, freq = (float(v) for v in rec[:3].view(np.float32))
            (seen_off, seen_len, bias_off, bias_len, blocked_off, blocked_len, last_row, allowed_off, allowed_len,
             pairs_off, pairs_len) = (int(v) for v in rec[3:])
            history = []
            for t, n in zip(seen_ids[seen_off:seen_off + seen_len], seen_counts[seen_off:seen_off + seen_len]):
                history += [int(t)] * int(n)
            last = int(last_tokens[last_row]) if last_row >= 0 else -1
            if last_row >= 0:
                history.append(last)
            row = plain_llama.apply_penalties(logits[r].float().cpu().numpy(), history, rep, pres, freq, -1,
                                              list(zip(bias_ids[bias_off:bias_off + bias_len].tolist(),
                                                       bias_values[bias_off:bias_off + bias_len].tolist())))
            row[[int(t) for t in blocked_ids[blocked_off:blocked_off + blocked_len] if 0 <= t < vocab]] = -np.inf
            for a, b in zip(if_last[pairs_off:pairs_off + pairs_len], then_blocked[pairs_off:pairs_off + pairs_len]):
                if int(a) == last and 0 <= b < vocab:
                    row[int(b)] = -np.inf
            if allowed_len:
                row = plain_llama.apply_generation_controls(row, 0, 0, (), (), allowed_ids[allowed_off:allowed_off + allowed_len].tolist())
            logits[r] = torch.from_numpy(row).to(logits.dtype)
        return logits

    def logprobs(self, logits, wanted_rows, tokens, top, values, ids):
        for w, r in enumerate(int(r) for r in wanted_rows):
            got = plain_llama.raw_logprobs(logits[r].float().cpu().numpy(), int(tokens[r]), top)
            ids[w, 0] = int(tokens[r])
            if got is None:
                values[w] = float("nan")
                ids[w, 1:] = torch.tensor([-1] * top, dtype=ids.dtype)
                continue
            values[w, 0] = got[0]
            for k in range(top):
                ids[w, 1 + k] = got[1][k][0] if k < len(got[1]) else -1
                values[w, 1 + k] = got[1][k][1] if k < len(got[1]) else float("nan")

    def logprobs_processed(self, logits, wanted_rows, tokens, params, top, values, ids):
        rec = np.frombuffer(params.cpu().numpy().tobytes(), dtype=np.dtype([("temperature", "<f4"), ("top_p", "<f4"), ("top_k", "<i4"),
                                                                            ("min_p", "<f4"), ("seed", "<u8"), ("draw", "<u8")]))
        for w, r in enumerate(int(r) for r in wanted_rows):
            p = rec[r]
            got = plain_llama.processed_logprobs(logits[r].float().cpu().numpy(), int(tokens[r]), top, float(p["temperature"]),
                                                 int(p["top_k"]), float(p["top_p"]), float(p["min_p"]))
            ids[w, 0] = int(tokens[r])
            if got is None:
                values[w] = float("nan")
                ids[w, 1:] = torch.tensor([-1] * top, dtype=ids.dtype)
                continue
            values[w, 0] = got[0]
            for k in range(top):
                ids[w, 1 + k] = got[1][k][0] if k < len(got[1]) else -1
                values[w, 1 + k] = got[1][k][1] if k < len(got[1]) else float("nan")

    def sample(self, logits, work, params, out, kinds=3):
        raw = params.cpu().numpy().tobytes()
        rec = np.frombuffer(raw, dtype=np.dtype([("temperature", "<f4"), ("top_p", "<f4"), ("top_k", "<i4"),
                                                 ("min_p", "<f4"), ("seed", "<u8"), ("draw", "<u8")]))
        for r in range(logits.shape[0]):
            p = rec[r]
            out[r] = plain_llama.device_sample(logits[r].float().cpu().numpy(), float(p["temperature"]), int(p["top_k"]),
                                               float(p["top_p"]), int(p["seed"]), int(p["draw"]), float(p["min_p"]))
        return out
