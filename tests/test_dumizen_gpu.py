"""Dumizen on the MI355X: each of its kernels alone against tests/reference_ops.py (float64), then the engine's steps however
a request is cut and batched, captured decode steps and greedy generation against tests/plain_dumizen.py."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import dumizen_configs as dc
import plain_dumizen as pd
import trace_tools as tt
from reference_ops import ReferenceOps

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
BF16_EPS = 2.0 ** -8


@pytest.fixture(scope="module")
def ops():
    from fllm_amd.kernels import Ops
    return Ops()


@pytest.fixture(scope="module")
def ref():
    return ReferenceOps()


def gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def close(got, want, rtol, atol, what=""):
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    err = (got - want).abs()
    worst = (err - (atol + rtol * want.abs())).max().item()
    assert worst <= 0, f"{what}: max err {err.max().item():.3e} (|want| max {want.abs().max().item():.3e}), over by {worst:.3e}"


class Scene:
    """Requests that hold `held` tokens in shuffled pages and bring `new` rows each; tensors on the CPU in float32."""

    def __init__(self, segments, G, d, dv, page, seed, pool=0):
        g = gen(seed)
        self.segments, self.page = segments, page
        self.key_chunk = 8 if d % 8 == 0 else 1
        pages_each = [-(-(held + new) // page) for held, new in segments]
        total = sum(pages_each) + 3
        order = torch.randperm(total - 1, generator=g) + 1            # page 0 stays unused: a wrong lookup shows
        self.tables = torch.full((len(segments), max(pages_each)), -1, dtype=torch.int32)
        at = 0
        for s, n in enumerate(pages_each):
            self.tables[s, :n] = order[at:at + n].to(torch.int32)
            at += n
        self.k_pages = torch.randn(total, G, d // self.key_chunk, page, self.key_chunk, generator=g)
        self.v_pages = torch.randn(total, G, dv, page, generator=g)
        slots = -(-page // pool) if pool else 1
        self.pool_k = torch.full((total, G, slots, d), 7.0)             # whatever an earlier request left
        self.pool_v = torch.full((total, G, slots, dv), -7.0)
        pos, seg, start = [], [], [0]
        for s, (held, new) in enumerate(segments):
            pos += list(range(held, held + new))
            seg += [s] * new
            start.append(start[-1] + new)
        self.row_pos, self.row_seg = torch.tensor(pos, dtype=torch.int32), torch.tensor(seg, dtype=torch.int32)
        self.seg_start = torch.tensor(start, dtype=torch.int32)
        self.rows = len(pos)
        self.max_pos = max(h + n for h, n in segments)

    def to(self, device, dtype):
        move = lambda t: t.to(device=device, dtype=dtype if t.is_floating_point() else t.dtype).contiguous()
        out = {k: move(getattr(self, k)) for k in ("tables", "k_pages", "v_pages", "row_pos", "row_seg", "seg_start")}
        out["pool_k"], out["pool_v"] = self.pool_k.to(device).clone(), self.pool_v.to(device).clone()
        if dtype == torch.float64:
            out["pool_k"], out["pool_v"] = out["pool_k"].double(), out["pool_v"].double()
        return out


SEGMENTS = [(0, 9), (37, 1), (100, 30), (61, 3), (250, 1), (300, 70)]
SINGLE_ROWS = [(0, 1), (37, 1), (100, 1), (63, 1), (250, 1), (64, 1), (1000, 1)]


# ---------------------------------------------------------------------------------------------
# norm, rotation and store
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mode,from_keys", [(0, False), (1, False), (2, False), (2, True), (1, True)])
@pytest.mark.parametrize("H,G,d,dv,rope", [(4, 2, 32, 16, 16), (3, 1, 12, 10, 6), (8, 4, 64, 64, 64), (2, 2, 24, 24, 0)])
def test_queries_and_keys_normed_rotated_and_stored(ops, ref, H, G, d, dv, rope, mode, from_keys, dtype):
    if from_keys:
        dv = d
    sc = Scene(SEGMENTS, G, d, dv, 16, seed=H * 10 + d)
    g = gen(5)
    width = H * d + G * d + (0 if from_keys else G * dv) + 8
    qkv = torch.randn(sc.rows, width, generator=g).to(dtype).float()
    qw = 1 + 0.4 * torch.rand(H * d if mode == 2 else d, generator=g)
    kw = 1 + 0.4 * torch.rand(G * d if mode == 2 else d, generator=g)
    cos, sin = torch.rand(400, rope // 2, generator=g) * 2 - 1, torch.rand(400, rope // 2, generator=g) * 2 - 1
    results = []
    for o, dev, kind in ((ref, "cpu", torch.float64), (ops, DEV, dtype)):
        t = sc.to(dev, kind)
        q_out = torch.zeros(sc.rows, H * d, dtype=kind, device=dev)
        o.normed_rope_store(qkv.to(dev, kind), mode, qw.to(dev), kw.to(dev), 1e-5, q_out, t["row_pos"], t["row_seg"], t["tables"],
                            cos.to(dev), sin.to(dev), t["k_pages"], t["v_pages"], H, G, d, dv, rope, 16, sc.key_chunk,
                            values_from_keys=from_keys)
        results.append((q_out, t["k_pages"], t["v_pages"]))
    tol = (1e-5, 1e-5) if dtype == torch.float32 else (BF16_EPS, 1e-3)
    close(results[1][0], results[0][0], *tol, "queries")
    close(results[1][1], results[0][1], *tol, "stored keys")
    assert torch.equal(results[1][2].double().cpu(), results[0][2].to(dtype).double()), "stored values"


# ---------------------------------------------------------------------------------------------
# blocks behind a window
# ---------------------------------------------------------------------------------------------
def pooled_attend(o, t, q, sc, H, G, d, dv, scale, window, pool, kind):
    o.pool_blocks(t["k_pages"], t["v_pages"], t["pool_k"], t["pool_v"], t["tables"], t["row_pos"], t["row_seg"], G, d, dv, sc.page,
                  sc.key_chunk, pool)
    out = torch.empty(sc.rows, H * dv, dtype=kind, device=q.device)
    o.pooled_window_attention(q, t["k_pages"], t["v_pages"], t["pool_k"], t["pool_v"], t["tables"], t["row_pos"], t["row_seg"],
                              t["seg_start"], out, H, G, d, dv, sc.page, scale, window, pool, sc.key_chunk, max_context=sc.max_pos)
    return out


def fill_pools(ref, sc, t, G, d, dv, pool):
    """The means of every block that the requests hold before the step, as earlier steps would have left them."""
    for s, (held, _) in enumerate(sc.segments):
        ends = [p for p in range(held) if (p + 1) % pool == 0]
        if ends:
            ref.pool_blocks(t["k_pages"], t["v_pages"], t["pool_k"], t["pool_v"], t["tables"], torch.tensor(ends, dtype=torch.int32),
                            torch.full((len(ends),), s, dtype=torch.int32), G, d, dv, sc.page, sc.key_chunk, pool)


@pytest.mark.parametrize("rows", ["mixed", "single"])
@pytest.mark.parametrize("fast", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv,page,window,pool", [(4, 1, 32, 16, 8, 12, 4), (3, 3, 32, 32, 16, 5, 1), (3, 1, 12, 10, 16, 7, 3),
                                                         (8, 2, 64, 32, 16, 40, 8), (2, 1, 128, 300, 32, 33, 16), (12, 2, 128, 128, 16, 100, 8),
                                                         (9, 3, 96, 64, 32, 50, 4)])
def test_windows_with_pooled_blocks_over_pages(ops, ref, H, G, d, dv, page, window, pool, dtype, fast, rows):
    """`fast` False: the plain kernel also where the matrix-core kernel would serve (bfloat16, heads of 32 to 128 lanes in
    steps of 32, pages of multiples of 16); "single": a step of one row a request, whose tiles are the heads of a key/value head."""
    if dtype == torch.float32 and not fast:
        pytest.skip("float32 has one kernel")
    sc = Scene(SINGLE_ROWS if rows == "single" else SEGMENTS, G, d, dv, page, seed=d + window, pool=pool)
    q = torch.randn(sc.rows, H * d, generator=gen(3)).to(dtype).float()
    want_t = sc.to("cpu", torch.float64)
    want_t["k_pages"], want_t["v_pages"] = want_t["k_pages"].to(dtype).double(), want_t["v_pages"].to(dtype).double()
    fill_pools(ref, sc, want_t, G, d, dv, pool)
    got_t = sc.to(DEV, dtype)
    got_t["pool_k"], got_t["pool_v"] = want_t["pool_k"].float().to(DEV), want_t["pool_v"].float().to(DEV)
    want = pooled_attend(ref, want_t, q.double(), sc, H, G, d, dv, 0.3, window, pool, torch.float64)
    ops.set_fast_kernels(fast)
    try:
        got = pooled_attend(ops, got_t, q.to(DEV, dtype), sc, H, G, d, dv, 0.3, window, pool, dtype)
        torch.cuda.synchronize()
    finally:
        ops.set_fast_kernels(True)
    close(got_t["pool_k"], want_t["pool_k"], 1e-6, 1e-6, "means of keys")
    close(got_t["pool_v"], want_t["pool_v"], 1e-6, 1e-6, "means of values")
    close(got, want, *((2e-5, 2e-5) if dtype == torch.float32 else (2 * BF16_EPS, 5e-3)), "attention")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("held", [63, 500])
@pytest.mark.parametrize("where", ["first of the window", "just left the window", "last of the newest block", "first block", "itself"])
def test_one_key_that_stands_out_at_the_edges(ops, ref, where, held, dtype):
    """Window 24, blocks of 8, pages of 16; one query at position `held`.  One position's key points along the query and its
    value is marked: inside the window it takes all the weight; in a block behind it, the block's mean does (an eighth of
    the mark); just outside the window in a block that is not complete behind it, nothing of it arrives."""
    H, G, d, dv, page, window, pool = 2, 1, 32, 16, 16, 24, 8
    sc = Scene([(held, 1)], G, d, dv, page, seed=held, pool=pool)
    lo = held - window + 1
    blocks = lo // pool
    at = {"first of the window": lo, "just left the window": lo - 1, "last of the newest block": blocks * pool - 1,
          "first block": 0, "itself": held}[where]
    t = sc.to("cpu", torch.float64)
    t["k_pages"] *= 0.05
    page_of, off = int(t["tables"][0, at // page]), at % page
    t["k_pages"][page_of, 0, :, off, :] = 3.0
    t["v_pages"][page_of, 0, :, off] = 1000.0
    q = torch.ones(1, H * d, dtype=torch.float64)
    fill_pools(ref, sc, t, G, d, dv, pool)
    got_t = {k: (v.to(DEV, dtype) if v.is_floating_point() and not k.startswith("pool") else v.to(DEV)) for k, v in t.items()}
    got_t["pool_k"], got_t["pool_v"] = t["pool_k"].float().to(DEV), t["pool_v"].float().to(DEV)
    got = pooled_attend(ops, got_t, q.to(DEV, dtype), sc, H, G, d, dv, 1.0, window, pool, dtype).float().cpu()
    want = pooled_attend(ref, t, q, sc, H, G, d, dv, 1.0, window, pool, torch.float64)
    close(got, want, 2e-2, 2.0, where)
    seen_as_token, in_block = at >= lo, at < blocks * pool
    expect = 1000.0 if seen_as_token else (125.0 if in_block else 0.0)
    assert abs(float(want[0, 0]) - expect) < 30.0 and abs(float(got[0, 0]) - expect) < 30.0, (where, float(want[0, 0]), float(got[0, 0]))


# ---------------------------------------------------------------------------------------------
# sigmoid weights
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("rows", ["mixed", "single"])
@pytest.mark.parametrize("fast", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv,page", [(4, 2, 16, 24, 8), (3, 3, 32, 32, 16), (3, 1, 12, 20, 16), (4, 2, 64, 64, 16), (2, 1, 96, 300, 32),
                                           (12, 2, 128, 128, 16), (6, 3, 96, 96, 32)])
def test_sigmoid_attention_over_pages(ops, ref, H, G, d, dv, page, dtype, fast, rows):
    if dtype == torch.float32 and not fast:
        pytest.skip("float32 has one kernel")
    sc = Scene(SINGLE_ROWS if rows == "single" else SEGMENTS, G, d, dv, page, seed=d + dv)
    g = gen(4)
    q = torch.randn(sc.rows, H * d + 16, generator=g).to(dtype).float()
    r1, r2, pb = torch.rand(H, generator=g) + 0.2, torch.rand(H, generator=g) * 0.5 + 0.05, torch.randn(H, generator=g) - 1.0
    outs = []
    for o, dev, kind in ((ref, "cpu", torch.float64), (ops, DEV, dtype)):
        t = sc.to(dev, kind)
        if kind == torch.float64:
            t["k_pages"], t["v_pages"] = t["k_pages"].to(dtype).double(), t["v_pages"].to(dtype).double()
        out = torch.empty(sc.rows, H * dv, dtype=kind, device=dev)
        if o is ops:
            ops.set_fast_kernels(fast)
        try:
            o.sigmoid_attention(q.to(dev, kind)[:, :H * d], t["k_pages"], t["v_pages"], t["tables"], t["row_pos"], t["row_seg"], t["seg_start"],
                                out, H, G, d, dv, page, 0.2, 4.0, r1.to(dev), r2.to(dev), pb.to(dev), 0.4, 8, sc.key_chunk, max_context=sc.max_pos)
            if o is ops:
                torch.cuda.synchronize()
        finally:
            if o is ops:
                ops.set_fast_kernels(True)
        outs.append(out)
    scale = outs[0].abs().max().item()
    close(outs[1], outs[0], *((2e-5, 2e-5 * scale) if dtype == torch.float32 else (2 * BF16_EPS, 4e-3 * scale)), "sigmoid attention")


def test_a_far_key_weighs_by_its_distance_and_the_temperature_steps(ops, ref):
    """One query at position 700 over keys that all point along it: the weight of key j is a function of 700 - j alone, and
    the temperature has stepped floor(701 / 128) times."""
    H, G, d, dv, page = 1, 1, 32, 16, 16
    sc = Scene([(700, 1)], G, d, dv, page, seed=1)
    t = sc.to(DEV, torch.float32)
    t["k_pages"][:] = 0.1
    t["v_pages"][:] = 0.0
    far = 3
    t["v_pages"][int(sc.tables[0, far // page]), 0, :, far % page] = 1.0
    q = torch.full((1, d), 0.5, device=DEV)
    r1, r2, pb = (torch.tensor([v], device=DEV) for v in (0.7, 0.3, 0.5))
    out = torch.empty(1, dv, device=DEV)
    ops.sigmoid_attention(q, t["k_pages"], t["v_pages"], t["tables"], t["row_pos"], t["row_seg"], t["seg_start"], out, H, G, d, dv, page,
                          1.0, 2.0, r1, r2, pb, 0.3, 128, sc.key_chunk)
    temp = 1 + 0.3 * np.log(701 // 128 + 1)
    s = 2.0 * np.tanh(32 * 0.05 * temp / 2.0) - 0.7 * np.log(1 + 0.3 * (700 - far)) + 0.5
    assert abs(out[0, 0].item() - 1 / (1 + np.exp(-s))) < 1e-6


# ---------------------------------------------------------------------------------------------
# what retention takes from the shared kernels
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,vdim,rope", [(2, 16, 24, 8), (3, 10, 6, 10), (4, 64, 64, 64), (1, 32, 32, 0)])
def test_operands_rotated_and_scaled_in_float32(ops, ref, heads, dim, vdim, rope, dtype):
    g = gen(7)
    rows = 21
    qkvg = torch.randn(rows, heads * (2 * dim + 2 * vdim), generator=g).to(dtype)
    pos = torch.randint(0, 200, (rows,), generator=g, dtype=torch.int32)
    cos, sin = torch.rand(200, rope // 2, generator=g) * 2 - 1, torch.rand(200, rope // 2, generator=g) * 2 - 1
    want = torch.empty(rows, heads * (2 * dim + vdim), dtype=torch.float64)
    ref.rotate_scale(qkvg.double(), want, pos, cos, sin, heads, dim, vdim, rope, dim ** -0.5)
    got = torch.empty(rows, heads * (2 * dim + vdim), dtype=torch.float32, device=DEV)
    ops.rotate_scale(qkvg.to(DEV), got, pos.to(DEV), cos.to(DEV), sin.to(DEV), heads, dim, vdim, rope, dim ** -0.5)
    close(got, want, 1e-6, 1e-6, "operands")          # float32 whatever the rows' type: nothing is rounded behind the projection


@pytest.mark.parametrize("x_dtype,out_dtype", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16), (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("activation", ["silu", "sigmoid"])
@pytest.mark.parametrize("rows,width,group", [(1, 48, 24), (7, 60, 6), (33, 256, 64), (70, 1536, 128), (3, 600, 300)])
def test_every_head_normed_alone_and_gated(ops, ref, rows, width, group, activation, x_dtype, out_dtype):
    g = gen(9)
    x = (torch.randn(rows, width, generator=g) * 3).to(x_dtype)
    gate = torch.randn(rows, width + 40, generator=g).to(out_dtype)
    want = torch.empty(rows, width, dtype=torch.float64)
    ref.group_norm_gate(x.double(), 1e-5, group, gate.double()[:, 8:8 + width], want, activation=activation)
    got = torch.empty(rows, width, dtype=out_dtype, device=DEV)
    ops.group_norm_gate(x.to(DEV), 1e-5, group, gate.to(DEV)[:, 8:8 + width], got, activation=activation)
    close(got, want, *((1e-5, 1e-5) if out_dtype == torch.float32 else (BF16_EPS, 1e-3)), "normed heads")


# ---------------------------------------------------------------------------------------------
# router with corrections and groups; experts without a gate; small passes
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width,experts,top,groups,kept", [(1, 64, 6, 2, 3, 2), (9, 68, 4, 2, 4, 2), (40, 320, 8, 4, 2, 1), (200, 1024, 64, 6, 8, 3),
                                                                (3, 50, 130, 4, 1, 1), (5, 96, 3, 3, 1, 1), (17, 128, 256, 8, 128, 40)])
def test_the_router_with_corrections_and_groups(ops, ref, rows, width, experts, top, groups, kept, dtype):
    g = gen(rows + experts)
    h = torch.randn(rows, width, generator=g).to(dtype)
    w = (torch.randn(experts, width, generator=g) * 1.5 * width ** -0.5).to(dtype)
    correction = torch.randn(experts, generator=g) * 0.3
    ids_w, wts_w = torch.empty(rows, top, dtype=torch.int32), torch.empty(rows, top)
    ref.route_grouped(h.double(), w.double(), correction, top, groups, kept, ids_w, wts_w, route_scale=2.5)
    ids, wts = torch.empty(rows, top, dtype=torch.int32, device=DEV), torch.empty(rows, top, device=DEV)
    ops.route_grouped(h.to(DEV), w.to(DEV), correction.to(DEV), top, groups, kept, ids, wts, route_scale=2.5)
    same = (ids.cpu() == ids_w).all(dim=1)
    assert same.float().mean() >= (0.97 if rows >= 40 else 1.0), "picks differ on more than close calls"
    close(wts.cpu()[same], wts_w[same], 1e-4, 1e-5, "weights")
    assert torch.allclose(wts.sum(1).cpu(), torch.full((rows,), 2.5), atol=1e-4)
    per = experts // groups
    assert all(len({int(e) // per for e in row}) <= kept for row in ids.cpu())


def test_equal_choices_go_to_the_lower_index_and_negative_groups_count_as_they_are(ops):
    h = torch.zeros(1, 8, device=DEV)
    h[0, 0] = 1.0
    w = torch.zeros(6, 8, device=DEV)
    ids, wts = torch.empty(1, 2, dtype=torch.int32, device=DEV), torch.empty(1, 2, device=DEV)
    ops.route_grouped(h, w, torch.zeros(6, device=DEV), 2, 3, 1, ids, wts)               # all equal: group 0, experts 0 and 1
    assert ids.cpu().tolist() == [[0, 1]] and torch.allclose(wts.cpu(), torch.full((1, 2), 0.5))
    correction = torch.tensor([0.0, 0.0, 0.1, 0.0, 2.0, -9.0], device=DEV)
    ops.route_grouped(h, w, correction, 2, 3, 1, ids, wts)       # group 2 sums 2.5 - 8.5: a negative choice is no zero
    assert ids.cpu().tolist() == [[2, 3]]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width,inter,experts,top", [(1, 64, 24, 6, 2), (9, 68, 18, 4, 2), (40, 320, 96, 8, 4), (70, 256, 130, 3, 3)])
def test_experts_without_a_gate(ops, ref, rows, width, inter, experts, top, dtype):
    g = gen(rows * 3 + inter)
    h = torch.randn(rows, width, generator=g).to(dtype)
    w_up = (torch.randn(experts, inter, width, generator=g) * 2 * width ** -0.5).to(dtype)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(rows)]).to(torch.int32)
    want = torch.empty(rows * top, inter, dtype=torch.float64)
    ref.experts_up(h.double(), ids, w_up.double(), want)
    got = torch.empty(rows * top, inter, dtype=dtype, device=DEV)
    ops.experts_up(h.to(DEV), ids.to(DEV), w_up.to(DEV), got)
    close(got, want, *((1e-5, 1e-5) if dtype == torch.float32 else (BF16_EPS, 1e-3)), "activations")
    assert (want == 0).float().mean() > 0.2          # the negative half is cut off


@pytest.mark.parametrize("spread", ["random", "one expert"])
@pytest.mark.parametrize("rows,width,inter,experts,top", [(17, 64, 24, 6, 2), (70, 136, 40, 4, 2), (300, 320, 96, 8, 4), (1000, 256, 136, 16, 3),
                                                          (4, 128, 64, 2, 2)])
def test_experts_without_a_gate_grouped_on_the_matrix_cores(ops, ref, rows, width, inter, experts, top, spread):
    g = gen(rows + inter)
    h = torch.randn(rows, width, generator=g).to(torch.bfloat16)
    w_up = (torch.randn(experts, inter, width, generator=g) * 2 * width ** -0.5).to(torch.bfloat16)
    w_down = (torch.randn(experts, width, inter, generator=g) * inter ** -0.5).to(torch.bfloat16)
    if spread == "random":
        ids = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(rows)]).to(torch.int32)
    else:
        ids = torch.arange(top, dtype=torch.int32).repeat(rows, 1)
    act = torch.empty(rows * top, inter, dtype=torch.float64)
    ref.experts_up(h.double(), ids, w_up.double(), act)
    want = torch.empty(rows * top, width, dtype=torch.float64)
    ref.experts_down(act.to(torch.bfloat16).double(), ids, w_down.double(), want)
    got = torch.full((rows * top, width), float("nan"), device=DEV)
    assert ops.experts_grouped_ungated(h.to(DEV), ids.to(DEV), w_up.to(DEV), w_down.to(DEV), got)
    close(got, want, 2 * BF16_EPS, 2e-2 * want.abs().max().item(), "grouped experts")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_small_passes(ops, ref, dtype):
    g = gen(2)
    rows, width, vocab = 13, 200, 50
    x, y = torch.randn(rows, width, generator=g), torch.randn(rows, width, generator=g)
    out = torch.randn(rows, width, generator=g)
    want = out.double() + 0.8 * x.double() + 1.1 * y.double()
    got = out.to(DEV)
    ops.weighted_sum(got, x.to(DEV), 0.8, y.to(DEV), 1.1, accumulate=True)
    close(got, want, 1e-6, 1e-6, "sum into the stream")
    ops.weighted_sum(got, x.to(DEV), 0.5, y.to(DEV), -2.0)
    close(got, 0.5 * x.double() - 2.0 * y.double(), 1e-6, 1e-6, "sum")
    table = torch.randn(vocab, width, generator=g).to(dtype)
    ids = torch.randint(0, vocab, (rows,), generator=g, dtype=torch.int32)
    both = torch.empty(rows, 2 * width, dtype=dtype, device=DEV)
    ops.stream_concat(x.to(DEV), ids.to(DEV), table.to(DEV), 1.0, both)
    assert torch.equal(both.cpu()[:, :width], x.to(dtype)) and torch.equal(both.cpu()[:, width:], table[ids.long()])
    z = torch.randn(rows, width, generator=g).to(dtype)
    act = z.to(DEV)
    ops.activation(act, act, "relu2")
    close(act, torch.clamp(z.double(), min=0) ** 2, *((1e-6, 1e-6) if dtype == torch.float32 else (BF16_EPS, 1e-6)), "activation")


def test_a_sink_behind_parts_of_a_long_row_tile(ops, ref):
    """A portion of a prompt over a long context, whose row tiles' keys several workgroups share: the sink's term joins the
    denominator once, against the maximum of all parts."""
    H, G, d, page = 8, 4, 64, 16
    sc = Scene([(1000, 64)], G, d, d, page, seed=12)
    q = (torch.randn(sc.rows, H * d, generator=gen(1)) * 0.5).to(torch.bfloat16)
    sinks = torch.zeros(H)
    want_t = sc.to("cpu", torch.float64)
    want_t["k_pages"], want_t["v_pages"] = want_t["k_pages"].to(torch.bfloat16).double(), want_t["v_pages"].to(torch.bfloat16).double()
    want = torch.empty(sc.rows, H * d, dtype=torch.float64)
    ref.attention(q.double(), want_t["k_pages"], want_t["v_pages"], want_t["tables"], want_t["row_pos"], want_t["row_seg"], want_t["seg_start"],
                  want, H, G, d, page, 0.125, None, sc.max_pos, sinks=sinks)
    t = sc.to(DEV, torch.bfloat16)
    got = torch.empty(sc.rows, H * d, dtype=torch.bfloat16, device=DEV)
    need = ops.attention_workspace_bytes(sc.rows, H, G, d, sc.max_pos)
    ops.attention(q.to(DEV), t["k_pages"], t["v_pages"], t["tables"], t["row_pos"], t["row_seg"], t["seg_start"], got, H, G, d, page, 0.125,
                  None, sc.max_pos, single_from=1, workspace=torch.empty(max(need, 1), dtype=torch.uint8, device=DEV), sinks=sinks.to(DEV))
    close(got, want, 3 * BF16_EPS, 2e-2, "attention with a sink")


# ---------------------------------------------------------------------------------------------
# the engine
# ---------------------------------------------------------------------------------------------
LENGTHS = {"A": [5, 30, 61, 120], "B": [45, 83, 2], "C": [9, 50, 77], "D": [100, 37, 260]}
TOL = {"float32": 2e-5, "bfloat16": 6e-2}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """(configuration, precision) -> folder, configuration, requests, plain logits, weights.  float32 runs random routers;
    bfloat16 runs routers whose every pick has a margin, since a pick that flips under rounding is a large error that says
    nothing about the kernels."""
    out = {}
    for name, cfg in dc.CONFIGS.items():
        for dtype in ("float32", "bfloat16"):
            tensors = dc.weights(cfg, 30 + ord(name), decided_router=dtype == "bfloat16")
            folder = dc.write_model(str(tmp_path_factory.mktemp(f"dumizen_{name}_{dtype}")), cfg, tensors)
            requests = {f"r{i}": dc.random_ids(n, cfg["vocab"], 100 * ord(name) + i) for i, n in enumerate(LENGTHS[name])}
            w64 = dc.to_float64(tensors)
            plain = {rid: pd.forward(cfg, w64, toks) for rid, toks in requests.items()}
            out[name, dtype] = (folder, cfg, requests, plain, w64)
    return out


def make_runner(folder, dtype, page_size, max_tokens, **kw):
    from fllm_amd.engine import ModelRunner
    return ModelRunner.from_folder(folder, dtype=dtype, page_size=page_size, max_tokens=max_tokens, max_requests=4, **kw)


def check(got, plain, dtype, what):
    for rid, want in plain.items():
        assert rid in got and got[rid].shape == want.shape, f"{what}: request {rid}"
        err = np.abs(got[rid].astype(np.float64) - want)
        scale = np.abs(want).max()
        tt.observe(f"dumizen {what.split()[0]} {dtype}", err.max() / scale)
        over = err.max(axis=1) > TOL[dtype] * scale
        assert not over.any(), (f"{what}: request {rid}: max error {err.max():.3e} (limit {TOL[dtype] * scale:.3e}); first "
                                f"position over the limit: {int(np.argmax(over))}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("family", ["whole", "last40", "portions", "mixed"])
def test_replay(models, tmp_path, name, dtype, family):
    folder, cfg, requests, plain, _ = models[name, dtype]
    refed = [rid for rid, toks in requests.items() if len(toks) >= 60][:1]
    steps = {"whole": tt.whole, "last40": lambda r: tt.last_tokens_one_by_one(r, 40), "portions": tt.portions,
             "mixed": lambda r: tt.mixed(r, seed=5, refeed=refed)}[family](requests)
    steps = tt.number(steps)
    runner = make_runner(folder, dtype, dc.PAGE_SIZES[name], tt.live_tokens_bound(steps))
    handed_out = tt.record_allocations(runner.cache)
    got = tt.run_in_process(runner, steps, cfg["vocab"], str(tmp_path))
    check(got, plain, dtype, f"{family} {name} {dtype}")
    runner.cache.check_invariants()
    assert all(pool.available == pool.num_pages for pool in runner.cache.pools), "pages were lost"
    if family == "mixed":
        assert all(len(pages) > len(set(pages)) for pages in handed_out), "the trace was meant to use pages again"


@pytest.mark.parametrize("page_size", [4, 32, 64])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_at_other_page_sizes(models, tmp_path, page_size, dtype):
    # C in float32: blocks of three straddle pages of every size, and the tolerance is tight enough to show one lost block.  In
    # bfloat16 C, whose three layers run three times each, rounds up to a twelfth of its largest logit at single positions
    # however it is cut; A takes its place there.
    name = "C" if dtype == "float32" else "A"
    folder, cfg, requests, plain, _ = models[name, dtype]
    steps = tt.number(tt.mixed(requests, seed=8))
    runner = make_runner(folder, dtype, page_size, tt.live_tokens_bound(steps, round_to=max(64, page_size)))
    got = tt.run_in_process(runner, steps, cfg["vocab"], str(tmp_path))
    check(got, plain, dtype, f"pages-of-{page_size} {name} {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_first_tokens_and_long_decoding(models, tmp_path, name, dtype):
    """Token by token from the very first token, across windows, blocks and temperature steps."""
    folder, cfg, requests, plain, _ = models[name, dtype]
    rid = max(requests, key=lambda r: len(requests[r]))
    one = {rid: requests[rid]}
    steps = tt.number(tt.last_tokens_one_by_one(one, tail=len(requests[rid])))
    runner = make_runner(folder, dtype, dc.PAGE_SIZES[name], 320)
    got = tt.run_in_process(runner, steps, cfg["vocab"], str(tmp_path))
    check(got, {rid: plain[rid]}, dtype, f"token-by-token {name} {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C", "D"])
def test_decode_graphs_and_eager_steps_agree(models, tmp_path, name, dtype):
    folder, cfg, requests, plain, _ = models[name, dtype]
    steps = tt.number(tt.last_tokens_one_by_one(requests) + tt.mixed(requests, seed=21, decode_tail=40))
    results = []
    for i, use_graphs in enumerate((True, False)):
        runner = make_runner(folder, dtype, dc.PAGE_SIZES[name], tt.live_tokens_bound(steps), use_graphs=use_graphs)
        results.append(tt.run_in_process(runner, steps, cfg["vocab"], str(tmp_path / str(i))))
        assert (runner.graph_replays > 30) == use_graphs
    for rid, want in plain.items():
        a, b = results[0][rid].astype(np.float64), results[1][rid].astype(np.float64)
        if dtype == "float32":
            assert np.array_equal(a, b), f"{rid}: graph and eager steps differ in float32"
        else:
            assert np.abs(a - b).max() <= TOL[dtype] * np.abs(want).max()
    check(results[0], plain, dtype, f"graphs {name} {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_whole_and_in_portions(models, tmp_path, dtype):
    """1,100 tokens in one step, in two portions, and with the last 40 decoded one by one: keys a thousand positions back, a
    retention state carried over a thousand tokens, more than a hundred blocks behind the window."""
    folder, cfg, _, _, w64 = models["D", dtype]
    toks = dc.random_ids(1100, cfg["vocab"], 77)
    want = {"long": pd.forward(cfg, w64, toks)}
    from fllm_amd.engine import StepEntry
    for cuts in ([1100], [600, 500], [1060] + [1] * 40):
        runner = make_runner(folder, dtype, 16, 1152, max_context=2048)
        got, at = [], 0
        for n in cuts:
            got.append(runner.step([StepEntry("long", toks[at:at + n], list(range(n)))]).float().cpu().numpy())
            at += n
        check({"long": np.concatenate(got)}, want, dtype, f"long-prompt-{len(cuts)} D {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(models, tmp_path, dtype):
    folder, cfg, requests, plain, _ = models["A", dtype]
    steps = tt.number(tt.mixed(requests, seed=9))
    got = tt.run_subprocess(folder, dtype, steps, cfg["vocab"], str(tmp_path), tt.live_tokens_bound(steps))
    check(got, plain, dtype, f"trace_run A {dtype}")


def test_the_residual_stream_after_every_layer_run(models):
    folder, cfg, requests, plain, w64 = models["A", "float32"]
    runner = make_runner(folder, "float32", 8, 320)
    from fllm_amd.engine import StepEntry
    seen = []
    for block in runner.model.blocks:
        def wrapped(ctx, x, binding, _inner=block.forward):
            _inner(ctx, x, binding)
            seen.append(x.clone().cpu().numpy())
        block.forward = wrapped
    toks = requests["r2"]
    runner.step([StepEntry("a", toks, [])])
    want, _ = pd.layer_outputs(cfg, w64, toks)
    assert len(seen) == len(want) == 6
    for got, ref_x in zip(seen, want):
        assert np.abs(got - ref_x).max() <= 1e-5 * np.abs(ref_x).max()


def test_decode_steps_take_the_fused_forms_and_prompts_the_tile_kernels(models, monkeypatch):
    """D in bfloat16 (4 layer runs: sigmoid, windowed twice, a pair): a decode step reads the stream through a layer's first
    norm inside the first product of every mixer (a pair's two sides each), so no norm kernel of its own runs but the model's
    last; a prompt runs the norm, and its experts go to the matrix cores grouped by expert."""
    from fllm_amd.engine import StepEntry
    from fllm_amd.kernels import Ops
    folder, cfg, requests, _, _ = models["D", "bfloat16"]
    runner = make_runner(folder, "bfloat16", 16, 256, use_graphs=False)
    calls = []
    for name in ("rmsnorm", "norm_linear", "normed_rope_store", "pool_blocks", "pooled_window_attention", "sigmoid_attention",
                 "rotate_scale", "linear_attention", "group_norm_gate", "weighted_sum", "route_grouped", "experts_grouped_ungated",
                 "experts_up", "postnorm_add", "stream_concat"):
        inner = getattr(Ops, name)
        monkeypatch.setattr(Ops, name, lambda self, *a, _n=name, _i=inner, **k: (calls.append(_n), _i(self, *a, **k))[1])
    toks = requests["r0"]
    runner.step([StepEntry("a", toks[:40], [])])
    assert calls.count("rmsnorm") == 4 and calls.count("norm_linear") == 0 and calls.count("experts_up") == 0
    assert calls.count("experts_grouped_ungated") == 4 and calls.count("stream_concat") == 2
    calls.clear()
    runner.step([StepEntry("a", toks[40:41], [0])])
    assert calls.count("norm_linear") == 5 and calls.count("rmsnorm") == 1          # the pair's two sides; the model's last norm
    assert calls.count("normed_rope_store") == 3 and calls.count("pool_blocks") == 2 and calls.count("pooled_window_attention") == 2
    assert calls.count("sigmoid_attention") == 1 and calls.count("rotate_scale") == calls.count("linear_attention") == 1
    assert calls.count("group_norm_gate") == calls.count("weighted_sum") == 1
    assert calls.count("route_grouped") == 4 and calls.count("postnorm_add") == 12   # a layer run: norm 1b, the picks' sum, norm 2b


@pytest.mark.parametrize("name", ["A", "D"])
def test_greedy_generation_through_the_scheduler(models, name):
    from fllm_amd import Engine, SamplingParams
    folder, cfg, _, _, w64 = models[name, "float32"]
    prompts = [dc.random_ids(n, cfg["vocab"], 20 + n) for n in (3, 26, 41, 90)]
    want = []
    for p in prompts:
        toks = list(p)
        for _ in range(10):
            toks.append(int(np.argmax(pd.forward(cfg, w64, toks)[-1])))
        want.append(toks[len(p):])
    for opts in (dict(num_blocks=64), dict(num_blocks=14, max_batched_tokens=16)):
        engine = Engine(folder, dtype="float32", ctx=256, max_seqs=3, block_size=dc.PAGE_SIZES[name],
                        **{"max_batched_tokens": 64, **opts})
        assert engine.generate(prompts, SamplingParams(max_tokens=10)) == want
        engine.runner.cache.check_invariants()
    folder, cfg, _, _, w64 = models[name, "bfloat16"]
    engine = Engine(folder, dtype="bfloat16", ctx=256, max_seqs=4, block_size=dc.PAGE_SIZES[name])
    out = engine.generate(prompts, SamplingParams(max_tokens=10))
    assert [len(o) for o in out] == [10] * 4


def test_the_command_line_generates(models):
    folder, cfg, _, _, w64 = models["A", "float32"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prompt = dc.random_ids(30, cfg["vocab"], 4)
    cmd = [sys.executable, "-m", "fllm_amd", "run", folder, "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "8",
           "--dtype", "float32", "--ctx", "256", "--kv-blocks", "32", "--max-seqs", "2"]
    proc = subprocess.run(cmd, cwd=root, capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr[-2000:]
    record = json.loads(proc.stdout.strip().splitlines()[0])
    toks = list(prompt)
    for _ in range(8):
        toks.append(int(np.argmax(pd.forward(cfg, w64, toks)[-1])))
    assert record["finish_reason"] == "length" and record["token_ids"] == toks[30:]
    proc = subprocess.run([sys.executable, "-m", "fllm_amd", "inspect", folder], cwd=root, capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0 and "architecture: dumizen" in proc.stdout
