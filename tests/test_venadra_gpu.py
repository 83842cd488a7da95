"""Venadra on the MI355X: each of its kernels alone against tests/reference_ops.py (float64), then the engine's steps however
a request is cut and batched, captured decode steps and greedy generation against tests/plain_venadra.py."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_venadra as pv
import trace_tools as tt
import venadra_configs as vc
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


def rows_of(segments):
    """(rows a segment) -> row_seg, seg_start; a segment of -n rows is n rows of padding."""
    seg, start = [], [0]
    for s, n in enumerate(segments):
        seg += [s if n > 0 else -1] * abs(n)
        start.append(start[-1] + abs(n))
    return torch.tensor(seg, dtype=torch.int32), torch.tensor(start, dtype=torch.int32)


# ---------------------------------------------------------------------------------------------
# the convolution in front of a mixer
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,taps", [(64, 4), (203, 2), (48, 1), (1024, 5), (136, 7)])
@pytest.mark.parametrize("segments", [[9], [1, 1, 1], [2, 30, 1, 5], [3, -4, 6], [1, 2]])
def test_short_convolution_over_steps(ops, ref, segments, width, taps, dtype):
    """Two steps one after the other: the second reads the first's last inputs from the slots' state, also where a step brought
    fewer rows than the state holds; slots are dealt out of order."""
    row_seg, seg_start = rows_of(segments)
    rows = int(seg_start[-1])
    slots = torch.tensor([3, 0, 5, 1][:len(segments)], dtype=torch.int32)
    w = 0.5 * torch.randn(width, taps, generator=gen(1))
    state = torch.randn(6, max(taps - 1, 0), width, generator=gen(2)).to(dtype)
    want_state, got_state = state.double(), state.clone().to(DEV)
    for step in range(2):
        x = torch.randn(rows, width, generator=gen(3 + step)).to(dtype)
        want = torch.empty(rows, width, dtype=torch.float64)
        ref.short_conv(x.double(), w, want_state, row_seg, seg_start, slots, want)
        got = torch.full((rows, width), 7.0, dtype=dtype, device=DEV)
        ops.short_conv(x.to(DEV), w.to(DEV), got_state if taps > 1 else None, row_seg.to(DEV), seg_start.to(DEV), slots.to(DEV), got)
        live = row_seg >= 0
        close(got[live.to(DEV)], want[live], 1e-6 if dtype == torch.float32 else BF16_EPS, 1e-6 if dtype == torch.float32 else 1e-2, f"step {step}")
        if taps > 1:
            assert torch.equal(got_state.cpu().double(), want_state), f"state behind step {step}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,taps", [(64, 4), (203, 2), (48, 1), (1536, 4)])
def test_the_norm_and_the_convolution_in_one_kernel(ops, ref, width, taps, dtype):
    rows = 5
    row_seg = torch.tensor([0, 1, -1, 3, 4], dtype=torch.int32)
    slots = torch.tensor([2, 0, 1, 4, 3], dtype=torch.int32)
    w = 0.5 * torch.randn(width, taps, generator=gen(1))
    norm_w = torch.full((width,), 1.3)
    state = torch.randn(6, max(taps - 1, 0), width, generator=gen(2)).to(dtype)
    want_state, got_state = state.double(), state.clone().to(DEV)
    x = 3 * torch.randn(rows, width, generator=gen(5))
    normed = torch.empty(rows, width, dtype=torch.float64)
    ref.rmsnorm(x.double(), norm_w, 1e-5, normed)
    normed = normed.to(dtype).double()                 # the unfused path rounds the norm's output to the compute type
    want = torch.empty(rows, width, dtype=torch.float64)
    seg_start = torch.arange(rows + 1, dtype=torch.int32)
    ref.short_conv(normed, w, want_state, row_seg, seg_start, slots, want)
    got = torch.empty(rows, width, dtype=dtype, device=DEV)
    ops.norm_short_conv(x.to(DEV), norm_w.to(DEV), 1e-5, w.to(DEV), got_state if taps > 1 else None, row_seg.to(DEV), slots.to(DEV), got)
    live = row_seg >= 0
    close(got[live.to(DEV)], want[live], 2e-6 if dtype == torch.float32 else 2 * BF16_EPS, 2e-6 if dtype == torch.float32 else 2e-2)
    if taps > 1:
        close(got_state, want_state, 1e-6 if dtype == torch.float32 else BF16_EPS, 1e-6)
        untouched = [s for s in range(6) if s not in (2, 0, 4, 3)]
        assert torch.equal(got_state[untouched].cpu(), state[untouched])


# ---------------------------------------------------------------------------------------------
# linear attention with a decay a head
# ---------------------------------------------------------------------------------------------
def decay_pair(decay):
    d = torch.tensor(decay, dtype=torch.float64)
    hi = d.float()
    return hi, (d - hi.double()).float()


LA_SHAPES = [(2, 16, 24), (1, 20, 12), (3, 10, 6), (2, 64, 64), (4, 128, 128), (2, 32, 16), (3, 48, 80), (2, 128, 32), (1, 96, 128)]


@pytest.mark.parametrize("form", ["tokens", "chunks"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", LA_SHAPES)
def test_linear_attention_over_steps(ops, ref, shape, dtype, form):
    """Portions of one token, of two, of a chunk less one, a chunk, a chunk and one, several chunks, beside padding rows; a
    second step goes on from the state the first left; the state of a slot no segment names stays as it is."""
    heads, dim, vdim = shape
    if form == "chunks" and (dim % 16 or vdim % 16):
        pytest.skip("the chunked kernel takes heads in blocks of sixteen lanes")
    decay = [1.0, 0.3, 0.97, 0.9990234375][:heads]
    hi, lo = decay_pair(decay)
    segments = [31, 1, 2, -3, 32, 33, 100, 64]
    row_seg, seg_start = rows_of(segments)
    rows = int(seg_start[-1])
    slots = torch.tensor([5, 0, 7, 8, 2, 1, 4, 3], dtype=torch.int32)
    width = heads * (2 * dim + vdim)
    state = 0.1 * torch.randn(10, heads, dim, vdim, generator=gen(1))
    want_state, got_state = state.double(), state.clone().to(DEV)
    tol = dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-5, atol=2e-5)    # the inputs are exact in both
    for step in range(2):
        qkv = (0.7 * torch.randn(rows, width + 8, generator=gen(10 + step))).to(dtype)      # rows wider than q | k | v
        want = torch.empty(rows, heads * vdim, dtype=torch.float64)
        ref.linear_attention(qkv.double(), hi, lo, want_state, row_seg, seg_start, slots, want, heads, dim, vdim)
        got = torch.full((rows, heads * vdim), 7.0, dtype=torch.float32, device=DEV)
        ops.linear_attention(qkv.to(DEV), hi.to(DEV), lo.to(DEV), got_state, row_seg.to(DEV), seg_start.to(DEV), slots.to(DEV), got,
                             heads, dim, vdim, form=form)
        scale = want.abs().max().item()
        close(got, want, tol["rtol"], tol["atol"] * scale, f"step {step}")
        close(got_state, want_state, 2e-5, 2e-5 * want_state.abs().max().item(), f"state behind step {step}")
    assert torch.equal(got_state[[6, 8, 9]].cpu(), state[[6, 8, 9]]), "slots of no segment and of padding stay"


@pytest.mark.parametrize("form", ["tokens", "chunks"])
@pytest.mark.parametrize("decay", [1.0, 0.999, 0.9])
def test_a_key_far_back_is_felt_by_its_decay(ops, form, decay):
    """One key of the prompt's early tokens is the query's own direction, all others are small: the output at the last token is
    that key's value times decay^distance (and times the product of query and key), whether the key sits right behind a
    chunk's edge or right before one, and whether the last tokens come in the same step or one by one afterwards."""
    heads, dim, vdim, n = 2, 64, 32, 700
    hi, lo = decay_pair([decay, decay])
    direction = torch.randn(dim, generator=gen(2))
    direction = direction / direction.norm()
    for target in (0, 31, 32, 33, 255, 256, 350, n - 1):        # a whole prompt of 700 tokens runs in parts of 256
        qkv = 1e-3 * torch.randn(n, heads * (2 * dim + vdim), generator=gen(3))
        qkv[target, heads * dim + dim:heads * dim + 2 * dim] = 6 * direction            # key of head 1
        qkv[n - 1, dim:2 * dim] = 6 * direction                                         # query of head 1
        value = qkv[target, 2 * heads * dim + vdim:2 * heads * dim + 2 * vdim] = torch.randn(vdim, generator=gen(4))
        want = 36.0 * decay ** (n - 1 - target) * value.double()
        for cut in (n, n - 40, 33):
            state = torch.zeros(1, heads, dim, vdim, device=DEV)
            out = torch.empty(n, heads * vdim, device=DEV)
            pieces = [(0, cut)] + [(t, t + 1) for t in range(cut, n)]
            for a, b in pieces:
                seg = torch.zeros(b - a, dtype=torch.int32, device=DEV)
                start = torch.tensor([0, b - a], dtype=torch.int32, device=DEV)
                ops.linear_attention(qkv[a:b].to(DEV), hi.to(DEV), lo.to(DEV), state, seg, start, torch.zeros(1, dtype=torch.int32, device=DEV),
                                     out[a:b], heads, dim, vdim, activation="none", form=form if b - a > 1 else "tokens")
            # the other keys are small, not nothing: their sum is the floor under a key that has all but decayed away
            close(out[n - 1, vdim:], want, 2e-3, 2e-3 * decay ** (n - 1 - target) + 5e-4, f"key at {target}, cut at {cut}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 64, 64), (3, 128, 48), (2, 128, 128), (1, 32, 16)])
def test_long_segments_run_in_parts(ops, ref, shape, dtype):
    """A step of 512 rows and more cuts its segments into parts of 256 tokens that start from zeros; a second kernel hands the
    states on and adds what the tokens lack.  Segments of one part, of a part and one token, of two parts exactly, of several
    with a short last one, beside padding rows and single tokens; a second step goes on from the first's state."""
    heads, dim, vdim = shape
    hi, lo = decay_pair([1.0, 0.97, 0.9990234375][:heads])
    segments = [700, 1, 300, -5, 256, 257, 512, 2, 1000]
    row_seg, seg_start = rows_of(segments)
    rows = int(seg_start[-1])
    slots = torch.tensor([5, 0, 7, 8, 2, 1, 4, 3, 6], dtype=torch.int32)
    state = 0.1 * torch.randn(10, heads, dim, vdim, generator=gen(1))
    want_state, got_state, single_state = state.double(), state.clone().to(DEV), state.clone().to(DEV)
    for step in range(2):
        qkv = (0.2 * torch.randn(rows, heads * (2 * dim + vdim), generator=gen(10 + step))).to(dtype)
        want = torch.empty(rows, heads * vdim, dtype=torch.float64)
        ref.linear_attention(qkv.double(), hi, lo, want_state, row_seg, seg_start, slots, want, heads, dim, vdim)
        args = (qkv.to(DEV), hi.to(DEV), lo.to(DEV))
        where = (row_seg.to(DEV), seg_start.to(DEV), slots.to(DEV))
        got = torch.full((rows, heads * vdim), 7.0, dtype=torch.float32, device=DEV)
        ops.linear_attention(*args, got_state, *where, got, heads, dim, vdim, form="chunks")
        single = torch.empty_like(got)
        ops.linear_attention(*args, single_state, *where, single, heads, dim, vdim, form="chunks", parts=False)
        scale = want.abs().max().item()
        close(got, want, 3e-5, 3e-5 * scale, f"step {step}")
        close(got, single, 1e-5, 1e-5 * scale, f"step {step}: parts against one pass")
        close(got_state, want_state, 3e-5, 3e-5 * want_state.abs().max().item(), f"state behind step {step}")
        assert not torch.equal(got, single), "the step was meant to run in parts"
    assert torch.equal(got_state[[8, 9]].cpu(), state[[8, 9]]), "slots of no segment and of padding stay"


def test_chunks_and_tokens_agree_and_a_row_does_not_depend_on_the_batch(ops):
    heads, dim, vdim = 3, 128, 64
    hi, lo = decay_pair([0.99, 0.95, 1.0])
    width = heads * (2 * dim + vdim)
    qkv = (0.5 * torch.randn(150, width, generator=gen(1))).to(torch.bfloat16).to(DEV)
    outs = {}
    for form in ("tokens", "chunks"):
        state = torch.zeros(4, heads, dim, vdim, device=DEV)
        row_seg, seg_start = rows_of([70, 80])
        out = torch.empty(150, heads * vdim, device=DEV)
        ops.linear_attention(qkv, hi.to(DEV), lo.to(DEV), state, row_seg.to(DEV), seg_start.to(DEV), torch.tensor([2, 1], dtype=torch.int32, device=DEV),
                             out, heads, dim, vdim, form=form)
        outs[form] = (out.cpu(), state.cpu())
    close(outs["chunks"][0], outs["tokens"][0], 1e-5, 1e-5 * outs["tokens"][0].abs().max().item(), "outputs")
    close(outs["chunks"][1], outs["tokens"][1], 1e-5, 1e-5 * outs["tokens"][1].abs().max().item(), "states")
    # the second request alone, in another slot: the same bits
    state = torch.zeros(4, heads, dim, vdim, device=DEV)
    row_seg, seg_start = rows_of([80])
    out = torch.empty(80, heads * vdim, device=DEV)
    ops.linear_attention(qkv[70:], hi.to(DEV), lo.to(DEV), state, row_seg.to(DEV), seg_start.to(DEV), torch.tensor([3], dtype=torch.int32, device=DEV),
                         out, heads, dim, vdim, form="chunks")
    assert torch.equal(out.cpu(), outs["chunks"][0][70:]) and torch.equal(state[3].cpu(), outs["chunks"][1][1])
    with pytest.raises(Exception, match="chunked"):
        ops.linear_attention(qkv[70:, :3 * 50].contiguous(), hi.to(DEV), lo.to(DEV), torch.zeros(4, 3, 20, 10, device=DEV), row_seg.to(DEV),
                             seg_start.to(DEV), torch.tensor([3], dtype=torch.int32, device=DEV), torch.empty(80, 30, device=DEV), 3, 20, 10,
                             form="chunks")


# ---------------------------------------------------------------------------------------------
# the gated norm behind the heads, PolyNorm
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("weighted", [True, False])
@pytest.mark.parametrize("rows,width", [(1, 48), (7, 203), (33, 1536), (130, 4096)])
def test_heads_normed_together_and_gated(ops, ref, rows, width, weighted, out_dtype):
    for x_dtype in {torch.float32, out_dtype}:
        x = (3 * torch.randn(rows, width, generator=gen(1))).to(x_dtype)
        wide = torch.randn(rows, width + 40, generator=gen(2)).to(out_dtype)
        gate = wide[:, 24:24 + width]                         # a column slice of a wider matrix
        weight = 1 + 0.3 * torch.randn(width, generator=gen(3)) if weighted else None
        want = torch.empty(rows, width, dtype=torch.float64)
        ref.gated_norm(x.double(), weight, 1e-5, gate.double(), want)
        got = torch.empty(rows, width, dtype=out_dtype, device=DEV)
        ops.gated_norm(x.to(DEV), weight.to(DEV) if weighted else None, 1e-5, wide.to(DEV)[:, 24:24 + width], got)
        close(got, want, 3e-6 if out_dtype == torch.float32 else BF16_EPS, 1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width", [(1, 50), (9, 80), (40, 1000), (70, 8960)])
def test_polynorm(ops, ref, rows, width, dtype):
    wide = (2 * torch.randn(rows, width + 16, generator=gen(1))).to(dtype)
    coeffs = torch.tensor([0.9, -0.4, 0.25, 0.1])
    want = torch.empty(rows, width, dtype=torch.float64)
    ref.polynorm(wide[:, :width].double(), coeffs, 1e-5, want)
    got = torch.empty(rows, width, dtype=dtype, device=DEV)
    ops.polynorm(wide.to(DEV)[:, :width], coeffs.to(DEV), 1e-5, got)
    close(got, want, 5e-6 if dtype == torch.float32 else BF16_EPS, 5e-6 if dtype == torch.float32 else 1e-3)
    alone = torch.empty(1, width, dtype=dtype, device=DEV)
    ops.polynorm(wide[rows - 1:, :width].contiguous().to(DEV), coeffs.to(DEV), 1e-5, alone)
    assert torch.equal(alone[0], got[rows - 1])


# ---------------------------------------------------------------------------------------------
# heads divided by their root mean square on their way into the pages; softmax with a sink over a chunk of positions
# ---------------------------------------------------------------------------------------------
from test_purivik_gpu import Scene, SEGMENTS, SINGLE_ROWS      # noqa: E402  (scattered pages full of loud numbers)

# heads, kv heads, key size, value size, chunk, page
SINK_SHAPES = [(4, 2, 32, 16, 24, 8), (3, 3, 32, 32, 40, 16), (8, 2, 64, 64, 80, 16), (3, 1, 24, 40, 7, 16), (4, 1, 64, 32, None, 16),
               (12, 2, 128, 128, 100, 64), (2, 1, 20, 12, 33, 8)]


def norm_store_attend(o, t, sc, chunk, scale, sinks, eps, dtype, on_device=True):
    rows = t["qkv"].shape[0]
    H, G, d, dv = sc.H, sc.G, sc.d, sc.dv
    o.head_norm_kv_store(t["qkv"], eps, d, t["row_pos"], t["row_seg"], t["tables"], t["k_pages"], t["v_pages"], H, G, d, sc.page,
                         v_dim=dv, key_chunk=sc.key_chunk)
    out = torch.empty(rows, H * dv, dtype=dtype, device=t["qkv"].device)
    extra = {}
    if on_device:
        need = o.attention_workspace_bytes(rows, H, G, d, sc.max_pos)
        extra = {"single_from": sc.single_from, "workspace": torch.empty(max(need, 1), dtype=torch.uint8, device=t["qkv"].device)}
    o.attention(t["qkv"][:, :H * d], t["k_pages"], t["v_pages"], t["tables"], t["row_pos"], t["row_seg"], t["seg_start"], out, H, G, d,
                sc.page, scale, None, sc.max_pos, v_dim=dv, chunk=chunk, key_chunk=sc.key_chunk, sinks=sinks, **extra)
    return out


@pytest.mark.parametrize("rows", ["mixed", "single"])
@pytest.mark.parametrize("fast", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", SINK_SHAPES)
def test_normed_heads_and_a_sink_over_pages(ops, ref, shape, dtype, fast, rows):
    H, G, d, dv, chunk, page = shape
    segments = SINGLE_ROWS if rows == "single" else SEGMENTS
    if dtype == torch.float32 and not fast:
        pytest.skip("float32 has one kernel")
    scale = 0.35
    loud = []
    for s, (held, new) in enumerate(segments):
        last = held + new - 1
        if chunk and last - last % chunk > 0 and held > 0:
            loud.append((s, min(last - last % chunk, held) - 1, 8.0))
        loud.append((s, last + 1, 8.0))
    sc = Scene(segments, H, G, d, dv, page, 0, seed=H * 100 + d + 1, dtype=dtype, loud=loud)
    # cached keys are what an earlier step stored: of unit root mean square
    flat = sc.k_pages.float().permute(0, 1, 3, 2, 4).reshape(sc.k_pages.shape[0], G, page, d)
    flat = flat / torch.sqrt((flat * flat).mean(-1, keepdim=True) + 1e-5)
    sc.k_pages = flat.view(sc.k_pages.shape[0], G, page, d // sc.key_chunk, sc.key_chunk).permute(0, 1, 3, 2, 4).contiguous().to(dtype)
    sinks = torch.linspace(-2.0, 3.0, H)
    want_t = sc.tensors("cpu", torch.float64)
    want = norm_store_attend(ref, want_t, sc, chunk, scale, sinks, 1e-5, torch.float64, on_device=False)
    none = norm_store_attend(ref, sc.tensors("cpu", torch.float64), sc, chunk, scale, None, 1e-5, torch.float64, on_device=False)
    assert (want - none).abs().max() > 0.05, "the sinks of this test take weight"
    ops.set_fast_kernels(fast)
    try:
        got_t = sc.tensors(DEV)
        got = norm_store_attend(ops, got_t, sc, chunk, scale, sinks.to(DEV), 1e-5, dtype)
        torch.cuda.synchronize()
    finally:
        ops.set_fast_kernels(True)
    assert torch.equal(got_t["v_pages"].cpu().double(), want_t["v_pages"]), "stored values"
    if dtype == torch.float32:
        close(got_t["k_pages"], want_t["k_pages"], 1e-5, 1e-5, "stored keys")
        close(got_t["qkv"][:, :H * d], want_t["qkv"][:, :H * d], 1e-5, 1e-5, "normed queries")
        close(got, want, 5e-4, 5e-4, "attention")
        return
    close(got_t["k_pages"], want_t["k_pages"], BF16_EPS, 1e-3, "stored keys")
    again = torch.empty_like(want)
    ref.attention(got_t["qkv"][:, :H * d].cpu().double(), got_t["k_pages"].cpu().double(), got_t["v_pages"].cpu().double(),
                  want_t["tables"], want_t["row_pos"], want_t["row_seg"], want_t["seg_start"], again, H, G, d, page, scale, None,
                  sc.max_pos, v_dim=dv, chunk=chunk, key_chunk=sc.key_chunk, sinks=sinks)
    close(got, again, 3 * BF16_EPS, 3e-2, "attention")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(64, 64), (128, 128), (24, 40)])
@pytest.mark.parametrize("sink", [-30.0, 2.0, 9.0])
def test_a_sink_takes_its_share_of_a_lone_key(ops, sink, sizes, dtype):
    """The first row of a chunk sees one key: its output is that key's value times e^s / (e^s + e^sink), as a single row and
    inside a portion that crosses the chunk's edge."""
    d, dv = sizes
    H, G, chunk, page = 2, 1, 50, 16
    for segs in ([(100, 1)], [(95, 10)], [(0, 3)]):
        sc = Scene(segs, H, G, d, dv, page, 0, seed=4, dtype=dtype)
        t = sc.tensors(DEV)
        pos = 100 if segs[0][0] else 0
        row = pos - segs[0][0]
        sinks = torch.tensor([sink, sink - 1.0], device=DEV)
        got = norm_store_attend(ops, t, sc, chunk, 0.2, sinks, 1e-5, dtype)
        q = t["qkv"][row, :H * d].double().view(H, d).cpu()
        pg, off = int(sc.tables[0, pos // page]), pos % page
        k = t["k_pages"][pg, 0, :, off, :].double().reshape(d).cpu()
        v = t["v_pages"][pg, 0, :, off].double().cpu()
        for h in range(H):
            s = 0.2 * (q[h] @ k)
            share = 1.0 / (1.0 + torch.exp(sinks[h].double().cpu() - s))
            close(got[row, h * dv:(h + 1) * dv], share * v, 1e-4 if dtype == torch.float32 else 3 * BF16_EPS, 1e-5 if dtype == torch.float32 else 1e-2,
                  f"head {h}, rows {segs}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width,experts,top", [(1, 64, 5, 2), (9, 68, 7, 7), (40, 320, 1, 1), (200, 1024, 64, 6), (3, 50, 130, 4)])
def test_a_softmax_router_divides_by_the_sum_of_its_picks(ops, ref, rows, width, experts, top, dtype):
    h = torch.randn(rows, width, generator=gen(1)).to(dtype)
    w = (torch.randn(experts, width, generator=gen(2)) * 0.3).to(dtype)
    ids, weights = torch.empty(rows, top, dtype=torch.int32), torch.empty(rows, top, dtype=torch.float32)
    ref.route_topk(h.float(), w.float(), top, ids, weights, score="softmax", renormalize=True, route_scale=2.5)
    got_ids = torch.empty(rows, top, dtype=torch.int32, device=DEV)
    got_w = torch.empty(rows, top, dtype=torch.float32, device=DEV)
    ops.route_topk(h.to(DEV), w.to(DEV), top, got_ids, got_w, score="softmax", renormalize=True, route_scale=2.5)
    same = got_ids.cpu() == ids
    assert same.float().mean() > 0.97          # near ties may swap
    close(got_w.cpu()[same], weights[same], 2e-5, 1e-6)
    close(got_w.sum(1), torch.full((rows,), 2.5), 1e-5, 0)


# ---------------------------------------------------------------------------------------------
# the engine
# ---------------------------------------------------------------------------------------------
LENGTHS = {"A": [5, 30, 61, 100, 49], "B": [45, 83, 161, 2, 120], "C": [9, 50, 300, 130], "D": [100, 37, 250, 81, 160], "E": [31, 2, 75, 120]}
TOL = {"float32": 1.5e-5, "bfloat16": 6e-2}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """(configuration, precision) -> folder, configuration, requests, plain logits, weights.  float32 runs random routers;
    bfloat16 runs routers whose every pick has a margin, since a pick that flips under rounding is a large error that says
    nothing about the kernels."""
    out = {}
    for name, cfg in vc.CONFIGS.items():
        for dtype in ("float32", "bfloat16"):
            tensors = vc.weights(cfg, 30 + ord(name), decided_router=dtype == "bfloat16")
            folder = vc.write_model(str(tmp_path_factory.mktemp(f"venadra_{name}_{dtype}")), cfg, tensors)
            requests = {f"r{i}": vc.random_ids(n, cfg["vocab"], 100 * ord(name) + i) for i, n in enumerate(LENGTHS[name])}
            w64 = vc.to_float64(tensors)
            plain = {rid: pv.forward(cfg, w64, toks) for rid, toks in requests.items()}
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
        tt.observe(f"venadra {what.split()[0]} {dtype}", err.max() / scale)
        over = err.max(axis=1) > TOL[dtype] * scale
        assert not over.any(), (f"{what}: request {rid}: max error {err.max():.3e} (limit {TOL[dtype] * scale:.3e}); first "
                                f"position over the limit: {int(np.argmax(over))}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
@pytest.mark.parametrize("family", ["whole", "last40", "portions", "mixed"])
def test_replay(models, tmp_path, name, dtype, family):
    folder, cfg, requests, plain, _ = models[name, dtype]
    refed = [rid for rid, toks in requests.items() if len(toks) >= 60][:1]
    steps = {"whole": tt.whole, "last40": lambda r: tt.last_tokens_one_by_one(r, 40), "portions": tt.portions,
             "mixed": lambda r: tt.mixed(r, seed=5, refeed=refed)}[family](requests)
    steps = tt.number(steps)
    runner = make_runner(folder, dtype, vc.PAGE_SIZES[name], tt.live_tokens_bound(steps))
    handed_out = tt.record_allocations(runner.cache)
    given_up = {}
    got = tt.run_in_process(runner, steps, cfg["vocab"], str(tmp_path), given_up)
    check(got, plain, dtype, f"{family} {name} {dtype}")
    if family == "mixed" and dtype == "float32":
        for rid, feedings in given_up.items():
            for first in feedings:         # other pages, a slot that another request has used in between
                assert np.abs(first - got[rid][:len(first)]).max() <= 2e-6 * np.abs(first).max(), f"{rid}: fed again, other logits"
    runner.cache.check_invariants()
    assert all(pool.available == pool.num_pages for pool in runner.cache.pools), "pages were lost"
    for pages in handed_out:
        assert len(pages) > len(set(pages)), "the trace was meant to use pages again"


@pytest.mark.parametrize("page_size", [4, 32, 64])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_at_other_page_sizes(models, tmp_path, page_size, dtype):
    folder, cfg, requests, plain, _ = models["D", dtype]
    steps = tt.number(tt.mixed(requests, seed=8))
    runner = make_runner(folder, dtype, page_size, tt.live_tokens_bound(steps, round_to=max(64, page_size)))
    got = tt.run_in_process(runner, steps, cfg["vocab"], str(tmp_path))
    check(got, plain, dtype, f"pages-of-{page_size} D {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "D"])
def test_cuts_agree_beyond_rounding(models, tmp_path, name, dtype):
    """The same request whole, in portions and in a mixed batch: a portion's edge moves where the linear attention's chunks
    begin, so the sums differ in their order and in nothing else."""
    folder, cfg, requests, plain, _ = models[name, dtype]
    results = []
    for i, make in enumerate([tt.whole, tt.portions, lambda r: tt.mixed(r, seed=3)]):
        steps = tt.number(make(requests))
        runner = make_runner(folder, dtype, vc.PAGE_SIZES[name], tt.live_tokens_bound(steps))
        results.append(tt.run_in_process(runner, steps, cfg["vocab"], str(tmp_path / str(i))))
    limit = 3e-6 if dtype == "float32" else 3e-2
    for rid in requests:
        scale = np.abs(results[0][rid]).max()
        assert np.abs(results[0][rid] - results[1][rid]).max() <= limit * scale, f"whole vs portions differ for {rid}"
        assert np.abs(results[0][rid] - results[2][rid]).max() <= limit * scale, f"whole vs mixed differ for {rid}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C", "E"])
def test_first_tokens_and_long_decoding(models, tmp_path, name, dtype):
    """Token by token from the very first token: the convolution's first inputs are zeros, the state starts empty, and the
    chunks of positions of the attention pass by several times."""
    folder, cfg, requests, plain, _ = models[name, dtype]
    rid = "r2"
    one = {rid: requests[rid]}
    steps = tt.number(tt.last_tokens_one_by_one(one, tail=len(requests[rid])))
    runner = make_runner(folder, dtype, vc.PAGE_SIZES[name], 320)
    got = tt.run_in_process(runner, steps, cfg["vocab"], str(tmp_path))
    check(got, {rid: plain[rid]}, dtype, f"token-by-token {name} {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C", "D"])
def test_decode_graphs_and_eager_steps_agree(models, tmp_path, name, dtype):
    folder, cfg, requests, plain, _ = models[name, dtype]
    steps = tt.number(tt.last_tokens_one_by_one(requests) + tt.mixed(requests, seed=21, decode_tail=40))
    results = []
    for i, use_graphs in enumerate((True, False)):
        runner = make_runner(folder, dtype, vc.PAGE_SIZES[name], tt.live_tokens_bound(steps), use_graphs=use_graphs)
        results.append(tt.run_in_process(runner, steps, cfg["vocab"], str(tmp_path / str(i))))
        assert (runner.graph_replays > 30) == use_graphs
    for rid, want in plain.items():
        a, b = results[0][rid].astype(np.float64), results[1][rid].astype(np.float64)
        if dtype == "float32":
            assert np.array_equal(a, b), f"{rid}: graph and eager steps differ in float32"
        else:
            assert np.abs(a - b).max() <= TOL[dtype] * np.abs(want).max()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_whole_and_in_portions(models, tmp_path, dtype):
    """1,100 tokens in one step (the linear attention runs in parts of 256 tokens), in two portions, and with the last 40
    decoded one by one."""
    folder, cfg, _, _, w64 = models["D", dtype]
    toks = vc.random_ids(1100, cfg["vocab"], 77)
    want = {"long": pv.forward(cfg, w64, toks)}
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
        def wrapped(ctx, x, binding, pending=None, _inner=block.forward):
            out = _inner(ctx, x, binding, pending)
            seen.append(x.clone().cpu().numpy())
            return out
        block.forward = wrapped
    toks = requests["r1"]
    runner.step([StepEntry("a", toks, [])])
    _, want = pv.forward(cfg, w64, toks, True)
    assert len(seen) == len(want) == 5
    for got, ref_x in zip(seen, want):
        assert np.abs(got - ref_x).max() <= 1e-5 * np.abs(ref_x).max()


def test_prompts_take_the_chunked_linear_attention_and_decode_steps_the_fused_forms(models, monkeypatch):
    """A portion of a prompt runs the linear attention in chunks on the matrix cores where the heads allow it (D: 64 lanes),
    a decode step token after token; the decode step reads the stream through norm and convolution in one kernel."""
    from fllm_amd.engine import StepEntry
    from fllm_amd.kernels import Ops
    calls = []
    for name in ("rmsnorm", "short_conv", "norm_short_conv", "linear_attention", "gated_norm", "polynorm", "head_norm_kv_store", "route_topk"):
        inner = getattr(Ops, name)
        monkeypatch.setattr(Ops, name, lambda self, *a, _n=name, _i=inner, **k: (calls.append(_n), _i(self, *a, **k))[1])
    folder, cfg, requests, _, _ = models["A", "bfloat16"]
    runner = make_runner(folder, "bfloat16", 8, 256, use_graphs=False)
    toks = requests["r3"]
    runner.step([StepEntry("a", toks[:40], [])])
    assert calls.count("linear_attention") == 3 and calls.count("head_norm_kv_store") == 2 and calls.count("polynorm") == 2
    assert calls.count("short_conv") == 5 and calls.count("gated_norm") == 5
    calls.clear()
    runner.step([StepEntry("a", toks[40:41], [0])])
    assert calls.count("norm_short_conv") == 5 and calls.count("short_conv") == 0 and calls.count("linear_attention") == 3
    assert calls.count("route_topk") == 2


@pytest.mark.parametrize("name", ["A", "D", "E"])
def test_greedy_generation_through_the_scheduler(models, name):
    from fllm_amd import Engine, SamplingParams
    folder, cfg, _, _, w64 = models[name, "float32"]
    prompts = [vc.random_ids(n, cfg["vocab"], 20 + n) for n in (3, 26, 41, 90)]
    want = [pv.greedy(cfg, w64, p, 12) for p in prompts]
    for opts in (dict(num_blocks=64), dict(num_blocks=14, max_batched_tokens=16)):
        engine = Engine(folder, dtype="float32", ctx=256, max_seqs=3, block_size=vc.PAGE_SIZES[name],
                        **{"max_batched_tokens": 64, **opts})
        assert engine.generate(prompts, SamplingParams(max_tokens=12)) == want
        engine.runner.cache.check_invariants()
    folder, cfg, _, _, w64 = models[name, "bfloat16"]
    engine = Engine(folder, dtype="bfloat16", ctx=256, max_seqs=4, block_size=vc.PAGE_SIZES[name])
    out = engine.generate(prompts, SamplingParams(max_tokens=12))
    assert [len(o) for o in out] == [12] * 4
    for p, o in zip(prompts, out):
        logits = pv.forward(cfg, w64, p)[-1]
        top = np.sort(logits)[-2:]
        if top[1] - top[0] > 0.1 * np.abs(logits).max():
            assert o[0] == int(np.argmax(logits))


def test_the_command_line_generates_and_samples(models):
    folder, cfg, _, _, w64 = models["A", "float32"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prompt = vc.random_ids(30, cfg["vocab"], 4)
    cmd = [sys.executable, "-m", "fllm_amd", "run", folder, "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "8",
           "--dtype", "float32", "--ctx", "256", "--kv-blocks", "32", "--max-seqs", "2"]
    proc = subprocess.run(cmd, cwd=root, capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr[-2000:]
    record = json.loads(proc.stdout.strip().splitlines()[0])
    assert record["finish_reason"] == "length" and record["token_ids"] == pv.greedy(cfg, w64, prompt, 8)
    flags = ["--temperature", "0.8", "--top-k", "20", "--top-p", "0.9", "--seed", "3", "--repeat-penalty", "1.3", "--n", "2",
             "--logprobs", "2", "--dtype", "bfloat16"]
    proc = subprocess.run(cmd + flags, cwd=root, capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr[-2000:]
    records = [json.loads(line) for line in proc.stdout.strip().splitlines()]
    assert len(records) == 2 and all(len(r["token_ids"]) == 8 for r in records)
