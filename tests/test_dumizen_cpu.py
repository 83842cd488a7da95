"""Dumizen on the CPU: configuration, the model's description, and the engine's own logic (pages with pooled blocks beside
them, state slots, looped layers with caches of their own, batches, portions, scheduler) with the plain kernels of
tests/reference_ops.py in place of the HIP library, against the plain implementation of tests/plain_dumizen.py; and that
plain implementation's mechanisms one by one."""
import copy

import numpy as np
import pytest
import torch

import dumizen_configs as dc
import plain_dumizen as pd
import trace_tools as tt
from reference_ops import ReferenceOps
from fllm_amd import Engine, SamplingParams
from fllm_amd.config.spec import ConfigError
from fllm_amd.engine import ModelRunner, StepEntry
from fllm_amd.registry import model_spec_from_config
from fllm_amd.weights.loader import WeightsError, check_tensors


def runner_for(name, max_tokens, seed=3, **kw):
    cfg = dc.CONFIGS[name]
    _, spec = model_spec_from_config(cfg)
    tensors = dc.weights(cfg, seed)
    r = ModelRunner(spec, dict(tensors), dtype="float32", device="cpu", page_size=dc.PAGE_SIZES[name], max_tokens=max_tokens,
                    max_requests=4, max_context=512, ops=ReferenceOps(), **kw)
    return cfg, dc.to_float64(tensors), r


# ---- the plain implementation's mechanisms, each alone ----------------------------------------------------------------
def test_plain_rotation_pairs_lane_i_with_lane_i_plus_half_and_leaves_the_rest():
    x = np.zeros((3, 1, 6))
    x[:, 0, 0], x[:, 0, 5] = 1.0, 7.0
    out = pd.rotate(x, {"dims": 4, "base": 10.0}, [0, 1, 2])
    assert np.allclose(out[:, 0, 0], np.cos([0, 1, 2])) and np.allclose(out[:, 0, 2], np.sin([0, 1, 2]))      # lane 0 turns into lane 2
    assert np.allclose(out[:, 0, 1], 0) and np.allclose(out[:, 0, 3], 0) and np.allclose(out[:, 0, 4:], x[:, 0, 4:])
    second = np.zeros((2, 1, 4))
    second[:, 0, 1] = 1.0
    assert np.allclose(pd.rotate(second, {"dims": 4, "base": 10.0}, [0, 5])[1, 0, 3], np.sin(5 * 10.0 ** -0.5))


def test_plain_band_scaling_keeps_fast_lanes_divides_slow_ones_and_grows_the_magnitude():
    dims, base, s = 16, 100.0, {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}
    plain, one = pd.rotary_angles(dims, base, None, [1])
    scaled, magnitude = pd.rotary_angles(dims, base, s, [1])
    assert one == 1.0 and np.isclose(magnitude, 0.1 * np.log(4.0) + 1.0)
    lane = lambda turns: dims * np.log(32 / (2 * np.pi * turns)) / (2 * np.log(base))
    lo, hi = max(np.floor(lane(8.0)), 0), min(np.ceil(lane(1.0)), dims - 1)
    assert 0 <= lo < hi < dims // 2              # the ramp lies inside the lanes of this table: all three bands occur
    for i in range(dims // 2):
        ramp = min(max((i - lo) / (hi - lo), 0.0), 1.0)
        assert np.isclose(scaled[0, i], plain[0, i] * (ramp / 4.0 + 1 - ramp))
    assert np.isclose(scaled[0, 0], plain[0, 0]) and np.isclose(scaled[0, -1], plain[0, -1] / 4.0)


def test_plain_window_edges_and_pooled_blocks():
    """One value lane tells the positions apart: v_j = j.  With equal scores the output is the mean of what is seen."""
    T, size, pool = 14, 5, 3
    q, k = np.zeros((T, 1, 2)), np.zeros((T, 1, 2))
    v = np.arange(T, dtype=float).reshape(T, 1, 1)
    out = pd.pooled_window_attention(q, k, v, 1.0, size, pool)[:, 0, 0]
    for i in range(T):
        tokens = list(range(max(0, i - size + 1), i + 1))
        blocks = [b for b in range(T // pool) if b * pool + pool - 1 <= i - size]
        seen = [float(np.mean(range(b * pool, b * pool + pool))) for b in blocks] + [float(j) for j in tokens]
        assert np.isclose(out[i], np.mean(seen)), i
    # keys 0..2 stand out for every query.  Position 5 sees tokens 1..5: tokens 1 and 2 carry it.  Position 6 sees 2..6 and
    # block 0 not yet (it ends at 2 > 6 - 5): token 2 alone.  Position 7 sees 3..7 and block 0 (2 <= 7 - 5): the block's mean.
    # Position 9 sees 5..9 and block 0; tokens 3 and 4 are out of the window and their block is not complete behind it.
    k2, q2 = np.zeros((T, 1, 2)), np.zeros((T, 1, 2))
    k2[0:3, 0, 0], q2[:, 0, 0] = 30.0, 1.0
    out2 = pd.pooled_window_attention(q2, k2, v, 1.0, size, pool)[:, 0, 0]
    assert np.allclose(out2[[5, 6, 7, 9]], [1.5, 2.0, 1.0, 1.0], atol=1e-6)
    v3 = v.copy()
    v3[3:5] = 1e6                             # what tokens 3 and 4 hold reaches position 9 in no way
    assert np.isclose(pd.pooled_window_attention(q, k, v3, 1.0, size, pool)[9, 0, 0], np.mean([1.0, 5, 6, 7, 8, 9]))


def test_plain_sigmoid_attention_sums_weights_that_are_not_normalized():
    T = 6
    q, k = np.zeros((T, 2, 2)), np.zeros((T, 1, 2))
    v = np.ones((T, 1, 1))
    r1, r2, pb = np.array([0.0, 1.0]), np.array([0.0, 0.5]), np.array([0.0, 2.0])
    out = pd.sigmoid_attention(q, k, v, 1.0, 5.0, r1, r2, pb)
    assert np.allclose(out[:, 0, 0], 0.5 * np.arange(1, T + 1))           # head 0: every key weighs 1/2, the sum grows
    want = [sum(pd.sigmoid(2.0 - np.log(1 + 0.5 * (i - j))) for j in range(i + 1)) for i in range(T)]
    assert np.allclose(out[:, 1, 0], want)
    capped = pd.sigmoid_attention(np.full((1, 1, 1), 100.0), np.full((1, 1, 1), 100.0), np.ones((1, 1, 1)), 1.0, 3.0,
                                  np.zeros(1), np.zeros(1), np.zeros(1))
    assert np.isclose(capped[0, 0, 0], pd.sigmoid(3.0 * np.tanh(1e4 / 3.0)))


def test_plain_sink_takes_weight_and_gives_nothing():
    q, k, v = np.zeros((3, 1, 2)), np.zeros((3, 1, 2)), np.ones((3, 1, 1))
    out = pd.sink_attention(q, k, v, 1.0)[:, 0, 0]
    assert np.allclose(out, [1 / 2, 2 / 3, 3 / 4])              # n keys of score 0 and the sink: n / (n + 1)


def test_plain_retention_is_a_decayed_sum_of_outer_products():
    rng = np.random.default_rng(0)
    T, H, d, dv = 7, 2, 3, 4
    q, k, v = rng.normal(size=(T, H, d)), rng.normal(size=(T, H, d)), rng.normal(size=(T, H, dv))
    decay = [0.5, 1.0]
    got = pd.retention(q, k, v, decay)
    for t in range(T):
        for h in range(H):
            want = sum(decay[h] ** (t - s) * (q[t, h] @ k[s, h]) * v[s, h] for s in range(t + 1))
            assert np.allclose(got[t, h], want)


def test_plain_router_corrections_choose_groups_limit_and_scores_weigh():
    h = np.eye(4)[:1]                                            # one token; the router's first column holds the logits
    logits = np.array([2.0, -1.0, 1.5, 1.4, 0.0, -3.0])
    w_router = np.zeros((6, 4))
    w_router[:, 0] = logits
    s = pd.sigmoid(logits)
    router = {"experts": 6, "top": 2, "scale": 3.0, "groups": {"count": 3, "keep": 1}}
    ids, weights = pd.route(h, w_router, np.zeros(6), router)    # groups (0, 1), (2, 3), (4, 5): sums s0 + s1 < s2 + s3
    assert ids.tolist() == [[2, 3]] and np.allclose(weights[0], s[[2, 3]] / s[[2, 3]].sum() * 3.0)
    router["groups"]["keep"] = 2
    ids, _ = pd.route(h, w_router, np.zeros(6), router)
    assert ids.tolist() == [[0, 2]]                              # the best two experts of the two best groups
    correction = np.array([0.0, 0.0, 0.0, 0.0, 5.0, 0.0])        # a correction lifts expert 4 into the picks; its weight stays its score
    ids, weights = pd.route(h, w_router, correction, router)
    assert 4 in ids[0].tolist() and np.isclose(weights.sum(), 3.0)
    k = ids[0].tolist().index(4)
    assert np.isclose(weights[0, k], s[4] / s[ids[0]].sum() * 3.0)
    router["groups"] = {"count": 3, "keep": 1}
    ids, _ = pd.route(h, w_router, np.array([0.0, 0.0, 0.0, 0.0, 1.5, -9.0]), router)
    assert ids.tolist() == [[2, 3]]                              # a negative choice score is no zero: group 2 sums (s4 + 1.5) + (s5 - 9), not s4 + 1.5


def test_plain_run_order_repeats_the_looped_layers():
    assert pd.run_order(dc.A) == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (3, None)]
    assert pd.run_order(dc.C) == [(0, 0), (1, None), (2, None), (0, 1), (1, None), (2, None), (0, 2), (1, None), (2, None)]
    assert pd.run_order(dc.B) == [(0, None), (1, None), (2, None)]


# ---- configuration and description ------------------------------------------------------------------------------------
def test_the_description_names_the_parts():
    typed, spec = model_spec_from_config(dc.A)
    assert spec.architecture == "dumizen" and [e.layer for e in spec.run_order] == [0, 1, 2, 1, 2, 3]
    assert [e.before is not None for e in spec.run_order] == [False, True, False, True, False, False]
    assert spec.run_order[3].before["row"] == 1 and spec.run_order[1].before.tensors == {"mix": "loop.in", "steps": "loop.step"}
    kinds = [layer.mixer.kind for layer in spec.layers]
    assert kinds == ["sigmoid_attention", "normed_attention", "mixer_pair", "normed_attention"]
    second = spec.layers[1].mixer
    assert second["window"] == 12 and second["pool"] == 4 and second["qk_norm"] == "head" and second["position"]["scaling"] == "yarn"
    left, right = spec.layers[2].mixer["left"], spec.layers[2].mixer["right"]
    assert left["values"] == "keys" and left["sink"] == "zero" and left["output_gate"] and left["qk_norm"] == "projection"
    assert right.kind == "lightning_attention" and right["head_norm"] and right["key_scale"] == 16 ** -0.5
    ff = spec.layers[0].feed_forward
    assert ff["groups"] == 3 and ff["groups_kept"] == 2 and ff["shared"] == 40 and not ff["gated"] and ff["weight_on"] == "output"
    assert spec.layers[3].feed_forward is None and "l3.norm2b" in spec.ignorable_tensors
    assert all(layer.block.kind == "sandwich" for layer in spec.layers)
    _, spec_b = model_spec_from_config(dc.B)
    assert "loop.in" in spec_b.ignorable_tensors and spec_b.layers[0].feed_forward["shared"] == 0


def test_every_run_of_a_layer_has_pages_pools_and_state_of_its_own():
    _, _, r = runner_for("A", 64)
    b = r.model.bindings
    assert len(b) == 6
    assert b[1].pool_k.shape[1:] == (1, 2, 32) and b[1].pool_v.shape[1:] == (1, 2, 16)        # pages of 8, blocks of 4: two slots
    assert b[1].k_pages.data_ptr() != b[3].k_pages.data_ptr() and b[1].pool_k.data_ptr() != b[3].pool_k.data_ptr()
    assert b[0].pool_k is None and b[2].pool_k is None
    assert set(b[2].state) == {"right."} and b[2].state["right."].shape == (4, 2, 16, 24)
    assert b[2].state["right."].data_ptr() != b[4].state["right."].data_ptr()
    _, _, c = runner_for("C", 64)
    assert c.model.bindings[0].pool_k.shape[2] == 6                                            # ceil(16 / 3) blocks can end in a page


@pytest.mark.parametrize("change,match", [
    (lambda c: c["layers"][0].__setitem__("type", "recurrent"), "no mixer of this design"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "dense"), "no feed-forward of this design"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("kv_heads", 3), "not a multiple"),
    (lambda c: c["layers"][2]["mixer"]["right"].__setitem__("decay", [0.5]), "for each of the 2 heads"),
    (lambda c: c["layers"][0]["mlp"]["router"].__setitem__("top", 5), "more than the 4 experts of the kept groups"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].__setitem__("count", 4), "equal groups"),
    (lambda c: c["layers"][1]["mixer"]["mask"].__setitem__("pool", 0), "positive"),
    (lambda c: c["layers"][1]["mixer"].pop("mask"), "requires layers\\[1\\].mixer.mask"),
    (lambda c: c["layers"][2]["mixer"]["left"].__setitem__("vdim", 16), "values of this mixer are its keys"),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 34), "even and at most dim"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("softcap", 0.0), "positive"),
    (lambda c: c["loop"].__setitem__("stop", 9), "must name a run"),
    (lambda c: c["norm"].__setitem__("eps", 0), "positive"),
])
def test_configurations_that_are_refused(change, match):
    cfg = copy.deepcopy(dc.A)
    change(cfg)
    with pytest.raises(ConfigError, match=match):
        model_spec_from_config(cfg)


def test_the_loader_names_what_does_not_fit():
    _, spec = model_spec_from_config(dc.A)
    shapes = {n: tuple(t.shape) for n, t in dc.weights(dc.A, 1).items()}
    check_tensors(spec, shapes)
    broken = dict(shapes)
    del broken["l1.mlp.correction"]
    del broken["l2.mix.left.q.norm"]
    broken["l1.mix.q.norm"] = (4 * 32,)              # one vector for all heads, not one a head
    broken["l2.mix.left.v"] = (64, 64)               # this mixer has no value projection
    broken["l3.mlp.router"] = (6, 64)                # a layer without feed-forward holds none
    with pytest.raises(WeightsError) as err:
        check_tensors(spec, broken)
    assert err.value.missing == ["l1.mlp.correction", "l2.mix.left.q.norm"]
    assert err.value.unexpected == ["l2.mix.left.v", "l3.mlp.router"] and [w[0] for w in err.value.wrong_shape] == ["l1.mix.q.norm"]


# ---- the engine's logic -------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name,lengths", [("A", [5, 30, 61]), ("B", [45, 33]), ("C", [9, 50]), ("D", [70, 37])])
@pytest.mark.parametrize("family", ["whole", "last", "portions", "mixed"])
def test_every_way_of_cutting_gives_the_plain_logits(tmp_path, name, lengths, family):
    vocab = dc.CONFIGS[name]["vocab"]
    requests = {f"r{i}": dc.random_ids(n, vocab, 70 + i) for i, n in enumerate(lengths)}
    steps = {"whole": tt.whole, "last": lambda r: tt.last_tokens_one_by_one(r, 19), "portions": tt.portions,
             "mixed": lambda r: tt.mixed(r, seed=4, decode_tail=6, refeed=[f"r{len(lengths) - 1}"])}[family](requests)
    steps = tt.number(steps)
    cfg, w64, runner = runner_for(name, tt.live_tokens_bound(steps, round_to=dc.PAGE_SIZES[name]))
    handed_out = tt.record_allocations(runner.cache)
    given_up = {}
    got = tt.run_in_process(runner, steps, vocab, str(tmp_path), given_up)
    for rid, feedings in given_up.items():          # ended half way and fed again: other pages, a cleared slot, the same logits
        again = got[rid][:len(feedings[0])]
        assert np.abs(feedings[0] - again).max() <= 1e-5 * np.abs(again).max()
    for rid, toks in requests.items():
        want = pd.forward(cfg, w64, toks)
        assert np.abs(got[rid] - want).max() <= 3e-5 * np.abs(want).max(), (family, rid)
    runner.cache.check_invariants()
    assert all(p.available == p.num_pages for p in runner.cache.pools)
    if family == "mixed":
        assert all(len(pages) > len(set(pages)) for pages in handed_out), "the trace was meant to use pages again"


def test_the_residual_stream_after_every_layer_run():
    cfg, w64, runner = runner_for("A", 64)
    seen = []
    for block in runner.model.blocks:
        def wrapped(ctx, x, binding, _inner=block.forward):
            _inner(ctx, x, binding)
            seen.append(x.clone().numpy())
        block.forward = wrapped
    toks = dc.random_ids(29, cfg["vocab"], 5)
    runner.step([StepEntry("a", toks, [])])
    want, _ = pd.layer_outputs(cfg, w64, toks)
    assert len(seen) == len(want) == 6
    for got, ref in zip(seen, want):
        assert np.abs(got - ref).max() <= 2e-5 * np.abs(ref).max()


def _one_far_key(cfg_name, layer, far, length, boost=6.0):
    """Weights and tokens in which ONE early position stands out for the last query of one windowed layer: its key and the
    last token's query are scaled up through the tokens' embeddings, so that whether that position (or its block) is seen
    shows in the logits."""
    cfg = dc.CONFIGS[cfg_name]
    tensors = dc.weights(cfg, 9)
    toks = dc.random_ids(length, cfg["vocab"], 77)
    toks[far], toks[-1] = 1, 2
    toks = [t if i in (far, length - 1) or t not in (1, 2) else 3 for i, t in enumerate(toks)]
    tensors["embed"][1] *= boost
    tensors["embed"][2] *= boost
    return cfg, tensors, toks


@pytest.mark.parametrize("far", [0, 3, 4, 7, 8, 11, 12, 15, 16, 20])
def test_keys_around_the_edges_of_window_and_blocks(far):
    """A, pages of 8, windows of 12, blocks of 4; the last query sits at position 23: tokens 12..23 are in its window, the
    blocks 0..2 (positions 0..11) behind it, each as one mean.  Decoded token by token and fed as one prompt, the engine
    follows the plain implementation whichever position carries the key that stands out."""
    cfg, tensors, toks = _one_far_key("A", 1, far, 24)
    _, spec = model_spec_from_config(cfg)
    w64 = dc.to_float64(tensors)
    want = pd.forward(cfg, w64, toks)
    for cut in ("prompt", "decoded"):
        r = ModelRunner(spec, dict(tensors), dtype="float32", device="cpu", page_size=8, max_tokens=64, max_requests=2,
                        max_context=128, ops=ReferenceOps())
        if cut == "prompt":
            got = r.step([StepEntry("a", toks, [23])]).numpy()[0]
        else:
            r.step([StepEntry("a", toks[:10], [])])
            for t in toks[10:-1]:
                r.step([StepEntry("a", [t], [])])
            got = r.step([StepEntry("a", toks[-1:], [0])]).numpy()[0]
        assert np.abs(got - want[23]).max() <= 3e-5 * np.abs(want).max(), (far, cut)


def test_a_slot_and_pages_that_are_used_again_start_clean():
    """Two requests one after the other in the same state slot and pages: the second finds neither the first's retention
    matrix nor its blocks' means."""
    cfg, w64, runner = runner_for("C", 64)
    first, second = dc.random_ids(40, cfg["vocab"], 1), dc.random_ids(27, cfg["vocab"], 2)
    runner.step([StepEntry("a", first, [])])
    slot, pages = runner.cache.slot("a"), list(runner.cache.table("a", 0))
    runner.free_request("a")
    got = runner.step([StepEntry("b", second, list(range(27)))]).numpy()
    assert runner.cache.slot("b") == slot and set(runner.cache.table("b", 0)) <= set(pages)
    want = pd.forward(cfg, w64, second)
    assert np.abs(got - want).max() <= 3e-5 * np.abs(want).max()


def test_long_decoding_from_the_first_token():
    cfg, w64, runner = runner_for("B", 128)
    toks = dc.random_ids(90, cfg["vocab"], 8)
    got = np.concatenate([runner.step([StepEntry("a", [t], [0])]).numpy() for t in toks])
    want = pd.forward(cfg, w64, toks)
    assert np.abs(got - want).max() <= 3e-5 * np.abs(want).max()


def test_batches_of_unequal_requests_agree_with_each_alone():
    cfg, w64, runner = runner_for("A", 192)
    a, b, c = (dc.random_ids(n, cfg["vocab"], 40 + n) for n in (37, 2, 21))
    runner.step([StepEntry("a", a[:30], []), StepEntry("c", c[:20], [])])
    got = runner.step([StepEntry("a", a[30:], list(range(7))), StepEntry("b", b, [0, 1]), StepEntry("c", c[20:], [0])]).numpy()
    want = np.concatenate([pd.forward(cfg, w64, a)[30:], pd.forward(cfg, w64, b), pd.forward(cfg, w64, c)[20:]])
    assert np.abs(got - want).max() <= 3e-5 * np.abs(want).max()


@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_scheduler(tmp_path, name):
    cfg = dc.CONFIGS[name]
    tensors = dc.weights(cfg, 11)
    folder = dc.write_model(str(tmp_path / "m"), cfg, tensors)
    prompts = [dc.random_ids(n, cfg["vocab"], 20 + n) for n in (3, 26, 41)]
    w64 = dc.to_float64(tensors)
    want = []
    for p in prompts:
        toks = list(p)
        for _ in range(8):
            toks.append(int(np.argmax(pd.forward(cfg, w64, toks)[-1])))
        want.append(toks[len(p):])
    for opts in (dict(num_blocks=64), dict(num_blocks=12, max_batched_tokens=12)):       # roomy; few pages and small portions
        engine = Engine(folder, dtype="float32", device="cpu", ctx=256, max_seqs=3, block_size=dc.PAGE_SIZES[name],
                        ops=ReferenceOps(), **{"max_batched_tokens": 32, **opts})
        assert engine.generate(prompts, SamplingParams(max_tokens=8)) == want
        engine.runner.cache.check_invariants()
