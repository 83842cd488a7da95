"""Venadra on the CPU: configuration, the model's description, and the engine's own logic (layers that run another layer's
tensors, state slots beside pages, batches, portions, scheduler) with the plain kernels of tests/reference_ops.py in place of
the HIP library, against the plain implementation of tests/plain_venadra.py; and that plain implementation's mechanisms one
by one."""
import copy

import numpy as np
import pytest
import torch

import plain_venadra as pv
import trace_tools as tt
import venadra_configs as vc
from reference_ops import ReferenceOps
from fllm_amd import Engine, SamplingParams
from fllm_amd.config.spec import ConfigError
from fllm_amd.engine import ModelRunner, StepEntry
from fllm_amd.registry import model_spec_from_config
from fllm_amd.weights.loader import WeightsError, check_tensors


def runner_for(name, max_tokens, seed=3, **kw):
    cfg = vc.CONFIGS[name]
    _, spec = model_spec_from_config(cfg)
    tensors = vc.weights(cfg, seed)
    r = ModelRunner(spec, dict(tensors), dtype="float32", device="cpu", page_size=vc.PAGE_SIZES[name], max_tokens=max_tokens,
                    max_requests=4, max_context=512, ops=ReferenceOps(), **kw)
    return cfg, vc.to_float64(tensors), r


# ---- the plain implementation's mechanisms, each alone ----------------------------------------------------------------
def test_plain_convolution_reaches_back_taps_minus_one_and_starts_on_zeros():
    h = np.arange(1.0, 6.0).reshape(5, 1)
    w = np.array([[100.0, 10.0, 1.0]])                       # the last column meets the token itself
    out = pv.input_convolution(h, w)
    assert out[:, 0].tolist() == [1 + 1, 2 + 12, 3 + 123, 4 + 234, 5 + 345]
    assert np.array_equal(pv.input_convolution(h, np.array([[2.0]])), 3 * h)       # one tap: no neighbour


def test_plain_lightning_is_a_decayed_sum_of_outer_products():
    rng = np.random.default_rng(0)
    T, W, H, d, dv = 6, 5, 2, 3, 4
    h = rng.normal(size=(T, W))
    wq, wk, wv, wg = (rng.normal(size=(H * n, W)) for n in (d, d, dv, dv))
    wo, nw, decay = rng.normal(size=(W, H * dv)), rng.uniform(0.5, 1.5, H * dv), [0.5, 1.0]
    got = pv.lightning(h, wq, wk, wv, wg, wo, nw, decay, H, d, dv, 1e-5)
    q, k, v = (pv.silu(h @ m.T).reshape(T, H, -1) for m in (wq, wk, wv))
    o = np.zeros((T, H, dv))
    for t in range(T):
        for a in range(H):
            for s in range(t + 1):               # the closed form: every earlier token, decayed by its distance, itself by none
                o[t, a] += decay[a] ** (t - s) * (q[t, a] @ k[s, a]) * v[s, a]
    want = (pv.rms(o.reshape(T, -1), 1e-5) * nw * pv.sigmoid(h @ wg.T)) @ wo.T
    assert np.allclose(got, want)


def test_plain_attention_chunks_count_from_zero_and_the_sink_only_takes_weight():
    rng = np.random.default_rng(1)
    T, W, H, G, d, dv = 9, 6, 2, 1, 4, 3
    h = rng.normal(size=(T, W))
    wq, wk, wv, wg, wo = (rng.normal(size=s) for s in ((H * d, W), (G * d, W), (G * dv, W), (H * dv, W), (W, H * dv)))
    args = dict(heads=H, kv_heads=G, dim=d, vdim=dv, scale=0.7, eps=1e-5)
    low = pv.chunk_attention(h, wq, wk, wv, wg, wo, np.array([-50.0, -50.0]), chunk=4, **args)
    # position 4 begins a chunk: it sees itself alone, so with a sink that takes nothing its output is its own gated value
    v4 = (h[4] @ wv.T).reshape(G, dv)
    alone = (np.concatenate([v4[0], v4[0]]) * pv.sigmoid(h[4] @ wg.T)) @ wo.T
    assert np.allclose(low[4], alone)
    # a token of another chunk changes nothing behind the edge
    h2 = h.copy()
    h2[3] += 5.0
    assert np.allclose(pv.chunk_attention(h2, wq, wk, wv, wg, wo, np.array([-50.0, -50.0]), chunk=4, **args)[4:], low[4:])
    # a large sink takes nearly all the weight and has no value: the output shrinks, its direction at a lone key stays
    high = pv.chunk_attention(h, wq, wk, wv, wg, wo, np.array([5.0, 5.0]), chunk=4, **args)
    q4 = pv.rms((h[4] @ wq.T).reshape(H, d), 1e-5)
    k4 = pv.rms((h[4] @ wk.T).reshape(G, d), 1e-5)
    share = [np.exp(0.7 * q4[a] @ k4[0]) / (np.exp(0.7 * q4[a] @ k4[0]) + np.exp(5.0)) for a in range(H)]
    by_hand = (np.concatenate([share[0] * v4[0], share[1] * v4[0]]) * pv.sigmoid(h[4] @ wg.T)) @ wo.T
    assert np.allclose(high[4], by_hand)
    # without a mask every earlier key is seen
    assert not np.allclose(pv.chunk_attention(h, wq, wk, wv, wg, wo, np.zeros(2), chunk=0, **args)[4], low[4])


def test_plain_polynorm_by_hand():
    z = np.array([[1.0, -2.0, 3.0]])
    up, down = np.eye(3), np.eye(3)
    got = pv.polynorm_ff(z, up, down, [2.0, 3.0, 5.0, 7.0], 0.0)
    n = lambda v: v / np.sqrt((v * v).mean())
    assert np.allclose(got, 2 * n(z) + 3 * n(z ** 2) + 5 * n(z ** 3) + 7)


def test_plain_router_renormalizes_the_picks_and_weighs_outputs():
    rng = np.random.default_rng(2)
    h = rng.normal(size=(3, 6))
    router = rng.normal(size=(4, 6))
    experts = [(rng.normal(size=(5, 6)), rng.normal(size=(5, 6)), rng.normal(size=(6, 5))) for _ in range(4)]
    got = pv.routed_ff(h, router, experts, 2, 1.5, 2.5)
    z = h[1] @ router.T
    s = np.exp(z) / np.exp(z).sum()
    picks = np.argsort(-s)[:2]
    w = s[picks] / s[picks].sum() * 2.5
    assert np.isclose(w.sum(), 2.5)
    by_hand = sum(wi * pv.expert(h[1:2], *experts[e], 1.5)[0] for wi, e in zip(w, picks))
    assert np.allclose(got[1], by_hand)
    g = np.minimum(h[1] @ experts[0][0].T, 1.5)
    u = np.clip(h[1] @ experts[0][1].T, -1.5, 1.5)
    assert np.allclose(pv.expert(h[1:2], *experts[0], 1.5)[0], (g * pv.sigmoid(1.702 * g) * (u + 1)) @ experts[0][2].T)


# ---- configuration and description -----------------------------------------------------------------------------------------
def test_the_description_names_the_parts_and_shares_tensors_by_run_order():
    typed, spec = model_spec_from_config(vc.A)
    assert typed.taps == 4 and typed.layers[2].weights_of == 0
    assert len(spec.layers) == 3 and [e.layer for e in spec.run_order] == [0, 1, 0, 1, 2]
    first = spec.layers[0]
    assert first.block.kind == "prenorm" and first.mixer.kind == "conv_input" and first.mixer["inner"].kind == "lightning_attention"
    assert first.mixer.tensors["conv"] == "l0.canon1" and first.mixer.tensors["inner.norm"] == "l0.mix.norm"
    assert first.feed_forward.kind == "polynorm_mlp" and first.norms["mixer"].kind == "rms_scalar"
    second = spec.layers[1]
    inner = second.mixer["inner"]
    assert inner.kind == "attention" and inner["chunk"] == 24 and inner["sink"] and inner["output_gate"] and inner["position"] is None
    assert second.feed_forward["score"] == "softmax" and second.feed_forward["weight_on"] == "output"
    assert second.feed_forward["route_scale"] == 2.0 and second.feed_forward["limit"] == 1.5
    assert spec.layers[2].feed_forward is None and "l4.norm2" in spec.ignorable_tensors
    _, spec_d = model_spec_from_config(vc.D)
    assert spec_d.layers[0].mixer.kind == "attention" and spec_d.layers[2].mixer["chunk"] is None      # no convolution, no mask
    assert spec.head.tensors["weight"] == "head"


def test_every_run_of_a_layer_has_state_or_pages_of_its_own():
    _, _, r = runner_for("A", 64)
    b = r.model.bindings
    assert len(b) == 5 and len(r.model.group_keys) == 1
    assert b[0].k_pages is None and b[1].k_pages is not None and b[1].k_pages.data_ptr() != b[3].k_pages.data_ptr()
    assert b[0].state[""].shape == (4, 2, 16, 24) and b[0].state[""].data_ptr() != b[2].state[""].data_ptr()
    assert b[1].state["conv_inputs"].shape == (4, 3, 64) and b[4].state[""].shape == (4, 3, 8, 8)
    _, _, c = runner_for("C", 64)
    assert len(c.model.group_keys) == 0 and all(isinstance(x.state, torch.Tensor) or "conv_inputs" not in x.state for x in c.model.bindings)


@pytest.mark.parametrize("change,match", [
    (lambda c: c["layers"][0].__setitem__("type", "recurrent"), "no mixer of this design"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "routed"), "no feed-forward of this design"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("kv_heads", 3), "not a multiple"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("decay", [0.5]), "one number for each"),
    (lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 6), "more than"),
    (lambda c: c["layers"][1]["mlp"].pop("expert"), "requires layers\\[1\\].mlp.expert"),
    (lambda c: c["layers"][2].__setitem__("weights_of", 3), "tensors of its own"),
    (lambda c: c["layers"][2].__setitem__("weights_of", 1), "names other sizes"),
    (lambda c: c["canon"].__setitem__("taps", 0), "positive"),
    (lambda c: c["norm"].__setitem__("eps", 0), "positive"),
    (lambda c: c["layers"][1]["mixer"]["mask"].__setitem__("size", 0), "positive"),
])
def test_configurations_that_are_refused(change, match):
    cfg = copy.deepcopy(vc.A)
    change(cfg)
    with pytest.raises(ConfigError, match=match):
        model_spec_from_config(cfg)


def test_the_loader_names_what_does_not_fit():
    _, spec = model_spec_from_config(vc.A)
    shapes = {n: tuple(t.shape) for n, t in vc.weights(vc.A, 1).items()}
    check_tensors(spec, shapes)
    broken = dict(shapes)
    del broken["l1.mlp.e3.up"]
    del broken["l1.mix.sink"]
    broken["l0.norm1"] = (64,)                       # one number, not a vector
    broken["l2.mix.q"] = (32, 64)                    # a layer that runs another's tensors holds none
    broken["l4.mlp.up"] = (80, 64)                   # a layer without feed-forward holds none
    with pytest.raises(WeightsError) as err:
        check_tensors(spec, broken)
    assert err.value.missing == ["l1.mix.sink", "l1.mlp.e3.up"] and err.value.unexpected == ["l2.mix.q", "l4.mlp.up"]
    assert [w[0] for w in err.value.wrong_shape] == ["l0.norm1"]


# ---- the engine's logic -------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name,lengths", [("A", [5, 30, 61]), ("B", [45, 83]), ("C", [9, 50]), ("D", [100, 37]), ("E", [20, 51])])
@pytest.mark.parametrize("family", ["whole", "last", "portions", "mixed"])
def test_every_way_of_cutting_gives_the_plain_logits(tmp_path, name, lengths, family):
    vocab = vc.CONFIGS[name]["vocab"]
    requests = {f"r{i}": vc.random_ids(n, vocab, 70 + i) for i, n in enumerate(lengths)}
    steps = {"whole": tt.whole, "last": lambda r: tt.last_tokens_one_by_one(r, 9), "portions": tt.portions,
             "mixed": lambda r: tt.mixed(r, seed=4, decode_tail=6, refeed=[f"r{len(lengths) - 1}"])}[family](requests)
    steps = tt.number(steps)
    cfg, w64, runner = runner_for(name, tt.live_tokens_bound(steps, round_to=vc.PAGE_SIZES[name]))
    given_up = {}
    got = tt.run_in_process(runner, steps, vocab, str(tmp_path), given_up)
    for rid, feedings in given_up.items():          # ended half way and fed again: other pages, a cleared slot, the same logits
        again = got[rid][:len(feedings[0])]
        assert np.abs(feedings[0] - again).max() <= 1e-5 * np.abs(again).max()
    for rid, toks in requests.items():
        want = pv.forward(cfg, w64, toks)
        assert np.abs(got[rid] - want).max() <= 3e-5 * np.abs(want).max(), (family, rid)
    runner.cache.check_invariants()
    assert all(p.available == p.num_pages for p in runner.cache.pools)


def test_the_residual_stream_after_every_layer_run():
    cfg, w64, runner = runner_for("A", 64)
    seen = []
    for block in runner.model.blocks:
        def wrapped(ctx, x, binding, pending=None, _inner=block.forward):
            out = _inner(ctx, x, binding, pending)
            assert out is None
            seen.append(x.clone().numpy())
            return out
        block.forward = wrapped
    toks = vc.random_ids(29, cfg["vocab"], 5)
    runner.step([StepEntry("a", toks, [])])
    _, want = pv.forward(cfg, w64, toks, True)
    assert len(seen) == len(want) == 5
    for got, ref in zip(seen, want):
        assert np.abs(got - ref).max() <= 2e-5 * np.abs(ref).max()


def test_a_slot_that_is_used_again_starts_from_zero():
    """Two requests one after the other in the same state slot: the second finds neither the first's matrix nor its last inputs."""
    cfg, w64, runner = runner_for("C", 64)
    first, second = vc.random_ids(40, cfg["vocab"], 1), vc.random_ids(17, cfg["vocab"], 2)
    runner.step([StepEntry("a", first, [])])
    slot = runner.cache.slot("a")
    runner.free_request("a")
    got = runner.step([StepEntry("b", second, list(range(17)))]).numpy()
    assert runner.cache.slot("b") == slot
    want = pv.forward(cfg, w64, second)
    assert np.abs(got - want).max() <= 3e-5 * np.abs(want).max()


@pytest.mark.parametrize("name", ["A", "D"])
def test_greedy_generation_through_the_scheduler(tmp_path, name):
    cfg = vc.CONFIGS[name]
    tensors = vc.weights(cfg, 11)
    folder = vc.write_model(str(tmp_path / "m"), cfg, tensors)
    prompts = [vc.random_ids(n, cfg["vocab"], 20 + n) for n in (3, 26, 41)]
    want = [pv.greedy(cfg, vc.to_float64(tensors), p, 10) for p in prompts]
    for opts in (dict(num_blocks=64), dict(num_blocks=9, max_batched_tokens=12)):       # roomy; few pages and small portions
        engine = Engine(folder, dtype="float32", device="cpu", ctx=256, max_seqs=3, block_size=vc.PAGE_SIZES[name],
                        ops=ReferenceOps(), **{"max_batched_tokens": 32, **opts})
        assert engine.generate(prompts, SamplingParams(max_tokens=10)) == want
        engine.runner.cache.check_invariants()
