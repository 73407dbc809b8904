"""Purivik on the CPU: configuration, the model's description, and the engine's own logic (run order with looped layers,
caches a pass, batches, pages, portions, scheduler) with the plain kernels of tests/reference_ops.py in place of the HIP
library, against the plain implementation of tests/plain_purivik.py; and that plain implementation's mechanisms one by one."""
import copy

import numpy as np
import pytest
import torch

import plain_purivik
import purivik_configs as pc
import trace_tools as tt
from reference_ops import ReferenceOps
from fllm_amd import Engine, SamplingParams
from fllm_amd.config.spec import ConfigError
from fllm_amd.engine import ModelRunner, StepEntry
from fllm_amd.registry import model_spec_from_config
from fllm_amd.weights.loader import WeightsError, check_tensors


def runner_for(name, max_tokens, seed=3, **kw):
    cfg = pc.CONFIGS[name]
    _, spec = model_spec_from_config(cfg)
    tensors = pc.weights(cfg, seed)
    r = ModelRunner(spec, dict(tensors), dtype="float32", device="cpu", page_size=pc.PAGE_SIZES[name], max_tokens=max_tokens,
                    max_requests=4, max_context=512, ops=ReferenceOps(), **kw)
    return cfg, pc.to_float64(tensors), r


# ---- the plain implementation's mechanisms, each alone ----------------------------------------------------------------
def test_plain_frequency_bands():
    rot = {"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 40}}
    f = plain_purivik.rotary_frequencies(rot)
    plainf = np.array([100.0 ** (-2.0 * i / 8) for i in range(4)])
    wave = 2 * np.pi / plainf                      # 6.3, 19.9, 62.8, 198.7 against the edges 10 and 40
    assert wave[0] < 10 and 10 < wave[1] < 40 and wave[2] > 40
    assert f[0] == plainf[0] and np.isclose(f[2], plainf[2] / 4) and np.isclose(f[3], plainf[3] / 4)
    t = (40 / wave[1] - 1.0) / 3.0
    assert np.isclose(f[1], (1 - t) * plainf[1] / 4 + t * plainf[1]) and plainf[1] / 4 < f[1] < plainf[1]
    assert np.array_equal(plain_purivik.rotary_frequencies({"dims": 8, "base": 100.0}), plainf)


def test_plain_rotation_keeps_lengths_and_the_lanes_behind():
    x = np.random.default_rng(0).normal(size=(5, 2, 12))
    y = plain_purivik.rotate(x, {"dims": 8, "base": 50.0}, [0, 1, 2, 30, 400])
    assert np.array_equal(y[0], x[0]) and np.array_equal(y[..., 8:], x[..., 8:])
    assert np.allclose((y[..., :8] ** 2).sum(-1), (x[..., :8] ** 2).sum(-1))
    # lane 1 turns with lane 5 (i + dims/2), by position * f_1
    a = 30 * 50.0 ** (-2.0 / 8)
    assert np.isclose(y[3, 0, 1], x[3, 0, 1] * np.cos(a) - x[3, 0, 5] * np.sin(a))
    assert np.isclose(y[3, 0, 5], x[3, 0, 5] * np.cos(a) + x[3, 0, 1] * np.sin(a))


def test_plain_mask_counts_blocks_from_position_zero():
    see = plain_purivik.visible(10, {"size": 4})
    assert see[3].tolist() == [True] * 4 + [False] * 6 and see[4].tolist() == [False] * 4 + [True] + [False] * 5
    assert see[9].tolist() == [False] * 8 + [True] * 2
    assert plain_purivik.visible(5, None)[4].all()


def test_plain_router_and_where_the_score_goes():
    rng = np.random.default_rng(1)
    W = {"m.router": rng.normal(size=(4, 6))}
    for e in range(4):
        W.update({f"m.e{e}.gate": rng.normal(size=(3, 6)), f"m.e{e}.up": rng.normal(size=(3, 6)), f"m.e{e}.down": rng.normal(size=(6, 3))})
    h = rng.normal(size=(2, 6))
    mlp = {"router": {"experts": 4, "top": 2}}
    picks, scores = plain_purivik.router(W, "m.", mlp, h)
    z = h @ W["m.router"].T
    assert picks[0].tolist() == np.argsort(-z[0])[:2].tolist() and np.allclose(scores[0], 1 / (1 + np.exp(-z[0][picks[0]])))
    assert (scores < 1).all() and scores.sum(1).max() != 1.0           # sigmoids, not renormalized
    out = plain_purivik.experts_ff(W, "m.", mlp, h)
    by_hand = sum(plain_purivik.expert(W, f"m.e{e}.", s * h[1]) for e, s in zip(picks[1], scores[1]))
    assert np.allclose(out[1], by_hand)
    scaled_after = sum(s * plain_purivik.expert(W, f"m.e{e}.", h[1]) for e, s in zip(picks[1], scores[1]))
    assert not np.allclose(out[1], scaled_after)                      # the expert is not linear: the place of the score matters


def test_plain_dense_layer_clamps_both_operands():
    W = {"m.gate": np.array([[5.0], [-5.0]]), "m.up": np.array([[9.0], [-9.0]]), "m.down": np.eye(2)}
    y = plain_purivik.dense_ff(W, "m.", {"limit": 2.0}, np.array([[1.0]]))
    g = np.array([2.0, -5.0])                      # the gate is bounded above only
    assert np.allclose(y[0], g / (1 + np.exp(-1.702 * g)) * (np.array([2.0, -2.0]) + 1))


# ---- configuration and description ------------------------------------------------------------------------------------
def test_the_description_follows_the_configuration():
    typed, spec = model_spec_from_config(pc.A)
    assert typed.loop == (1, 3, 3) and typed.layers[2].mlp is None and typed.layers[0].mixer.chunk == 24
    assert typed.layers[1].mlp.kind == "moe" and (typed.layers[1].mlp.experts, typed.layers[1].mlp.top) == (5, 2)
    assert typed.layers[0].mixer.rot_scaling.original == 64 and typed.residual_mult == 0.6
    assert [e.layer for e in spec.run_order] == [0, 1, 2, 1, 2, 1, 2]
    assert [i for i, e in enumerate(spec.run_order) if e.before is not None] == [3, 5]      # every pass but the first
    assert all(e.before["add_embedding"] and not e.before.tensors for e in spec.run_order if e.before is not None)
    assert spec.layers[2].feed_forward is None and "feed_forward" not in spec.layers[2].norms
    assert spec.layers[0].block.kind == "sandwich" and spec.layers[0].block.tensors == {"mixer_scale": "l0.ls1", "feed_forward_scale": "l0.ls2"}
    assert spec.layers[1].feed_forward.kind == "routed_experts" and spec.layers[1].feed_forward.tensors["down_4"] == "l1.mlp.e4.down"
    assert spec.layers[0].mixer.kind == "attention" and spec.layers[0].mixer["value_head_dim"] == 16
    assert spec.layers[0].mixer["position"]["scaling"] == "llama3"
    assert spec.head.tensors["weight"] == spec.embedding.tensors["weight"] == "embed" and spec.head.get("scale", 1.0) == 1.0
    _, spec_b = model_spec_from_config(pc.B)
    assert all(e.before is None for e in spec_b.run_order) and len(spec_b.run_order) == 2
    assert spec_b.layers[0].mixer["position"]["scaling"] == "none"
    _, spec_c = model_spec_from_config(pc.C)
    assert spec_c.layers[0].mixer["position"] is None and spec_c.layers[0].mixer["chunk"] is None
    assert all(e.before is None for e in spec_c.run_order)            # a loop of one pass adds nothing


def test_every_pass_of_a_looped_layer_has_a_cache_of_its_own():
    _, _, r = runner_for("D", 64)
    assert len(r.model.bindings) == 5
    assert len(r.model.group_keys) == 2                     # two geometries
    assert len({b.k_pages.data_ptr() for b in r.model.bindings}) == 5
    assert r.model.bindings[1].v_pages.shape[-2] == 32 and r.model.bindings[0].v_pages.shape[-2] == 64


@pytest.mark.parametrize("change,match", [
    (lambda c: c["layers"][0].__setitem__("type", "recurrent"), "no mixer of this design"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "routed"), "no feed-forward of this design"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 3), "not a multiple"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 7), "even"),
    (lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].__setitem__("low", 5.0), "low < high"),
    (lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 6), "more than"),
    (lambda c: c["layers"][1]["mlp"].pop("expert"), "requires layers\\[1\\].mlp.expert"),
    (lambda c: c["loop"].__setitem__("stop", 9), "must name a run"),
    (lambda c: c.pop("residual_mult"), "requires residual_mult"),
    (lambda c: c["norm"].__setitem__("eps", 0), "positive"),
    (lambda c: c["layers"][0]["mixer"]["mask"].__setitem__("size", 0), "positive"),
])
def test_configurations_that_are_refused(change, match):
    cfg = copy.deepcopy(pc.A)
    change(cfg)
    with pytest.raises(ConfigError, match=match):
        model_spec_from_config(cfg)


def test_the_loader_names_what_does_not_fit():
    _, spec = model_spec_from_config(pc.A)
    shapes = {n: tuple(t.shape) for n, t in pc.weights(pc.A, 1).items()}
    check_tensors(spec, shapes)
    broken = dict(shapes)
    del broken["l1.mlp.e3.up"]
    broken["l0.mix.v"] = (64, 64)                    # values are 2 heads of 16 lanes here, not of 32
    broken["l2.mlp.gate"] = (80, 64)                 # a layer without feed-forward holds none
    broken["l1.mlp.e5.gate"] = (24, 64)              # a sixth expert of five
    with pytest.raises(WeightsError) as err:
        check_tensors(spec, broken)
    assert err.value.missing == ["l1.mlp.e3.up"] and err.value.unexpected == ["l1.mlp.e5.gate", "l2.mlp.gate"]
    assert [w[0] for w in err.value.wrong_shape] == ["l0.mix.v"]


# ---- the engine's logic -------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name,lengths", [("A", [5, 30, 61]), ("B", [45, 83]), ("C", [9, 50]), ("D", [100, 37]), ("E", [20, 51]),
                                          ("F", [60, 23]), ("G", [170, 40])])
@pytest.mark.parametrize("family", ["whole", "last", "portions", "mixed"])
def test_every_way_of_cutting_gives_the_plain_logits(tmp_path, name, lengths, family):
    vocab = pc.CONFIGS[name]["vocab"]
    requests = {f"r{i}": pc.random_ids(n, vocab, 70 + i) for i, n in enumerate(lengths)}
    steps = {"whole": tt.whole, "last": lambda r: tt.last_tokens_one_by_one(r, 9), "portions": tt.portions,
             "mixed": lambda r: tt.mixed(r, seed=4, decode_tail=6, refeed=[f"r{len(lengths) - 1}"])}[family](requests)
    steps = tt.number(steps)
    cfg, w64, runner = runner_for(name, tt.live_tokens_bound(steps, round_to=pc.PAGE_SIZES[name]))
    given_up = {}
    got = tt.run_in_process(runner, steps, vocab, str(tmp_path), given_up)
    for rid, feedings in given_up.items():          # ended half way and fed again: other pages, the same logits (the stand-in
        again = got[rid][:len(feedings[0])]         # kernels' float64 products round differently by batch shape; the HIP
        assert np.abs(feedings[0] - again).max() <= 1e-5 * np.abs(again).max()      # kernels are compared bit for bit)
    for rid, toks in requests.items():
        want = plain_purivik.forward(cfg, w64, toks)
        assert np.abs(got[rid] - want).max() <= 3e-5 * np.abs(want).max(), (family, rid)
    runner.cache.check_invariants()
    assert all(p.available == p.num_pages for p in runner.cache.pools)


def test_the_residual_stream_after_every_layer_run():
    cfg, w64, runner = runner_for("A", 64)
    seen = []
    for block in runner.model.blocks:
        def wrapped(ctx, x, binding, _inner=block.forward):
            _inner(ctx, x, binding)
            seen.append(x.clone().numpy())
        block.forward = wrapped
    toks = pc.random_ids(29, cfg["vocab"], 5)
    runner.step([StepEntry("a", toks, [])])
    want = []
    plain_purivik.forward(cfg, w64, toks, want)
    assert len(seen) == len(want) == 7
    for got, ref in zip(seen, want):
        assert np.abs(got - ref).max() <= 2e-5 * np.abs(ref).max()


def test_a_block_takes_parts_that_only_add_to_the_stream():
    """The sandwich arrangement around a part that knows nothing of stored branches: it adds into a zeroed stand-in."""
    cfg, w64, runner = runner_for("B", 64)
    for block in runner.model.blocks:
        for part in (block.mixer, block.feed_forward):
            part.stores_branch = False
            inner = part.forward
            part.forward = (lambda ctx, h, residual, *rest, _inner=inner, **kw: _inner(ctx, h, residual, *rest))
    toks = pc.random_ids(21, cfg["vocab"], 6)
    got = runner.step([StepEntry("a", toks, list(range(21)))]).numpy()
    want = plain_purivik.forward(cfg, w64, toks)
    assert np.abs(got - want).max() <= 3e-5 * np.abs(want).max()


@pytest.mark.parametrize("name", ["A", "D"])
def test_greedy_generation_through_the_scheduler(tmp_path, name):
    cfg = pc.CONFIGS[name]
    tensors = pc.weights(cfg, 11)
    folder = pc.write_model(str(tmp_path / "m"), cfg, tensors)
    prompts = [pc.random_ids(n, cfg["vocab"], 20 + n) for n in (3, 26, 41)]
    want = [plain_purivik.greedy(cfg, pc.to_float64(tensors), p, 10) for p in prompts]
    for opts in (dict(num_blocks=64), dict(num_blocks=9, max_batched_tokens=12)):       # roomy; few pages and small portions
        engine = Engine(folder, dtype="float32", device="cpu", ctx=256, max_seqs=3, block_size=pc.PAGE_SIZES[name],
                        ops=ReferenceOps(), **{"max_batched_tokens": 32, **opts})
        assert engine.generate(prompts, SamplingParams(max_tokens=10)) == want
        engine.runner.cache.check_invariants()
