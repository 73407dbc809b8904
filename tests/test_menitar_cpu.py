"""Menitar on the CPU: configuration, the model's description, and the engine's own logic (run order with looped
layers, caches a pass, batches, pages, portions, scheduler) with the plain kernels of tests/reference_ops.py in place
of the HIP library, against the plain implementation of tests/plain_menitar.py."""
import copy

import numpy as np
import pytest
import torch

import menitar_configs as mc
import plain_menitar
import trace_tools as tt
from reference_ops import ReferenceOps
from fllm_amd import Engine, SamplingParams
from fllm_amd.config.spec import ConfigError
from fllm_amd.engine import ModelRunner, StepEntry
from fllm_amd.registry import model_spec_from_config
from fllm_amd.weights.loader import WeightsError, check_tensors


def runner_for(name, max_tokens, seed=3, **kw):
    cfg = mc.CONFIGS[name]
    _, spec = model_spec_from_config(cfg)
    tensors = mc.weights(cfg, seed)
    r = ModelRunner(spec, dict(tensors), dtype="float32", device="cpu", page_size=mc.PAGE_SIZES[name], max_tokens=max_tokens,
                    max_requests=4, max_context=512, ops=ReferenceOps(), **kw)
    return cfg, mc.to_float64(tensors), r


def test_the_description_follows_the_configuration():
    typed, spec = model_spec_from_config(mc.P)
    assert typed.loop == (0, 2, 3) and typed.layers[1].mlp is None and typed.layers[0].mixer.chunk == 24
    assert [e.layer for e in spec.run_order] == [0, 1, 0, 1, 0, 1, 2]
    enters = [(i, e.before["row"], e.before["add_embedding"]) for i, e in enumerate(spec.run_order) if e.before is not None]
    assert enters == [(0, 0, False), (2, 1, True), (4, 2, True)]
    assert spec.layers[1].feed_forward is None and "feed_forward" not in spec.layers[1].norms
    assert spec.head.tensors["weight"] == spec.embedding.tensors["weight"] == "embed"
    _, spec_q = model_spec_from_config(mc.Q)
    assert all(e.before is None for e in spec_q.run_order) and len(spec_q.run_order) == 2
    _, spec_s = model_spec_from_config(mc.S)
    assert [e.layer for e in spec_s.run_order] == [0, 1, 2, 1, 2]


def test_every_pass_of_a_looped_layer_has_a_cache_of_its_own():
    _, _, r = runner_for("S", 64)
    assert len(r.model.bindings) == 5
    assert len(r.model.group_keys) == 2                     # two geometries
    k_of = [b.k_pages.data_ptr() for b in r.model.bindings]
    assert len(set(k_of)) == 5


@pytest.mark.parametrize("change,match", [
    (lambda c: c["layers"][0].__setitem__("type", "recurrent"), "no mixer of this design"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "routed"), "no feed-forward of this design"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 3), "not a multiple"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 7), "even"),
    (lambda c: c["loop"].__setitem__("stop", 9), "must name a run"),
    (lambda c: c.pop("width"), "requires width"),
    (lambda c: c["norm"].__setitem__("eps", 0), "positive"),
    (lambda c: c["layers"][0]["mixer"]["mask"].__setitem__("size", 0), "positive"),
])
def test_configurations_that_are_refused(change, match):
    cfg = copy.deepcopy(mc.P)
    change(cfg)
    with pytest.raises(ConfigError, match=match):
        model_spec_from_config(cfg)


def test_the_loader_names_what_does_not_fit():
    _, spec = model_spec_from_config(mc.P)
    shapes = {n: tuple(t.shape) for n, t in mc.weights(mc.P, 1).items()}
    check_tensors(spec, shapes)
    broken = dict(shapes)
    del broken["loop.step"]
    broken["l0.mix.talk"] = (4, 3)
    broken["l1.mlp.gate"] = (80, 64)                 # a layer without feed-forward holds none
    with pytest.raises(WeightsError) as err:
        check_tensors(spec, broken)
    assert err.value.missing == ["loop.step"] and err.value.unexpected == ["l1.mlp.gate"]
    assert [w[0] for w in err.value.wrong_shape] == ["l0.mix.talk"]


@pytest.mark.parametrize("name,lengths", [("P", [5, 30, 61]), ("Q", [45, 83]), ("R", [9, 50]), ("S", [100, 37]), ("U", [20, 51])])
@pytest.mark.parametrize("family", ["whole", "last", "portions", "mixed"])
def test_every_way_of_cutting_gives_the_plain_logits(tmp_path, name, lengths, family):
    vocab = mc.CONFIGS[name]["vocab"]
    requests = {f"r{i}": mc.random_ids(n, vocab, 70 + i) for i, n in enumerate(lengths)}
    steps = {"whole": tt.whole, "last": lambda r: tt.last_tokens_one_by_one(r, 9), "portions": tt.portions,
             "mixed": lambda r: tt.mixed(r, seed=4, decode_tail=6, refeed=[f"r{len(lengths) - 1}"])}[family](requests)
    steps = tt.number(steps)
    cfg, w64, runner = runner_for(name, tt.live_tokens_bound(steps, round_to=mc.PAGE_SIZES[name]))
    given_up = {}
    got = tt.run_in_process(runner, steps, vocab, str(tmp_path), given_up)
    for rid, feedings in given_up.items():          # ended half way and fed again: other pages, the same logits
        assert np.array_equal(feedings[0], got[rid][:len(feedings[0])])
    for rid, toks in requests.items():
        want = plain_menitar.forward(cfg, w64, toks)
        assert np.abs(got[rid] - want).max() <= 3e-5 * np.abs(want).max(), (family, rid)
    runner.cache.check_invariants()
    assert all(p.available == p.num_pages for p in runner.cache.pools)


def test_the_residual_stream_after_every_layer_run():
    cfg, w64, runner = runner_for("P", 64)
    seen = []
    for block in runner.model.blocks:
        def wrapped(ctx, x, binding, _inner=block.forward):
            _inner(ctx, x, binding)
            seen.append(x.clone().numpy())
        block.forward = wrapped
    toks = mc.random_ids(29, cfg["vocab"], 5)
    runner.step([StepEntry("a", toks, [])])
    want = []
    plain_menitar.forward(cfg, w64, toks, want)
    assert len(seen) == len(want) == 7
    for got, ref in zip(seen, want):
        assert np.abs(got - ref).max() <= 2e-5 * np.abs(ref).max()


@pytest.mark.parametrize("name", ["P", "S"])
def test_greedy_generation_through_the_scheduler(tmp_path, name):
    cfg = mc.CONFIGS[name]
    tensors = mc.weights(cfg, 11)
    folder = mc.write_model(str(tmp_path / "m"), cfg, tensors)
    prompts = [mc.random_ids(n, cfg["vocab"], 20 + n) for n in (3, 26, 41)]
    want = [plain_menitar.greedy(cfg, mc.to_float64(tensors), p, 10) for p in prompts]
    for opts in (dict(num_blocks=64), dict(num_blocks=9, max_batched_tokens=12)):       # roomy; few pages and small portions
        engine = Engine(folder, dtype="float32", device="cpu", ctx=256, max_seqs=3, block_size=mc.PAGE_SIZES[name],
                        ops=ReferenceOps(), **{"max_batched_tokens": 32, **opts})
        assert engine.generate(prompts, SamplingParams(max_tokens=10)) == want
        engine.runner.cache.check_invariants()
