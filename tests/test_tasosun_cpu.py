"""Tasosun without a GPU: its configuration, its plan, and the engine's bookkeeping around it (cache
groups of unlike layers, windows that give pages back, runs of one layer with caches of their own,
the embedding added again before a pass) against the plain implementation, the kernels replaced by
the emulation of their contracts."""
import copy

import pytest
import torch

from helpers import max_live_tokens, replay_and_collect, trace_mixed, trace_portions, trace_tail, trace_whole
from kernel_emulation import EmulatedKernels
from plain import tasosun_plain
from tasosun_helpers import CONFIGS, compare_rows, plain_logits, requests_for, write_folder
from wllm_amd.architectures import TasosunConfig
from wllm_amd.config import ConfigError
from wllm_amd.engine import ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.kernels import ops
from wllm_amd.parts import build_model, load_model

LENGTHS = {"mixed": [70, 45, 90, 33, 58], "odd": [40, 66, 25, 51], "sharp": [80, 37, 64, 50], "wide": [30, 140, 21], "small": [75, 20, 130]}
FAMILIES = {"whole": trace_whole, "tail": trace_tail, "portions": trace_portions, "mixed": trace_mixed}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("tasosun")
    return {name: write_folder(name, str(root / name)) for name in CONFIGS}


@pytest.fixture(scope="module")
def exact(folders):
    return {name: plain_logits(folders[name], requests_for(name, LENGTHS[name]), torch.float32) for name in CONFIGS}


# ---- configuration and plan ------------------------------------------------------------------------
def test_the_plan_follows_the_file():
    cfg = TasosunConfig.from_dict(copy.deepcopy(CONFIGS["mixed"]["config"]))
    assert cfg.runs() == [(0, False), (1, False), (2, False), (1, True), (2, False), (1, True), (2, False)]
    model = build_model(copy.deepcopy(CONFIGS["mixed"]["config"]))
    plan = model.plan
    assert [(e.layer, e.adds_embedding) for e in plan.schedule] == cfg.runs()
    assert plan.layers[1].feed_forward is None and plan.layers[0].arrangement == "parallel"
    a = plan.layers[1].mixer
    assert (a.num_heads, a.num_kv_heads, a.head_dim, a.window, a.softcap) == (2, 1, 64, 40, 20.0)
    assert a.position.pairing == "interleaved" and a.position.rotary_dim == 16 and a.position.scaling_factor == 4.0
    assert a.values_are_keys and a.v_weight == "" and a.qk_norm_eps == 1e-5
    names = set(model.expected_tensors())
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.mix.q", "l0.mix.q.b", "l0.mix.k.b", "l0.mix.g", "l0.mix.o.b",
            "l0.mlp.gate", "l0.mlp.up", "l0.mlp.down", "l1.mix.o"} <= names
    assert not any(n.startswith("l1.mlp") or n.endswith("mix.v") for n in names)
    # every run that owns a cache has one of its own, also where two runs share a layer's weights
    assert sorted(model.cache_needs()) == list(range(7))


def test_runs_of_a_file_without_a_loop_and_of_a_loop_that_is_empty():
    assert TasosunConfig.from_dict(copy.deepcopy(CONFIGS["odd"]["config"])).runs() == [(0, False), (1, False)]
    assert TasosunConfig.from_dict(copy.deepcopy(CONFIGS["wide"]["config"])).runs() == [(0, False), (1, False)]
    assert TasosunConfig.from_dict(copy.deepcopy(CONFIGS["sharp"]["config"])).runs() == [
        (0, False), (1, False), (2, False), (0, True), (1, False), (2, False)]


@pytest.mark.parametrize("change, words", [
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mixer"].update(vdim=16), "vdim"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "even"),
    (lambda c: c["layers"][0].update(type="scan"), "attention"),
    (lambda c: c["layers"][0]["mlp"].update(kind="experts"), "dense"),
    (lambda c: c.update(loop={"start": 2, "stop": 1, "times": 2}), "loop"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_a_file_that_the_design_does_not_cover_is_refused(change, words):
    raw = copy.deepcopy(CONFIGS["mixed"]["config"])
    change(raw)
    with pytest.raises(ConfigError, match=words):
        TasosunConfig.from_dict(raw)


def test_a_key_that_is_not_read_is_named_in_a_warning():
    from wllm_amd.architectures.tasosun_config import UnknownConfigKey
    raw = copy.deepcopy(CONFIGS["mixed"]["config"])
    raw["note"] = "drawn by hand"
    raw["layers"][0]["mixer"]["sinks"] = 4
    with pytest.warns(UnknownConfigKey) as caught:
        cfg = TasosunConfig.from_dict(raw)
    assert any("sinks" in str(w.message) for w in caught) and any("note" in str(w.message) for w in caught)
    assert cfg.layers[0].attention.heads == 4


def test_the_written_config_reads_back(folders):
    raw = tasosun_plain.read_config(folders["sharp"])
    assert raw == CONFIGS["sharp"]["config"]
    assert TasosunConfig.from_dict(raw).to_dict() == raw


# ---- the engine around emulated kernels --------------------------------------------------------------
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_replay_matches_plain(folders, exact, name, family):
    requests = requests_for(name, LENGTHS[name])
    trace = FAMILIES[family](requests)
    page_size = CONFIGS[name]["page_size"]
    # the products of few rows leave three partial sums each, as the kernels of a decode step do
    with ops.use_backend(EmulatedKernels(splits=3 if family in ("tail", "mixed") else 1)) as emulated:
        model = load_model(folders[name], "float32", "cpu")
        pages = pages_for_max_tokens(max_live_tokens(trace), page_size)
        runner = ModelRunner.create(model, num_pages=pages, page_size=page_size, max_requests=4, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
        assert not runner.cache.requests
        assert all(g.pool.num_free == g.pool.num_pages for g in runner.cache.groups)
        assert emulated.calls.get("head_prepare", 0) > 0 and "rope_and_cache_write" not in emulated.calls
    assert len(got) == sum(len(t) for t in requests.values())
    compare_rows(got, exact[name], float32_relative=1e-4)


def test_a_window_gives_its_pages_back_while_the_request_runs(folders):
    """A request far longer than the pool: only windows make it fit, and freed pages (filled with NaN
    when they are given back) are used again by the same request."""
    name = "sharp"
    requests = requests_for(name, [400])
    reference = plain_logits(folders[name], requests, torch.float32)
    trace = trace_portions(requests, sizes=(16, 5, 2, 11, 1, 1, 1, 7, 3, 2, 9))
    with ops.use_backend(EmulatedKernels()):
        model = load_model(folders[name], "float32", "cpu")
        runner = ModelRunner.create(model, num_pages=6, page_size=16, max_requests=2, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
    compare_rows(got, reference, float32_relative=1e-4)


def test_the_sharp_model_shows_a_key_lost_at_a_windows_edge(folders):
    """The plain implementation with every window one key shorter, or one longer, is far from itself: what
    the comparisons with it hold is that the edge key is there and the next one is not."""
    raw = tasosun_plain.read_config(folders["sharp"])
    w = tasosun_plain.read_weights(folders["sharp"], torch.float64)
    tokens = requests_for("sharp", [80])["q0"]
    right = tasosun_plain.forward(raw, w, tokens)
    for step in (-1, 1):
        other = copy.deepcopy(raw)
        for entry in other["layers"]:
            entry["mixer"]["mask"]["size"] += step
        wrong = tasosun_plain.forward(other, w, tokens)
        far = (wrong - right).pow(2).mean(-1).sqrt() / right.pow(2).mean(-1).sqrt()
        assert (far[40:] > 1e-2).float().mean() > 0.8, "most rows past the windows move by more than a hundredth"
