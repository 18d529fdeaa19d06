"""Tokuvik without a GPU: its configuration, its plan, the plain implementation's own mechanisms, and the
engine's bookkeeping around it (cache groups of unlike layers, chunks that give pages back, a layer that
reads another's cache, state slots that are zeroed and used again) against the plain implementation, the
kernels replaced by the emulation of their contracts."""
import copy

import pytest
import torch

from helpers import max_live_tokens, replay_and_collect, trace_mixed, trace_portions, trace_tail, trace_whole
from kernel_emulation import EmulatedKernels
from plain import tokuvik_plain as plain
from tokuvik_helpers import (CONFIGS, compare_rows, plain_logits, random_config, read_folder, requests_for, write_folder)
from wllm_amd.architectures import TokuvikConfig
from wllm_amd.cache.manager import CacheNeed
from wllm_amd.config import ConfigError
from wllm_amd.engine import ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.kernels import ops
from wllm_amd.parts import build_model, load_model

LENGTHS = {"trio": [70, 45, 90, 33, 58], "odd": [40, 66, 25, 51], "sharp": [80, 37, 64, 50]}
FAMILIES = {"whole": trace_whole, "tail": trace_tail, "portions": trace_portions, "mixed": trace_mixed}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("tokuvik")
    return {name: write_folder(name, str(root / name)) for name in CONFIGS}


@pytest.fixture(scope="module")
def exact(folders):
    return {name: plain_logits(folders[name], requests_for(name, LENGTHS[name]), torch.float64) for name in CONFIGS}


# ---- configuration and plan ------------------------------------------------------------------------
def test_the_plan_follows_the_file():
    model = build_model(copy.deepcopy(CONFIGS["trio"]["config"]))
    plan = model.plan
    assert [type(b.mixer).__name__ for b in plan.layers] == [
        "AttentionSpec", "LatentAttentionSpec", "StateSpaceSpec", "AttentionSpec", "StateSpaceSpec"]
    assert [e.reads_cache_of for e in plan.schedule] == [None, None, None, 0, None]
    a, shared = plan.layers[0].mixer, plan.layers[3].mixer
    assert (a.num_heads, a.num_kv_heads, a.head_dim, a.value_dim, a.chunk, a.release_chunk) == (4, 2, 32, 16, 24, 24)
    assert a.gate_per_head and a.position.kind == "none" and a.q_norm_weight == "l0.mix.q.norm"
    assert not shared.owns_cache and shared.k_weight == "" and shared.k_norm_weight is None
    assert plan.layers[2].feed_forward is None and plan.layers[2].feed_forward_norm is None
    assert plan.layers[0].arrangement == "sandwich" and plan.layers[0].mixer_norm.kind == "layer"
    assert plan.layers[1].side.offset == 8 and plan.layers[1].side.norm.kind == "rms"
    names = set(model.expected_tensors())
    assert {"embed", "side.embed", "final.norm", "l0.norm1b", "l0.norm2b", "l0.mix.q.norm", "l0.mix.k.norm", "l0.mix.g",
            "l1.mix.dq.norm", "l1.mix.uk", "l1.mix.sink", "l2.mix.conv.b", "l2.mix.A_log", "l2.mix.D", "l4.side.proj"} <= names
    assert not any(n.startswith(("l3.mix.k", "l3.mix.v", "l2.mlp", "l2.norm2")) for n in names) and "head" not in names
    # the cache: the run that reads another's has none of its own; the recurrent layers have state rows
    assert sorted(model.cache_needs()) == [0, 1] and sorted(model.state_shapes()) == [2, 4]
    assert model.state_shapes()[2] == (4 * 16 * 16 + 3 * (64 + 2 * 2 * 16),)


def test_a_cache_read_under_another_mask_keeps_everything():
    needs = build_model(copy.deepcopy(CONFIGS["odd"]["config"])).cache_needs()
    assert needs[0] == CacheNeed(3, 28, None, None)          # chunks of 7 and of 19 read it
    assert needs[4] == CacheNeed(1, 12, None, None)          # no mask at all
    assert build_model(copy.deepcopy(CONFIGS["sharp"]["config"])).cache_needs()[0].chunk == 16


@pytest.mark.parametrize("change, words", [
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0].update(type="scan"), "mixers"),
    (lambda c: c["layers"][0]["mlp"].update(kind="experts"), "dense"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=3), "earlier"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=1), "earlier"),
    (lambda c: c["layers"][3]["mixer"].update(vdim=32), "equal"),
    (lambda c: c["layers"][2]["mixer"].update(groups=3), "multiple"),
    (lambda c: c["layers"][2]["mixer"].update(norm_groups=5), "divide"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_a_file_that_the_design_does_not_cover_is_refused(change, words):
    raw = copy.deepcopy(CONFIGS["trio"]["config"])
    change(raw)
    with pytest.raises(ConfigError, match=words):
        TokuvikConfig.from_dict(raw)


def test_a_key_that_is_not_read_is_named_in_a_warning():
    from wllm_amd.architectures.tasosun_config import UnknownConfigKey
    raw = copy.deepcopy(CONFIGS["trio"]["config"])
    raw["layers"][0]["mixer"]["rot"] = {"dims": 8}
    with pytest.warns(UnknownConfigKey, match="rot"):
        TokuvikConfig.from_dict(raw)


def test_the_written_config_reads_back(folders):
    raw, _ = read_folder(folders["odd"])
    assert raw == CONFIGS["odd"]["config"]
    cfg = TokuvikConfig.from_dict(raw)
    assert cfg.to_dict() == raw and cfg.side_dim is None
    again = TokuvikConfig(cfg.vocab, cfg.width, cfg.norm_eps, cfg.side_dim, cfg.layers).to_dict()
    assert again == raw


# ---- the plain implementation's mechanisms, each against a second way of computing it ----------------
def test_chunk_mask_edges():
    seen = plain.chunk_mask(12, 5)
    assert seen[4, 0] and seen[4, 4] and not seen[5, 4] and seen[5, 5] and not seen[9, 4] and seen[9, 5] and not seen[3, 4]
    assert seen[11, 10] and not seen[11, 9]
    assert plain.chunk_mask(4, None).tolist() == torch.ones(4, 4).tril().bool().tolist()
    assert plain.chunk_mask(6, 1).tolist() == torch.eye(6).bool().tolist()


def test_a_sink_takes_its_share_and_gives_nothing():
    scores = torch.tensor([[[0.0, 1.0], [2.0, -1.0]]], dtype=torch.float64)
    seen = torch.tensor([[True, False], [True, True]])
    w = plain.softmax_with_sink(scores, seen, torch.tensor([0.5], dtype=torch.float64))
    e = torch.exp(torch.tensor([0.0, 0.5, 2.0, -1.0], dtype=torch.float64))
    assert torch.allclose(w[0, 0], torch.stack([e[0] / (e[0] + e[1]), torch.tensor(0.0, dtype=torch.float64)]))
    assert torch.allclose(w[0, 1], torch.stack([e[2], e[3]]) / (e[2] + e[3] + e[1]))
    assert torch.allclose(plain.softmax_with_sink(scores, seen).sum(-1), torch.ones(1, 2, dtype=torch.float64))


def test_the_convolution_starts_from_zeros_and_ends_on_the_current_token():
    u = torch.arange(1.0, 6.0, dtype=torch.float64)[:, None] * torch.tensor([[1.0, 10.0]], dtype=torch.float64)
    w = torch.tensor([[0.0, 0.0, 1.0], [1.0, 0.0, 0.0]], dtype=torch.float64)      # the current token; two back
    out = plain.causal_conv(u, w, torch.tensor([0.5, 0.0], dtype=torch.float64))
    assert out[:, 0].tolist() == [1.5, 2.5, 3.5, 4.5, 5.5] and out[:, 1].tolist() == [0.0, 0.0, 10.0, 20.0, 30.0]


def test_the_recurrence_is_the_sum_it_unrolls_to():
    """y_t = sum_s (prod of the decays after s) dt_s (C_t . B_s) x_s + D x_t, written out for one head."""
    torch.manual_seed(0)
    t, n, p = 6, 3, 2
    mixer = {"heads": 1, "vdim": p, "state": n, "groups": 1, "conv": 1, "norm_groups": 1}
    width = 4
    w = {"in": torch.randn(2 * p + 2 * n + 1, width), "conv": torch.ones(p + 2 * n, 1), "conv.b": torch.zeros(p + 2 * n),
         "dt_bias": torch.tensor([0.2]), "A_log": torch.tensor([-0.3]), "D": torch.tensor([0.7]),
         "norm": torch.ones(p), "o": torch.eye(p, p)}
    w = {"m." + k: v.double() for k, v in w.items()}
    h = torch.randn(t, width, dtype=torch.float64)
    got = plain.mamba2_mixer(h, w, "m.", mixer, 1e-6)
    row = h @ w["m.in"].T
    z, xbc, dt = row[:, :p], plain.silu(row[:, p:2 * p + 2 * n]), plain.softplus(row[:, -1] + 0.2)
    x, b, c = xbc[:, :p], xbc[:, p:p + n], xbc[:, p + n:]
    decay = torch.exp(-torch.exp(torch.tensor(-0.3, dtype=torch.float64)) * dt)
    ys = []
    for i in range(t):
        y = 0.7 * x[i]
        for s in range(i + 1):
            y = y + decay[s + 1:i + 1].prod() * dt[s] * (c[i] @ b[s]) * x[s]
        ys.append(y)
    y = torch.stack(ys) * plain.silu(z)
    want = y / torch.sqrt((y * y).mean(-1, keepdim=True) + 1e-6)
    assert torch.allclose(got, want, atol=1e-12)


def test_the_sharp_model_shows_a_key_lost_at_a_chunks_edge_and_a_sink_left_out(folders):
    raw, w = read_folder(folders["sharp"])
    tokens = requests_for("sharp", [80])["q0"]
    right = plain.forward(raw, w, tokens)
    for step in (-1, 1):
        other = copy.deepcopy(raw)
        for entry in other["layers"]:
            if "mask" in entry["mixer"]:
                entry["mixer"]["mask"]["size"] += step
        wrong = plain.forward(other, w, tokens)
        far = (wrong - right).pow(2).mean(-1).sqrt() / right.pow(2).mean(-1).sqrt()
        assert (far[24:] > 1e-2).float().mean() > 0.8, "most rows past the first chunks move by more than a hundredth"
    no_sink = {k: (v - 30.0 if k.endswith(".sink") else v) for k, v in w.items()}
    far = (plain.forward(raw, no_sink, tokens) - right).pow(2).mean(-1).sqrt() / right.pow(2).mean(-1).sqrt()
    assert (far > 1e-2).float().mean() > 0.8


# ---- the engine around emulated kernels --------------------------------------------------------------
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_replay_matches_plain(folders, exact, name, family):
    requests = requests_for(name, LENGTHS[name])
    trace = FAMILIES[family](requests)
    page_size = CONFIGS[name]["page_size"]
    with ops.use_backend(EmulatedKernels(splits=3 if family in ("tail", "mixed") else 1)) as emulated:
        model = load_model(folders[name], "float32", "cpu")
        pages = pages_for_max_tokens(max_live_tokens(trace), page_size)
        runner = ModelRunner.create(model, num_pages=pages, page_size=page_size, max_requests=4, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
        assert not runner.cache.requests
        assert all(g.pool.num_free == g.pool.num_pages for g in runner.cache.groups)
        assert emulated.calls.get("ssm_scan", 0) > 0 and emulated.calls.get("norm_add", 0) > 0
    assert len(got) == sum(len(t) for t in requests.values())
    # (the sharp model multiplies float32 rounding by some hundred; a lost key moves a row by more than a hundredth)
    compare_rows(got, exact[name], relative=5e-4 if name == "sharp" else 5e-5)


def test_chunks_give_their_pages_back_while_the_request_runs(folders):
    """A request far longer than the attention's pool: only the chunks make it fit, and freed pages (filled
    with NaN when they are given back) are used again by the same request."""
    raw = copy.deepcopy(CONFIGS["sharp"])
    raw["config"]["layers"] = [raw["config"]["layers"][i] for i in (0, 3, 4)]      # the chunked layers and a recurrent one
    raw["config"]["layers"][1]["mixer"]["kv_from"] = 0
    import tempfile
    with tempfile.TemporaryDirectory() as folder:
        write_folder(raw, folder)
        requests = requests_for(raw, [300])
        reference = plain_logits(folder, requests, torch.float64)
        trace = trace_portions(requests, sizes=(16, 5, 2, 11, 1, 1, 1, 7, 3, 2, 9))
        with ops.use_backend(EmulatedKernels()):
            model = load_model(folder, "float32", "cpu")
            runner = ModelRunner.create(model, num_pages=4, page_size=16, max_requests=2, poison_freed_pages=True)
            got = replay_and_collect(TraceReplayer(runner), trace)
            runner.cache.check()
    compare_rows(got, reference, relative=5e-4)


def test_a_state_slot_that_is_used_again_starts_from_zero(folders):
    """Two slots, five requests one after the other and side by side: a request's recurrence must not
    begin where the slot's last holder ended."""
    name = "trio"
    requests = requests_for(name, [30, 21, 17, 26, 12])
    reference = plain_logits(folders[name], requests, torch.float64)
    trace = trace_mixed(requests, seed=3, live=2)
    with ops.use_backend(EmulatedKernels()):
        model = load_model(folders[name], "float32", "cpu")
        runner = ModelRunner.create(model, num_pages=12, page_size=16, max_requests=2, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
    compare_rows(got, reference, relative=5e-4)


@pytest.mark.parametrize("seed", range(6))
def test_configurations_drawn_at_random(tmp_path, seed):
    c = random_config(100 + seed)
    folder = write_folder(c, str(tmp_path / "m"))
    requests = requests_for(c, [37, 18, 50])
    reference = plain_logits(folder, requests, torch.float64)
    trace = trace_mixed(requests, seed=seed, live=3)
    with ops.use_backend(EmulatedKernels()):
        model = load_model(folder, "float32", "cpu")
        pages = pages_for_max_tokens(max_live_tokens(trace), c["page_size"])
        runner = ModelRunner.create(model, num_pages=pages, page_size=c["page_size"], max_requests=3, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
    compare_rows(got, reference, relative=5e-4)


@pytest.mark.parametrize("layers", [
    [("mamba", (2, 8, 4, 1, 3, 2), 16), ("mamba", (3, 4, 5, 3, 2, 1), None)],        # no pages at all: state rows alone
    [("latent", (2, 8, 8, 8, 8), 16)],
    [("attention", (2, 1, 8, 4), None)],                                             # no mask, no state
])
def test_models_of_one_kind_of_mixer(tmp_path, layers):
    from tokuvik_helpers import attention, config, latent, layer, mamba
    make = {"mamba": mamba, "latent": latent, "attention": attention}
    c = dict(page_size=4, seed=5, config=config(40, 16, [layer(make[k](*sizes), ff) for k, sizes, ff in layers]))
    folder = write_folder(c, str(tmp_path / "m"))
    requests = requests_for(c, [21, 9, 14])
    reference = plain_logits(folder, requests, torch.float64)
    trace = trace_mixed(requests, seed=1, live=2)
    with ops.use_backend(EmulatedKernels()):
        model = load_model(folder, "float32", "cpu")
        runner = ModelRunner.create(model, num_pages=pages_for_max_tokens(max_live_tokens(trace), 4), page_size=4,
                                    max_requests=2, poison_freed_pages=True)
        got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
    compare_rows(got, reference, relative=5e-5)
