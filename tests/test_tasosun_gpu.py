"""Tasosun on the GPU: each new mechanism's kernel alone against the plain implementation's function
of that mechanism, then the engine (cache, batches, portions, windows, captured graphs, the entry
point) against the plain forward pass, in float32 and bfloat16."""
import copy
import json
import math
import os
import subprocess
import sys

import pytest
import torch

from helpers import max_live_tokens, replay_and_collect, trace_mixed, trace_portions, trace_tail, trace_whole
from plain import tasosun_plain
from tasosun_helpers import CONFIGS, compare_rows, plain_logits, requests_for, write_folder
from wllm_amd.engine import LLM, ModelRunner
from wllm_amd.engine.batch import StepEntry
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.kernels import ops
from wllm_amd.parts import load_model

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = {"mixed": [70, 45, 150, 33, 58], "odd": [40, 66, 25, 151], "sharp": [80, 137, 64, 50], "wide": [30, 140, 21], "small": [75, 20, 130]}
FAMILIES = {"whole": trace_whole, "tail": trace_tail, "portions": trace_portions, "mixed": trace_mixed}


def close(got, ref, dtype, what=""):
    atol, rtol = (2e-5, 2e-5) if dtype == torch.float32 else (1e-2, 8e-3)
    got, ref = got.double().cpu(), ref.double().cpu()
    err = ((got - ref).abs() / (atol + rtol * ref.abs())).max().item()
    assert err <= 1.0, f"{what}: worst error {err:.2f} x tolerance, max abs diff {(got - ref).abs().max().item():.3e}"


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("tasosun_gpu")
    return {name: write_folder(name, str(root / name)) for name in CONFIGS}


# ---- mechanisms alone ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,rot,factor,ps,stacked", [
    (4, 2, 32, 32, 1.0, 16, False), (3, 3, 20, 8, 2.0, 8, True), (2, 1, 160, 40, 8.0, 4, False), (5, 1, 64, 2, 3.0, 16, True),
    (1, 1, 256, 256, 1.0, 16, False), (6, 2, 12, 0, 1.0, 3, True)])
def test_rotation_unit_norm_and_cache_write(dtype, nh, nkv, d, rot, factor, ps, stacked):
    """`head_prepare` as Tasosun uses it (interleaved pairs, a part of the head, scaled positions, the
    unit norm, the keys as projected stored as values, gate columns behind the heads) against the
    plain functions; with and without a stack of partial sums."""
    g = torch.Generator().manual_seed(d + rot)
    n, eps, pages = 37, 1e-5, 16
    width = (2 * nh + nkv) * d
    pre = torch.randn(n, width, generator=g)
    bias = torch.randn(width, generator=g) * 0.3
    # (positions small enough that an angle worked out in float32, as the kernel must, is the exact one to 1e-5)
    positions = torch.randint(0, 150, (n,), generator=g, dtype=torch.int32)
    slots = torch.randperm(pages * ps, generator=g)[:n].to(torch.int32)
    rows = pre.to(dtype).to(DEV)
    parts = None
    if stacked:
        parts = torch.stack([pre * 0.25, pre * 0.5, pre * 0.25]).to(DEV)
        rows = torch.full_like(rows, float("nan"))          # what the row held is not read
    cache = torch.zeros(pages, 2, nkv, ps * d, dtype=dtype, device=DEV)
    spec = {"dims": rot, "base": 250.0, "scaling": {"factor": factor}}
    inv_freq = None
    if rot:
        inv_freq = (1.0 / (250.0 ** (torch.arange(0, rot, 2, dtype=torch.float64) / rot)) / factor).float().to(DEV)
    ops.head_prepare(rows, bias.to(DEV), positions.to(DEV), inv_freq, slots.to(DEV), cache, num_heads=nh, num_kv_heads=nkv,
                     head_dim=d, page_size=ps, interleaved=True, norm_eps=eps, values_are_keys=True, parts=parts)
    torch.cuda.synchronize()
    start = (pre if stacked else pre.to(dtype)).double() + bias.double()
    q, k = start[:, :nh * d].view(n, nh, d), start[:, nh * d:(nh + nkv) * d].view(n, nkv, d)
    if rot:
        q, k = tasosun_plain.rotate_interleaved(q, positions, spec), tasosun_plain.rotate_interleaved(k, positions, spec)
    q, k = tasosun_plain.unit_norm(q, eps), tasosun_plain.unit_norm(k, eps)
    close(rows[:, :nh * d], q.reshape(n, -1), dtype, "queries")
    close(rows[:, nh * d:(nh + nkv) * d], k.reshape(n, -1), dtype, "keys")
    close(rows[:, (nh + nkv) * d:], start[:, (nh + nkv) * d:], dtype, "gate columns")
    page, off = (slots // ps).long(), (slots % ps).long()
    kview = cache[:, 0].view(pages, nkv, ps, d).cpu()
    vview = cache[:, 1].view(pages, nkv, d, ps).cpu()
    close(kview[page, :, off, :], k, dtype, "cached keys")
    close(vview[page, :, :, off], start[:, nh * d:(nh + nkv) * d].view(n, nkv, d), dtype, "cached values: the keys as projected")
    assert torch.equal(kview[page, :, off, :].to(DEV), rows[:, nh * d:(nh + nkv) * d].view(n, nkv, d)), "row and cache hold the same key"


def test_half_pairing_without_a_norm_is_the_plain_rotation():
    """The general kernel with the options off does what `rope_and_cache_write` does."""
    g = torch.Generator().manual_seed(3)
    nh, nkv, d, ps, n = 3, 1, 40, 8, 19
    qkv = torch.randn(n, (nh + 2 * nkv) * d, generator=g).to(DEV)
    positions = torch.randint(0, 900, (n,), generator=g, dtype=torch.int32).to(DEV)
    slots = torch.randperm(6 * ps, generator=g)[:n].to(torch.int32).to(DEV)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, 24, 2, dtype=torch.float32) / 24))).to(DEV)
    a, b = qkv.clone(), qkv.clone()
    ca, cb = (torch.zeros(6, 2, nkv, ps * d, device=DEV) for _ in range(2))
    ops.rope_and_cache_write(a, None, positions, inv_freq, slots, ca, num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps)
    ops.head_prepare(b, None, positions, inv_freq, slots, cb, num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps)
    assert torch.equal(a, b) and torch.equal(ca, cb)


def _attention_problem(dtype, nh, nkv, d, ps, segs, seed, extra_columns):
    g = torch.Generator().manual_seed(seed)
    n = sum(q for q, _ in segs)
    pages = sum(-(-c // ps) for _, c in segs) + 3
    order = torch.randperm(pages, generator=g).tolist()
    bt = torch.zeros(len(segs), max(-(-c // ps) for _, c in segs), dtype=torch.int32)
    for s, (_, c) in enumerate(segs):
        for p in range(-(-c // ps)):
            bt[s, p] = order.pop()
    cache = torch.randn(pages, 2, nkv, ps * d, generator=g).to(dtype)
    rows = torch.randn(n, nh * d + extra_columns, generator=g).to(dtype)
    q_len = torch.tensor([q for q, _ in segs], dtype=torch.int32)
    ctx = torch.tensor([c for _, c in segs], dtype=torch.int32)
    q_start = (torch.cumsum(q_len, 0) - q_len).to(torch.int32)
    tok_seg = torch.repeat_interleave(torch.arange(len(segs), dtype=torch.int32), q_len.long())
    return rows, cache, bt, tok_seg, q_start, q_len, ctx


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,ps,window,cap,segs", [
    (4, 2, 32, 16, 24, 30.0, [(1, 100), (70, 70), (1, 24), (1, 25), (5, 200)]),      # matrix cores, decoded rows and blocks of 64
    (6, 2, 96, 16, 40, 20.0, [(1, 41), (130, 300)]),
    (2, 1, 64, 8, 0, 6.0, [(1, 300), (65, 65)]),                                     # a cap without a window
    (2, 1, 256, 16, 50, 12.0, [(1, 130), (80, 200)]),                               # the largest head
    (4, 4, 128, 16, 0, 10.0, [(1, 70), (100, 100), (3, 3)]),
    (3, 3, 20, 8, 7, 5.0, [(1, 50), (33, 40), (1, 7), (1, 8)]),                     # the kernel on the vector units
    (2, 2, 160, 4, 1, 15.0, [(1, 9), (20, 20)]),                                     # a window of one
])
def test_capped_scores_in_every_attention_kernel(dtype, nh, nkv, d, ps, window, cap, segs):
    """Scores bent under a cap before the softmax, rows wider than the query heads, windows: the kernels
    against the plain functions (`capped_scores`, `window_mask`, softmax), request by request.  The
    queries are scaled up so that the cap bites."""
    rows, cache, bt, tok_seg, q_start, q_len, ctx = _attention_problem(dtype, nh, nkv, d, ps, segs, seed=d + window, extra_columns=(nkv + nh) * d)
    rows[:, :nh * d] *= 3.0
    scale = 2.0 / math.sqrt(d)
    out = torch.zeros(rows.shape[0], nh * d, dtype=dtype, device=DEV)
    args = [t.to(DEV) for t in (rows, cache, bt, tok_seg, q_start, q_len, ctx)] + [out]
    kwargs = dict(num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps, scale=scale, window=window, softcap=cap,
                  max_q_len=int(q_len.max()), max_ctx_len=int(ctx.max()), exact_weights=True)
    kwargs["plan"] = ops.plan_paged_attention(q_len.numpy(), ctx.numpy(), num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps,
                                              window=window, dtype=dtype, device=torch.device(DEV))
    ops.paged_attention(*args, **kwargs)
    torch.cuda.synchronize()
    kview = cache[:, 0].view(-1, nkv, ps, d).double()
    vview = cache[:, 1].view(-1, nkv, d, ps).double()
    bent = 0
    for s, (ql, cl) in enumerate(segs):
        ids = bt[s, :-(-cl // ps)].long()
        keys = kview[ids].permute(0, 2, 1, 3).reshape(-1, nkv, d)[:cl]
        values = vview[ids].permute(0, 3, 1, 2).reshape(-1, nkv, d)[:cl]
        positions = torch.arange(cl)
        mask = tasosun_plain.window_mask(positions, window)[cl - ql:]
        q = rows[int(q_start[s]):int(q_start[s]) + ql, :nh * d].double().view(ql, nh, d)
        for head in range(nh):
            kv = head // (nh // nkv)
            qpad = torch.zeros(cl, d, dtype=torch.float64)
            qpad[cl - ql:] = q[:, head]
            sc = tasosun_plain.capped_scores(qpad, keys[:, kv], scale, cap)[cl - ql:]
            bent += int((sc.abs() > 0.5 * cap).sum())
            p = torch.softmax(sc.masked_fill(~mask, float("-inf")), dim=-1)
            close(out[int(q_start[s]):int(q_start[s]) + ql, head * d:(head + 1) * d], p @ values[:, kv], dtype,
                  f"segment {s} head {head}")
    assert bent > 0, "no score came near the cap: the case would pass without it"


@pytest.mark.parametrize("segs", [[(1, 3)] * 150, [(70, 70), (64, 67)]])
def test_bfloat16_kernels_weigh_the_values_with_more_than_bfloat16(segs):
    """With `exact_weights` the matrix-core kernels' only rounding is that of their result: their distance from
    the exact weighted sum is that of the exact sum's own rounding to bfloat16.  Without it the rounding of
    the weights shows on top (so the case can tell the two apart)."""
    nh, nkv, d, ps = 4, 2, 64, 16
    rows, cache, bt, tok_seg, q_start, q_len, ctx = _attention_problem(torch.bfloat16, nh, nkv, d, ps, segs, seed=9, extra_columns=0)
    window = 3          # few keys a query: single weights count
    dev = [t.to(DEV) for t in (rows, cache, bt, tok_seg, q_start, q_len, ctx)]
    plan = ops.plan_paged_attention(q_len.numpy(), ctx.numpy(), num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps,
                                    window=window, dtype=torch.bfloat16, device=torch.device(DEV))
    got = {}
    for exact in (True, False):
        out = torch.zeros(rows.shape[0], nh * d, dtype=torch.bfloat16, device=DEV)
        ops.paged_attention(*dev, out, num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps, scale=0.2, window=window,
                            max_q_len=int(q_len.max()), max_ctx_len=int(ctx.max()), plan=plan, exact_weights=exact)
        got[exact] = out.double().cpu()
    want = torch.zeros(rows.shape[0], nh * d, dtype=torch.float64)
    kview, vview = cache[:, 0].view(-1, nkv, ps, d).double(), cache[:, 1].view(-1, nkv, d, ps).double()
    for s, (ql, cl) in enumerate(segs):
        ids = bt[s, :-(-cl // ps)].long()
        keys = kview[ids].permute(0, 2, 1, 3).reshape(-1, nkv, d)[:cl]
        values = vview[ids].permute(0, 3, 1, 2).reshape(-1, nkv, d)[:cl]
        mask = tasosun_plain.window_mask(torch.arange(cl), window)[cl - ql:]
        q = rows[int(q_start[s]):int(q_start[s]) + ql].double().view(ql, nh, d)
        for head in range(nh):
            kv = head // (nh // nkv)
            sc = (q[:, head] @ keys[:, kv].T * 0.2).masked_fill(~mask, float("-inf"))
            want[int(q_start[s]):int(q_start[s]) + ql, head * d:(head + 1) * d] = torch.softmax(sc, -1) @ values[:, kv]
    rounding = (want.to(torch.bfloat16).double() - want).pow(2).mean().sqrt().item()
    exact_err = (got[True] - want).pow(2).mean().sqrt().item()
    rounded_err = (got[False] - want).pow(2).mean().sqrt().item()
    assert exact_err <= 1.01 * rounding, (exact_err, rounding)
    assert rounded_err > 1.04 * rounding, (rounded_err, rounding)     # (measured: 1.05 to 1.06)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gate_copy_and_sum_into_the_stream(dtype):
    g = torch.Generator().manual_seed(1)
    n, c, extra, hidden = 21, 52, 30, 70
    a = torch.randn(n, c, generator=g).to(dtype).to(DEV)
    wide = torch.randn(n, c + extra, generator=g).to(dtype).to(DEV)
    both = torch.zeros(n, c + 2 * extra, dtype=dtype, device=DEV)
    ops.sigmoid_gate(a, wide[:, extra:], both[:, :c])
    close(both[:, :c], a.double() * torch.sigmoid(wide[:, extra:].double()), dtype, "gated")
    ops.copy_columns(wide[:, :2 * extra], both[:, c:])
    assert torch.equal(both[:, c:], wide[:, :2 * extra])
    gu = torch.randn(n, 2 * extra, generator=g).to(dtype).to(DEV)
    ops.gated_activation(gu, both[:, c:c + extra], "silu")
    close(both[:, c:c + extra], torch.nn.functional.silu(gu[:, :extra].double()) * gu[:, extra:].double(), dtype, "silu band")
    assert torch.equal(both[:, c + extra:], wide[:, extra:2 * extra]), "the band's neighbours are untouched"
    x = torch.randn(n, hidden, generator=g).to(DEV)
    stack = torch.randn(3, n, hidden, generator=g).to(DEV)
    bias, addend = torch.randn(hidden, generator=g).to(DEV), torch.randn(n, hidden, generator=g).to(DEV)
    want = x.double() + stack.double().sum(0) + bias.double() + addend.double()
    ops.stream_add(x, addend, stack, bias)
    close(x, want, torch.float32, "stream sum")
    # the norm that takes a pending contribution and its bias: the stream moves on by both
    w = torch.randn(hidden, generator=g).to(DEV) * 0.1
    delta = torch.randn(n, hidden, generator=g).to(dtype).to(DEV)
    out = torch.zeros(n, hidden, dtype=dtype, device=DEV)
    moved = x.double() + delta.double() + bias.double()
    ops.rms_norm(x, w, 1e-5, 1.0, out, delta=delta, delta_bias=bias)
    close(x, moved, torch.float32, "stream after the norm")
    close(out, tasosun_plain.offset_norm(moved, w.double(), 1e-5), dtype, "normed")


# ---- the engine ---------------------------------------------------------------------------------------
def _references(folder, requests, dtype):
    exact = plain_logits(folder, requests, torch.float64)
    rounded = plain_logits(folder, requests, torch.float64, round_to=torch.bfloat16) if dtype == "bfloat16" else None
    return exact, rounded


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_replay_matches_plain(folders, name, family, dtype):
    requests = requests_for(name, LENGTHS[name])
    trace = FAMILIES[family](requests)
    page_size = CONFIGS[name]["page_size"]
    model = load_model(folders[name], dtype, DEV)
    runner = ModelRunner.create(model, num_pages=pages_for_max_tokens(max_live_tokens(trace), page_size), page_size=page_size,
                                max_requests=4, poison_freed_pages=True)
    with torch.inference_mode():
        got = replay_and_collect(TraceReplayer(runner), trace)
    runner.cache.check()
    assert all(g.pool.num_free == g.pool.num_pages for g in runner.cache.groups)
    exact, rounded = _references(folders[name], requests, dtype)
    compare_rows(got, exact, rounded, float32_relative=5e-5)


@pytest.mark.parametrize("seed", range(16))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Other sizes, head counts, orders of layers, windows, constants and loops than any fixed case: a mixed trace
    (portions beside decoded tokens, pages used again) in both precisions against the plain implementation."""
    from tasosun_helpers import random_config
    case = random_config(seed)
    folder = write_folder(case, str(tmp_path / "m"))
    requests = requests_for(case, [90, 41, 130, 23])
    trace = trace_mixed(requests, seed=seed)
    for dtype in ("float32", "bfloat16"):
        model = load_model(folder, dtype, DEV)
        runner = ModelRunner.create(model, num_pages=pages_for_max_tokens(max_live_tokens(trace), 16), page_size=16,
                                    max_requests=4, poison_freed_pages=True)
        with torch.inference_mode():
            got = replay_and_collect(TraceReplayer(runner), trace)
        runner.cache.check()
        exact, rounded = _references(folder, requests, dtype)
        compare_rows(got, exact, rounded, float32_relative=5e-5)


@pytest.mark.parametrize("seed", range(2))
def test_long_requests_at_middling_sizes(tmp_path, seed):
    """Requests of up to 1,100 tokens: whole, with a tail of 140 tokens decoded one by one (windows pass over
    decoded tokens), and four live at a time in portions beside decoded tokens, in a pool made for what is
    live; every 7th position is compared."""
    from tasosun_helpers import middling_config
    case = middling_config(seed)
    folder = write_folder(case, str(tmp_path / "m"))
    requests = requests_for(case, [1100, 400, 333, 90, 610])
    thin = lambda trace: [dict(st, entries=[dict(e, want=[w for w in e["want"] if (w + len(e["tokens"])) % 7 == 0 or len(e["tokens"]) == 1])
                                             for e in st["entries"]]) for st in trace]
    one = {"q0": requests["q0"]}
    traces = [thin(trace_whole(one)), thin(trace_tail(one, tail=140)),
              thin(trace_mixed(requests, seed=seed, portion_sizes=(2, 16, 37, 64, 130)))]
    for dtype in ("float32", "bfloat16"):
        model = load_model(folder, dtype, DEV)
        exact, rounded = _references(folder, requests, dtype)
        for trace in traces:
            runner = ModelRunner.create(model, num_pages=pages_for_max_tokens(max_live_tokens(trace), 16), page_size=16,
                                        max_requests=4, poison_freed_pages=True)
            with torch.inference_mode():
                got = replay_and_collect(TraceReplayer(runner), trace)
            runner.cache.check()
            compare_rows(got, exact, rounded, float32_relative=5e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_windows_in_a_small_pool(folders, dtype):
    """300 tokens decoded one by one after a short prompt, in a pool that only holds them because windows
    give pages back; freed pages are filled with NaN and used again."""
    name = "sharp"
    requests = requests_for(name, [340])
    trace = trace_tail(requests, tail=300)
    model = load_model(folders[name], dtype, DEV)
    runner = ModelRunner.create(model, num_pages=7, page_size=16, max_requests=2, poison_freed_pages=True)
    with torch.inference_mode():
        got = replay_and_collect(TraceReplayer(runner), trace)
    exact, rounded = _references(folders[name], requests, dtype)
    compare_rows(got, exact, rounded, float32_relative=5e-5)


def test_a_row_does_not_depend_on_the_batch_or_the_cut(folders):
    """float32: the logits of a position, from a whole prompt, from portions of two to sixteen tokens, decoded alone
    and decoded beside a long prompt of another request, agree to rounding."""
    name = "mixed"
    requests = requests_for(name, [90, 200])
    model = load_model(folders[name], "float32", DEV)

    def run(trace):
        runner = ModelRunner.create(model, num_pages=40, page_size=16, max_requests=4)
        with torch.inference_mode():
            return replay_and_collect(TraceReplayer(runner), trace)

    one = {"q0": requests["q0"]}
    whole, cut, tail = run(trace_whole(one)), run(trace_portions(one)), run(trace_tail(one, tail=40))
    beside = []
    toks = requests["q0"]
    beside.append({"step": 0, "entries": [{"id": "q0", "tokens": toks[:50], "want": list(range(50))}], "end": []})
    beside.append({"step": 1, "entries": [{"id": "q1", "tokens": requests["q1"][:137], "want": []},
                                          {"id": "q0", "tokens": [toks[50]], "want": [0]}], "end": []})
    beside.append({"step": 2, "entries": [{"id": "q0", "tokens": toks[51:], "want": list(range(39))},
                                          {"id": "q1", "tokens": requests["q1"][137:], "want": []}], "end": ["q0", "q1"]})
    mixed = run(beside)
    for key, ref in whole.items():
        for other in (cut, tail, mixed):
            assert (other[key] - ref).abs().max().item() <= 2e-4 * max(1.0, ref.abs().max().item()), key


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_entry_point(folders, graphs):
    """`LLM.generate` (scheduler, chunked prefill, sampling kernels, captured graphs or not) against greedy decoding
    with the plain implementation, in float32 so that the tokens are comparable one by one."""
    name = "sharp"
    prompts = list(requests_for(name, [37, 5, 64, 18, 1]).values())
    new = 24
    llm = LLM(folders[name], dtype="float32", num_blocks=64, block_size=16, max_prefill_tokens_per_step=32, max_requests=4,
              hip_graphs=graphs)
    outs = llm.generate(prompts, max_new_tokens=new)
    cfg = tasosun_plain.read_config(folders[name])
    w = tasosun_plain.read_weights(folders[name], torch.float64)
    for prompt, out in zip(prompts, outs):
        tokens = list(prompt)
        for step in range(new):
            logits = tasosun_plain.forward(cfg, w, tokens)[-1]
            top2 = logits.topk(2).values
            if (top2[0] - top2[1]).item() < 1e-3:       # a tie within rounding: the rest is not comparable
                break
            assert out.token_ids[step] == int(logits.argmax()), f"prompt of {len(prompt)}: token {step} differs"
            tokens.append(out.token_ids[step])
        assert len(out.token_ids) == new
        assert len(set(out.token_ids)) > 3, "the continuation hardly varies"
    if graphs:
        assert llm.runner.graph_steps > 0


def test_the_trace_runner_and_the_command_line(folders, tmp_path):
    name = "odd"
    toks = requests_for(name, [45])["q0"]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:30], "want": [0, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[30:32], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": toks[32:], "want": [12]}], "end": ["a"]}]
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders[name], "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "64"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [line for line in r.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1", "done 2"]
    exact = plain_logits(folders[name], {"a": toks}, torch.float64)
    first = torch.frombuffer(bytearray((out / "0.f32").read_bytes()), dtype=torch.float32).view(2, -1)
    last = torch.frombuffer(bytearray((out / "2.f32").read_bytes()), dtype=torch.float32).view(1, -1)
    assert not (out / "1.f32").exists()
    compare_rows({("a", 0): first[0], ("a", 29): first[1], ("a", 44): last[0]}, exact, float32_relative=5e-5)
    # the command line: a model folder of a named shape, then greedy generation from it
    made = tmp_path / "made"
    r = subprocess.run([sys.executable, "-m", "wllm_amd.cli", "random-model", "--out", str(made), "--config", "tasosun-tiny",
                        "--seed", "3", "--std", "0.3"], cwd=ROOT, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    r = subprocess.run([sys.executable, "-m", "wllm_amd.cli", "generate", "--model", str(made), "--dtype", "float32",
                        "--prompt-ids", "5,17,3,200,41", "--max-new-tokens", "6"], cwd=ROOT, capture_output=True, text=True,
                       timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    line = json.loads([x for x in r.stdout.splitlines() if x.startswith("{")][-1])
    cfg, w = tasosun_plain.read_config(str(made)), tasosun_plain.read_weights(str(made), torch.float64)
    tokens = [5, 17, 3, 200, 41]
    for t in line["token_ids"]:
        logits = tasosun_plain.forward(cfg, w, tokens)[-1]
        if (logits.topk(2).values[0] - logits.topk(2).values[1]).item() < 1e-3:
            break
        assert t == int(logits.argmax())
        tokens.append(t)
    assert len(line["token_ids"]) == 6
