"""Tokuvik on the GPU: each new mechanism's kernel alone against the plain implementation's function of
that mechanism, then the engine (cache, state slots, batches, portions, chunks, captured graphs, the entry
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
from plain import tokuvik_plain as plain
from tokuvik_helpers import (CONFIGS, compare_rows, middling_config, plain_logits, random_config, read_folder, requests_for,
                             write_folder)
from wllm_amd.engine import LLM, ModelRunner
from wllm_amd.engine.replay import TraceReplayer, pages_for_max_tokens
from wllm_amd.kernels import ops
from wllm_amd.parts import load_model

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = {"trio": [70, 45, 150, 33, 58], "odd": [40, 66, 25, 151], "sharp": [80, 137, 64, 50]}
FAMILIES = {"whole": trace_whole, "tail": trace_tail, "portions": trace_portions, "mixed": trace_mixed}
# a row's distance from the plain implementation, as a share of the row's own size: float32 sums in another
# order; bfloat16 activations through some ten roundings a layer
# (measured: float32 rows lie 1e-6 to 7e-6 away; bfloat16 rows 0.4 to 1% a handful of layers, with a row in a hundred up to
# 8% where rounding decides between two keys)
BOUND = {torch.float32: dict(relative=1e-4), torch.bfloat16: dict(relative=0.04, outliers=0.05, ceiling=6.0)}
# the sharp model multiplies every rounding by some hundred (in float32 a lost key still moves a row by far more than
# this; in bfloat16 single keys change places, and only the bulk of the rows says anything)
SHARP_BOUND = {torch.float32: dict(relative=6e-4), torch.bfloat16: dict(relative=0.3, outliers=0.2, ceiling=10.0)}


def close(got, ref, dtype, what="", scale=1.0):
    atol, rtol = (3e-5 * scale, 3e-5) if dtype == torch.float32 else (1.5e-2 * scale, 1e-2)
    got, ref = got.double().cpu(), ref.double().cpu()
    err = ((got - ref).abs() / (atol + rtol * ref.abs())).max().item()
    assert err <= 1.0, f"{what}: worst error {err:.2f} x tolerance, max abs diff {(got - ref).abs().max().item():.3e}"


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("tokuvik_gpu")
    return {name: write_folder(name, str(root / name)) for name in CONFIGS}


# ---- mechanisms alone ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,behind,before,stacked,gathered", [
    (64, "layer", "layer", False, False), (48, "rms", "layer", True, False), (200, "layer", "rms", True, True),
    (1030, None, "layer", False, True), (96, "layer", None, False, False), (5000, "rms", "rms", False, False)])
def test_norm_behind_a_sublayer_sum_and_norm_before_the_next(dtype, hidden, behind, before, stacked, gathered):
    g = torch.Generator().manual_seed(hidden)
    n = 19
    x = torch.randn(n, hidden, generator=g) * 3 + 0.7
    wb, wn = 1 + 0.3 * torch.randn(hidden, generator=g), 1 + 0.3 * torch.randn(hidden, generator=g)
    if stacked:
        delta = torch.randn(3, n, hidden, generator=g) + 0.4
        total = delta[0] + delta[1] + delta[2]
    else:
        delta = (torch.randn(n, hidden, generator=g) + 0.4).to(dtype)
        total = delta.float()
    rows = torch.tensor([5, 0, 18, 5], dtype=torch.int32) if gathered else None
    norms = {"layer": plain.layer_norm, "rms": plain.rms_norm, None: lambda v, w, eps: v}
    new_x = x.double() + norms[behind](total.double(), wb.double(), 1e-5)
    want = norms[before](new_x, wn.double(), 1e-6)
    xd = x.to(DEV)
    out = torch.zeros(len(rows) if gathered else n, hidden, dtype=dtype, device=DEV)
    recipe = lambda kind, w, eps: None if kind is None else ops.NormRecipe(kind, w.to(DEV), eps)
    ops.norm_add(xd, delta=delta.to(DEV), delta_norm=recipe(behind, wb, 1e-5), out=out, out_norm=recipe(before, wn, 1e-6),
                 rows=rows.to(DEV) if gathered else None)
    pick = rows.long() if gathered else slice(None)
    close(out, want[pick], dtype, "the normed sum", scale=3.0 if before is None else 1.0)
    if gathered:
        assert torch.equal(xd.cpu(), x), "gathered rows leave the stream alone"
    else:
        close(xd, new_x, torch.float32, "the stream")


@pytest.mark.parametrize("dtype", DTYPES)
def test_band_norms_of_a_wider_row(dtype):
    """Two bands of one row, each under an RMS norm with a weight: one in place with padding inside the band
    that does not count, one into a wider band of another tensor whose further columns become zero."""
    g = torch.Generator().manual_seed(3)
    n, a, b, pad = 23, 40, 28, 4
    row = torch.randn(n, a + 7 + b, generator=g).to(dtype)
    row[:, a - pad:a] = 0                                   # padding inside the first band
    wa, wb = 1 + 0.2 * torch.randn(a, generator=g), 1 + 0.2 * torch.randn(b, generator=g)
    wa[a - pad:] = 0
    dev = row.to(DEV)
    other = torch.full((n, 50), 7.0, dtype=dtype, device=DEV)
    ops.band_norm([(dev[:, :a], wa.to(DEV), a - pad, dev[:, :a]), (dev[:, a + 7:], wb.to(DEV), b, other[:, 10:10 + b + 6])], 1e-5)
    close(dev[:, :a - pad], plain.rms_norm(row[:, :a - pad].double(), wa[:a - pad].double(), 1e-5), dtype, "in place")
    assert (dev[:, a - pad:a] == 0).all() and torch.equal(dev[:, a:a + 7].cpu(), row[:, a:a + 7])
    close(other[:, 10:10 + b], plain.rms_norm(row[:, a + 7:].double(), wb.double(), 1e-5), dtype, "into another band")
    assert (other[:, 10 + b:10 + b + 6] == 0).all() and (other[:, :10] == 7).all() and (other[:, 10 + b + 6:] == 7).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,heads,outs,keys", [(37, 3, 20, 12), (70, 4, 96, 32), (1, 5, 7, 100), (130, 1, 64, 64), (8, 6, 130, 128),
                                               (16, 2, 64, 256), (3, 3, 40, 48), (9, 2, 33, 16)])
def test_products_head_by_head_and_the_gated_lookup(dtype, n, heads, outs, keys):
    g = torch.Generator().manual_seed(n + keys)
    wide = torch.randn(n, heads * keys + 5, generator=g).to(dtype)
    w = (torch.randn(heads, outs, keys, generator=g) * keys ** -0.5).to(dtype)
    y = torch.zeros(n, heads * outs + 3, dtype=dtype, device=DEV)
    ops.head_linear(wide.to(DEV)[:, 5:], w.to(DEV), y[:, :heads * outs])
    want = torch.einsum("nhk,hok->nho", wide[:, 5:].double().view(n, heads, keys), w.double()).reshape(n, -1)
    close(y[:, :heads * outs], want, dtype, "head by head")
    assert (y[:, heads * outs:] == 0).all()
    # the token input's lookup: a band of the token's row of a table, times the bent projection
    table = torch.randn(50, 3 * outs, generator=g).to(dtype)
    ids = torch.randint(0, 50, (n,), generator=g, dtype=torch.int32)
    gate = torch.randn(n, outs, generator=g).to(dtype)
    out = torch.zeros(n, outs, dtype=dtype, device=DEV)
    ops.gated_lookup(gate.to(DEV), ids.to(DEV), table.to(DEV), outs, out, "gelu_tanh")
    close(out, plain.gelu_tanh(gate.double()) * table.double()[ids.long(), outs:2 * outs], dtype, "lookup")


def _segments(lengths, generator, slots_total):
    q_len = torch.tensor(lengths, dtype=torch.int32)
    q_start = (torch.cumsum(q_len, 0) - q_len).to(torch.int32)
    tok_seg = torch.repeat_interleave(torch.arange(len(lengths), dtype=torch.int32), q_len.long())
    slots = torch.randperm(slots_total, generator=generator)[:len(lengths)].to(torch.int32)
    return q_len, q_start, tok_seg, slots


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("channels,taps", [(40, 4), (300, 2), (7, 1), (64, 7)])
def test_the_convolution_whole_and_cut_with_its_carried_inputs(dtype, channels, taps):
    """Three sequences side by side, each fed whole, then in portions of 1, 2 and more tokens through state
    slots that held other values before: every token against the plain convolution of its whole sequence."""
    g = torch.Generator().manual_seed(channels)
    lengths = [23, 1, 9]
    seqs = [torch.randn(t, channels + 6, generator=g).to(dtype) for t in lengths]
    weight, bias = torch.randn(channels, taps, generator=g) * 0.5, torch.randn(channels, generator=g) * 0.2
    want = [plain.silu(plain.causal_conv(s[:, 3:3 + channels].double(), weight.double(), bias.double())) for s in seqs]
    offset, slots_total = 11, 6
    for cuts in ([23], [1, 2, 1, 5, 3, 2, 1, 8]):
        state = torch.randn(slots_total, offset + (taps - 1) * channels + 2, generator=g).to(DEV)
        _, _, _, slots = _segments(lengths, g, slots_total)
        state[slots.long()] = 0                     # what opening a request does
        fed = [0, 0, 0]
        for cut in cuts:
            take = [min(cut, lengths[i] - fed[i]) for i in range(3)]
            live = [i for i in range(3) if take[i] > 0]
            q_len, q_start, tok_seg, _ = _segments([take[i] for i in live], g, slots_total)
            inp = torch.cat([seqs[i][fed[i]:fed[i] + take[i]] for i in live]).to(DEV)
            out = torch.zeros(inp.shape[0], channels, dtype=dtype, device=DEV)
            ops.causal_conv(inp[:, 3:3 + channels], weight.to(DEV), bias.to(DEV), state, offset, tok_seg.to(DEV), q_start.to(DEV),
                            q_len.to(DEV), slots[live].to(DEV), out)
            for j, i in enumerate(live):
                close(out[int(q_start[j]):int(q_start[j]) + take[i]], want[i][fed[i]:fed[i] + take[i]], dtype,
                      f"sequence {i} from {fed[i]}")
                fed[i] += take[i]
        assert fed == lengths


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,groups,n_state,p", [(4, 2, 16, 16), (3, 1, 7, 10), (2, 2, 130, 72), (6, 3, 48, 64), (1, 1, 256, 4)])
def test_the_recurrence_whole_and_token_by_token(dtype, heads, groups, n_state, p):
    """Sequences side by side through the recurrence's kernel: whole, and cut down to single tokens, from
    state slots that are zeroed as a fresh request's; then the gated norm in groups."""
    g = torch.Generator().manual_seed(n_state + p)
    lengths = [41, 3, 18]
    inner, slots_total = heads * p, 5
    width = inner + 2 * groups * n_state
    seqs = [(torch.randn(t, width, generator=g) * 0.7).to(dtype) for t in lengths]
    dts = [torch.randn(t, heads + 3, generator=g).to(dtype) for t in lengths]
    dt_bias, a_log, d_skip = 0.3 * torch.randn(heads, generator=g), -0.5 + 0.8 * torch.randn(heads, generator=g), 1 + 0.3 * torch.randn(heads, generator=g)
    want, last = [], []
    for s, d in zip(seqs, dts):
        s64 = s.double()
        y, state = plain.state_space_recurrence(
            s64[:, :inner].view(-1, heads, p), s64[:, inner:inner + groups * n_state].view(-1, groups, n_state),
            s64[:, inner + groups * n_state:].view(-1, groups, n_state), plain.softplus(d[:, 1:1 + heads].double() + dt_bias.double()),
            a_log.double(), d_skip.double())
        want.append(y.reshape(-1, inner))
        last.append(state)
    for cuts in ([41], [16, 1, 1, 2, 17, 1, 3]):
        state = torch.randn(slots_total, heads * n_state * p + 9, generator=g).to(DEV)
        _, _, _, slots = _segments(lengths, g, slots_total)
        state[slots.long()] = 0
        fed = [0, 0, 0]
        for cut in cuts:
            take = [min(cut, lengths[i] - fed[i]) for i in range(3)]
            live = [i for i in range(3) if take[i] > 0]
            q_len, q_start, _, _ = _segments([take[i] for i in live], g, slots_total)
            xbc = torch.cat([seqs[i][fed[i]:fed[i] + take[i]] for i in live]).to(DEV)
            dt = torch.cat([dts[i][fed[i]:fed[i] + take[i]] for i in live]).to(DEV)
            y = torch.zeros(xbc.shape[0], inner, device=DEV)
            ops.ssm_scan(xbc, dt[:, 1:1 + heads], dt_bias.to(DEV), a_log.to(DEV), d_skip.to(DEV), state, q_start.to(DEV),
                         q_len.to(DEV), slots[live].to(DEV), y, heads=heads, groups=groups, state_size=n_state, head_dim=p)
            for j, i in enumerate(live):
                close(y[int(q_start[j]):int(q_start[j]) + take[i]], want[i][fed[i]:fed[i] + take[i]], torch.float32,
                      f"sequence {i} from {fed[i]}", scale=float(want[i].abs().max()))
                fed[i] += take[i]
        for i in range(3):
            kept = state[int(slots[i]), :heads * n_state * p].view(heads, n_state, p)
            close(kept, last[i], torch.float32, f"the state sequence {i} leaves", scale=float(last[i].abs().max()))
    # the gated norm behind it
    y = want[0].float()
    z = torch.randn(lengths[0], inner + 4, generator=g).to(dtype)
    w = 1 + 0.2 * torch.randn(inner, generator=g)
    parts = heads if inner % heads == 0 else 1
    out = torch.zeros(lengths[0], inner, dtype=dtype, device=DEV)
    ops.gated_group_norm(y.to(DEV), z.to(DEV)[:, 2:2 + inner], w.to(DEV), out, parts, 1e-5)
    close(out, plain.gated_group_norm(y.double(), z[:, 2:2 + inner].double(), w.double(), parts, 1e-5), dtype, "gated norm")


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
@pytest.mark.parametrize("nh,nkv,d,ps,chunk,sinks,segs", [
    (4, 2, 32, 16, 24, False, [(1, 100), (70, 70), (1, 24), (1, 25), (1, 49), (5, 200)]),    # matrix cores: decoded rows, blocks of 64
    (6, 2, 96, 16, 40, False, [(1, 41), (1, 40), (130, 300)]),
    (2, 1, 64, 8, 120, False, [(1, 300), (1, 241), (1, 240), (65, 65), (200, 400)]),
    (2, 2, 160, 4, 1, False, [(1, 9), (20, 20)]),                                           # a chunk of one
    (4, 4, 128, 16, 1000, False, [(1, 70), (100, 100)]),                                    # a chunk beyond every request
    (3, 3, 20, 8, 7, False, [(1, 50), (33, 40), (1, 7), (1, 8), (1, 15)]),                  # the kernel on the vector units
    (6, 1, 28, 8, 19, True, [(1, 20), (1, 19), (40, 40), (3, 230)]),                        # ... with sinks
    (5, 1, 96, 16, 0, True, [(1, 300), (70, 70), (1, 1), (2, 131)]),                        # sinks, no mask, many heads on one
    (12, 1, 64, 16, 0, True, [(1, 129), (30, 45)]),
    (10, 1, 20, 8, 0, True, [(1, 150), (21, 40)]),                                          # more heads on a key head than a pass takes
    (11, 1, 36, 4, 9, True, [(1, 10), (1, 9), (30, 30)]),
    (20, 1, 256, 16, 0, True, [(1, 700), (300, 300), (64, 1000)]),                          # keys cut into pieces: the reduce kernels
    (4, 2, 128, 8, 50, True, [(1, 49), (1, 50), (1, 51), (200, 230)]),
])
def test_chunks_and_sinks_in_every_attention_kernel(dtype, nh, nkv, d, ps, chunk, sinks, segs):
    """Keys just inside and just outside a chunk's edge, decoded alone and inside prompts, with scores so
    sharp that one key decides: the kernels against the plain mask and softmax, request by request."""
    rows, cache, bt, tok_seg, q_start, q_len, ctx = _attention_problem(dtype, nh, nkv, d, ps, segs, seed=d + chunk, extra_columns=8)
    rows[:, :nh * d] *= 2.0
    scale = 2.0 / math.sqrt(d)
    sink = (2.0 + 2.0 * torch.randn(nh, generator=torch.Generator().manual_seed(1))) if sinks else None
    out = torch.zeros(rows.shape[0], nh * d, dtype=dtype, device=DEV)
    args = [t.to(DEV) for t in (rows, cache, bt, tok_seg, q_start, q_len, ctx)] + [out]
    kwargs = dict(num_heads=nh, num_kv_heads=nkv, head_dim=d, page_size=ps, scale=scale, chunk=chunk,
                  max_q_len=int(q_len.max()), max_ctx_len=int(ctx.max()), exact_weights=True)
    if sinks:
        kwargs["sinks"] = sink.to(DEV)
    kwargs["plan"] = ops.plan_paged_attention(q_len.numpy(), ctx.numpy(), num_heads=nh, num_kv_heads=nkv, head_dim=d,
                                              page_size=ps, window=-chunk, dtype=dtype, device=torch.device(DEV))
    assert (kwargs["plan"] is not None) == (d % 32 == 0 and ps % 4 == 0)
    ops.paged_attention(*args, **kwargs)
    torch.cuda.synchronize()
    kview = cache[:, 0].view(-1, nkv, ps, d).double()
    vview = cache[:, 1].view(-1, nkv, d, ps).double()
    for s, (ql, cl) in enumerate(segs):
        ids = bt[s, :-(-cl // ps)].long()
        keys = kview[ids].permute(0, 2, 1, 3).reshape(-1, nkv, d)[:cl].repeat_interleave(nh // nkv, dim=1)
        values = vview[ids].permute(0, 3, 1, 2).reshape(-1, nkv, d)[:cl].repeat_interleave(nh // nkv, dim=1)
        q = torch.zeros(cl, nh, d, dtype=torch.float64)
        q[cl - ql:] = rows[int(q_start[s]):int(q_start[s]) + ql, :nh * d].double().view(ql, nh, d)
        scores = torch.einsum("ihd,jhd->hij", q, keys) * scale
        weights = plain.softmax_with_sink(scores, plain.chunk_mask(cl, chunk or None), sink.double() if sinks else None)
        want = torch.einsum("hij,jhd->ihd", weights, values)[cl - ql:].reshape(ql, nh * d)
        close(out[int(q_start[s]):int(q_start[s]) + ql], want, dtype, f"segment {s} ({ql} of {cl})")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_gate_a_head(dtype):
    g = torch.Generator().manual_seed(5)
    n, heads, d = 21, 6, 20
    a = torch.randn(n, heads * d, generator=g).to(dtype)
    wide = torch.randn(n, 9 + heads, generator=g).to(dtype)
    out = torch.zeros(n, heads * d, dtype=dtype, device=DEV)
    ops.sigmoid_gate(a.to(DEV), wide.to(DEV)[:, 9:], out, per=d)
    want = a.double().view(n, heads, d) * torch.sigmoid(wide[:, 9:].double())[:, :, None]
    close(out, want.reshape(n, -1), dtype, "a gate a head")


# ---- the engine ----------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("name", list(CONFIGS))
def test_replay_matches_plain(folders, name, family, dtype):
    requests = requests_for(name, LENGTHS[name])
    exact = plain_logits(folders[name], requests, torch.float64)
    trace = FAMILIES[family](requests)
    page_size = CONFIGS[name]["page_size"]
    model = load_model(folders[name], dtype, DEV)
    pages = pages_for_max_tokens(max_live_tokens(trace), page_size)
    runner = ModelRunner.create(model, num_pages=pages, page_size=page_size, max_requests=4, poison_freed_pages=True)
    with torch.inference_mode():
        got = replay_and_collect(TraceReplayer(runner), trace)
    runner.cache.check()
    assert not runner.cache.requests
    compare_rows(got, exact, **(SHARP_BOUND if name == "sharp" else BOUND)[dtype])


@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_at_random(tmp_path, seed):
    c = random_config(200 + seed)
    folder = write_folder(c, str(tmp_path / "m"))
    requests = requests_for(c, [37, 18, 150, 64])
    exact = plain_logits(folder, requests, torch.float64)
    for dtype in DTYPES:
        for family in ("portions", "mixed"):
            trace = FAMILIES[family](requests)
            model = load_model(folder, dtype, DEV)
            pages = pages_for_max_tokens(max_live_tokens(trace), c["page_size"])
            runner = ModelRunner.create(model, num_pages=pages, page_size=c["page_size"], max_requests=4, poison_freed_pages=True)
            with torch.inference_mode():
                got = replay_and_collect(TraceReplayer(runner), trace)
            runner.cache.check()
            compare_rows(got, exact, **BOUND[dtype])


@pytest.mark.parametrize("seed", range(3))
def test_long_requests_at_middling_sizes(tmp_path, seed):
    """Widths of some hundred and requests of up to 700 tokens, whole (the library's products, the tiled
    kernels, blocks of 64 rows in the attention, several tiles of columns in the recurrence) and four at a time."""
    c = middling_config(300 + seed)
    folder = write_folder(c, str(tmp_path / "m"))
    requests = requests_for(c, [700, 129, 300, 65])
    exact = plain_logits(folder, requests, torch.float64)
    for dtype in DTYPES:
        for family in ("whole", "mixed"):
            trace = FAMILIES[family](requests) if family == "whole" else trace_mixed(requests, seed=seed, portion_sizes=(2, 64, 100, 128, 29))
            # every tenth row is enough of a long request
            for step in trace:
                for e in step["entries"]:
                    e["want"] = [w for w in e["want"] if w % 10 == 0 or len(e["tokens"]) == 1]
            model = load_model(folder, dtype, DEV)
            pages = pages_for_max_tokens(max_live_tokens(trace), 16)
            runner = ModelRunner.create(model, num_pages=pages, page_size=16, max_requests=4, poison_freed_pages=True)
            with torch.inference_mode():
                got = replay_and_collect(TraceReplayer(runner), trace)
            runner.cache.check()
            compare_rows(got, exact, **BOUND[dtype])


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_through_chunks_in_a_small_pool(folders, dtype):
    """300 tokens of which 260 are decoded one by one, in a pool that only the chunks make fit; the recurrent
    layer's state is carried through every step."""
    raw = copy.deepcopy(CONFIGS["sharp"])
    raw["config"]["layers"] = [raw["config"]["layers"][i] for i in (0, 3, 4)]
    raw["config"]["layers"][1]["mixer"]["kv_from"] = 0
    import tempfile
    with tempfile.TemporaryDirectory() as folder:
        write_folder(raw, folder)
        requests = requests_for(raw, [300])
        exact = plain_logits(folder, requests, torch.float64)
        model = load_model(folder, dtype, DEV)
        runner = ModelRunner.create(model, num_pages=4, page_size=16, max_requests=2, poison_freed_pages=True)
        with torch.inference_mode():
            got = replay_and_collect(TraceReplayer(runner), trace_tail(requests, tail=260))
        runner.cache.check()
    compare_rows(got, exact, **SHARP_BOUND[dtype])


def test_a_row_does_not_depend_on_the_batch_or_the_cut(folders):
    name = "sharp"
    requests = requests_for(name, [90, 200])
    model = load_model(folders[name], "float32", DEV)

    def run(trace):
        runner = ModelRunner.create(model, num_pages=40, page_size=16, max_requests=4)
        with torch.inference_mode():
            return replay_and_collect(TraceReplayer(runner), trace)

    one = {"q0": requests["q0"]}
    whole, cut, tail = run(trace_whole(one)), run(trace_portions(one)), run(trace_tail(one, tail=40))
    toks = requests["q0"]
    beside = [{"step": 0, "entries": [{"id": "q0", "tokens": toks[:50], "want": list(range(50))}], "end": []},
              {"step": 1, "entries": [{"id": "q1", "tokens": requests["q1"][:137], "want": []},
                                      {"id": "q0", "tokens": [toks[50]], "want": [0]}], "end": []},
              {"step": 2, "entries": [{"id": "q0", "tokens": toks[51:], "want": list(range(39))},
                                      {"id": "q1", "tokens": requests["q1"][137:], "want": []}], "end": ["q0", "q1"]}]
    mixed = run(beside)
    for key, ref in whole.items():
        for other in (cut, tail, mixed):
            assert (other[key] - ref).abs().max().item() <= 2e-4 * max(1.0, ref.abs().max().item()), key


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_entry_point(folders, graphs):
    """`LLM.generate` (scheduler, chunked prefill, sampling kernels, captured graphs or not) against greedy decoding
    with the plain implementation, in float32 so that the tokens are comparable one by one."""
    name = "trio"
    prompts = list(requests_for(name, [37, 5, 64, 18, 1]).values())
    new = 24
    llm = LLM(folders[name], dtype="float32", num_blocks=64, block_size=16, max_prefill_tokens_per_step=32, max_requests=4,
              hip_graphs=graphs)
    outs = llm.generate(prompts, max_new_tokens=new)
    raw, w = read_folder(folders[name])
    for prompt, out in zip(prompts, outs):
        tokens = list(prompt)
        for step in range(new):
            logits = plain.forward(raw, w, tokens)[-1]
            top2 = logits.topk(2).values
            if (top2[0] - top2[1]).item() < 1e-3:       # a tie within rounding: the rest is not comparable
                break
            assert out.token_ids[step] == int(logits.argmax()), f"prompt of {len(prompt)}: token {step} differs"
            tokens.append(out.token_ids[step])
        assert len(out.token_ids) == new
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
    compare_rows({("a", 0): first[0], ("a", 29): first[1], ("a", 44): last[0]}, exact, relative=1e-4)
    # the command line: a model folder of a named shape, then greedy generation from it
    made = tmp_path / "made"
    r = subprocess.run([sys.executable, "-m", "wllm_amd.cli", "random-model", "--out", str(made), "--config", "tokuvik-tiny",
                        "--seed", "3", "--std", "0.3", "--norm-std", "0.6"], cwd=ROOT, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    r = subprocess.run([sys.executable, "-m", "wllm_amd.cli", "generate", "--model", str(made), "--dtype", "float32",
                        "--prompt-ids", "5,17,3,200,41", "--max-new-tokens", "6"], cwd=ROOT, capture_output=True, text=True,
                       timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    line = json.loads([x for x in r.stdout.splitlines() if x.startswith("{")][-1])
    raw, w = read_folder(str(made))
    tokens = [5, 17, 3, 200, 41]
    for t in line["token_ids"]:
        logits = plain.forward(raw, w, tokens)[-1]
        if (logits.topk(2).values[0] - logits.topk(2).values[1]).item() < 1e-3:
            break
        assert t == int(logits.argmax())
        tokens.append(t)
    assert len(line["token_ids"]) == 6
