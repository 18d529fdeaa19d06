"""A plain, slow Tasosun forward pass: whole sequences, no cache, no batching.

The oracle of the Tasosun tests.  It shares no code with the engine: it reads config.json
with the `json` module and model.safetensors with the `safetensors` package, and computes
with ordinary torch arithmetic in one floating-point type (float32 or float64), one
function a mechanism.  `round_to=torch.bfloat16` rounds where a bfloat16 model may hold a
tensor (products and activations); everything the design wants in 32-bit stays wide.

The design, in this file's notation (t a token at position p_t, counted from 0):

    x_t       = E[token_t] * s_emb
    layer     : h = N(x);  x <- x + (A(h) + F(h))          (one norm, both sublayers read it)
    N(x)      = x / sqrt(mean(x^2) + eps) * (1 + w)
    A(h)      : q = Wq h + bq;  k = Wk h + bk;  v = k (as projected);  g = sigmoid(Wg h)
                q, k <- R(q), R(k);  q, k <- U(q), U(k)      (per head)
                s_tj = c tanh((q_t . k_j) a / c);   j visible to t iff 0 <= p_t - p_j < W
                o_t = sum_j softmax_j(s_tj) v_j;   A = Wo (g * concat(o)) + bo
    R         : of the first r elements of a head, (u_2i, u_2i+1) turn by the angle
                p * base^(-2i/r) / factor
    U(u)      = u / sqrt(mean(u^2) + eps)
    F(h)      = Wd (silu(Wg h) * (Wu h))
    loop      : layers start..stop-1 run `times` times with the same weights; before every
                pass but the first the embedding output is added to x
    logits    = H N_final(x)
"""
from __future__ import annotations

import json
import math
import os

import torch
from safetensors import safe_open


def read_config(folder: str) -> dict:
    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as f:
        return json.load(f)


def read_weights(folder: str, dtype: torch.dtype = torch.float32) -> dict:
    out = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            out[name] = f.get_tensor(name).to(dtype)
    return out


def _r(t: torch.Tensor, round_to) -> torch.Tensor:
    return t if round_to is None else t.to(round_to).to(t.dtype)


def embedding(table: torch.Tensor, tokens, scale: float) -> torch.Tensor:
    return table[torch.as_tensor(tokens, dtype=torch.long)] * scale


def offset_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * (1 + w): what is stored is the weight's distance from one."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * (1.0 + w)


def unit_norm(u: torch.Tensor, eps: float) -> torch.Tensor:
    """u divided by its root mean square over the last axis; no weight."""
    return u / torch.sqrt((u * u).mean(dim=-1, keepdim=True) + eps)


def rotate_interleaved(u: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """u [tokens, heads, dim]; the first rot['dims'] elements of every head turn, pair (2i, 2i+1) by
    position * base^(-2i/dims) / factor; the rest pass."""
    r = rot["dims"]
    out = u.clone()
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    for i in range(r // 2):
        f = rot["base"] ** (-2.0 * i / r) / factor
        a = positions.to(u.dtype) * f
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        lo, hi = u[..., 2 * i], u[..., 2 * i + 1]
        out[..., 2 * i] = lo * c - hi * s
        out[..., 2 * i + 1] = hi * c + lo * s
    return out


def capped_scores(q: torch.Tensor, k: torch.Tensor, scale: float, softcap) -> torch.Tensor:
    """q [T, d], k [T, d] of one head -> [T, T] scores, scaled and then bent under the cap."""
    s = (q @ k.T) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    return s


def window_mask(positions: torch.Tensor, window) -> torch.Tensor:
    """[T, T] True where query row i sees key column j: 0 <= p_i - p_j < window."""
    d = positions[:, None] - positions[None, :]
    m = d >= 0
    if window:
        m &= d < window
    return m


def attention_mixer(h: torch.Tensor, w: dict, prefix: str, m: dict, eps: float, positions: torch.Tensor,
                    round_to=None) -> torch.Tensor:
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    T = h.shape[0]
    q = _r(h @ w[prefix + "q"].T + w[prefix + "q.b"], round_to).view(T, H, d)
    k = _r(h @ w[prefix + "k"].T + w[prefix + "k.b"], round_to).view(T, G, d)
    v = k                                       # the values are the keys as projected
    gate = torch.sigmoid(_r(h @ w[prefix + "g"].T, round_to))
    if m.get("rot"):
        q, k = rotate_interleaved(q, positions, m["rot"]), rotate_interleaved(k, positions, m["rot"])
    q, k = _r(unit_norm(q, eps), round_to), _r(unit_norm(k, eps), round_to)
    mask = window_mask(positions, (m.get("mask") or {}).get("size"))
    heads = []
    for head in range(H):
        kv = head // (H // G)
        s = capped_scores(q[:, head], k[:, kv], m["scale"], m.get("softcap"))
        s = s.masked_fill(~mask, float("-inf"))
        p = torch.softmax(s, dim=-1)
        heads.append(p @ v[:, kv])
    o = _r(torch.cat(heads, dim=-1), round_to)
    o = _r(o * gate, round_to)
    return _r(o @ w[prefix + "o"].T + w[prefix + "o.b"], round_to)


def dense_feed_forward(h: torch.Tensor, w: dict, prefix: str, round_to=None) -> torch.Tensor:
    g = _r(h @ w[prefix + "gate"].T, round_to)
    u = _r(h @ w[prefix + "up"].T, round_to)
    a = _r(g * torch.sigmoid(g) * u, round_to)
    return _r(a @ w[prefix + "down"].T, round_to)


def layer_runs(config: dict) -> list:
    """[(layer index, the embedding output is added before this run)] in the order the layers run."""
    n = len(config["layers"])
    loop = config.get("loop") or {"start": 0, "stop": 0, "times": 1}
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, False) for i in range(start)]
    for t in range(times):
        runs += [(i, t > 0 and i == start) for i in range(start, stop)]
    runs += [(i, False) for i in range(stop, n)]
    return runs


def forward(config: dict, w: dict, tokens, round_to=None, return_layers: bool = False):
    """Logits [T, vocab] of one whole sequence (and the residual stream after every layer run)."""
    dtype = w["embed"].dtype
    eps = config["norm"]["eps"]
    positions = torch.arange(len(tokens))
    x0 = embedding(w["embed"], tokens, config["embedding"]["scale"])
    x = x0.clone()
    after = []
    for i, add_embedding in layer_runs(config):
        layer = config["layers"][i]
        if add_embedding:
            x = x + x0
        h = _r(offset_norm(x, w[f"l{i}.norm1"], eps), round_to)
        assert layer["type"] == "attention"
        y = attention_mixer(h, w, f"l{i}.mix.", layer["mixer"], eps, positions, round_to)
        if layer.get("mlp") is not None:
            assert layer["mlp"]["kind"] == "dense"
            y = y + dense_feed_forward(h, w, f"l{i}.mlp.", round_to)
        x = x + y
        after.append(x.clone())
    h = _r(offset_norm(x, w["final.norm"], eps), round_to)
    logits = h @ w["head"].T
    return (logits, torch.stack(after)) if return_layers else logits
