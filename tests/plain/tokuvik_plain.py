"""A plain, slow Tokuvik: whole sequences, no cache, one function a mechanism.

Written from the design's equations and sharing nothing with the engine.  Every function takes
and returns torch tensors of one dtype (float64 for an oracle, float32 to see what 32-bit sums
do); `weights` maps tensor names to tensors, `config` is the parsed config.json.

The design: a decoder whose layers are x += post_norm(mixer(pre_norm(x))), then (if the layer
has a feed-forward) x += post_norm(ff(pre_norm(x))), then a per-layer token input; the norms are
layer norms with a weight and no bias.  Three mixers: grouped attention inside chunks of the
sequence with a norm over the whole query and key projections, one gate a head and, optionally,
the keys and values of an earlier layer; latent attention (keys and values expanded from one
compressed vector a token) with a sink in the softmax and an elementwise gate; and the
state-space recurrence of Mamba-2 with its short convolution and gated group norm.
"""
from __future__ import annotations

import math

import torch


def layer_norm(x, w, eps):
    mean = x.mean(-1, keepdim=True)
    dev = x - mean
    var = (dev * dev).mean(-1, keepdim=True)
    return dev / torch.sqrt(var + eps) * w


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    # log(1 + e^z), stable for large |z|
    return torch.where(z > 0, z + torch.log1p(torch.exp(-z.abs())), torch.log1p(torch.exp(-z.abs())))


def chunk_mask(t: int, size):
    """[t, t] bool: query i sees key j iff j <= i and both lie in the same chunk of `size`
    positions counted from 0 (size None: plain causal)."""
    i = torch.arange(t)[:, None]
    j = torch.arange(t)[None, :]
    seen = j <= i
    if size is not None:
        seen = seen & ((i // size) == (j // size))
    return seen


def softmax_with_sink(scores, seen, sink=None):
    """Softmax over the seen keys of each row; with `sink` ([heads], broadcast over rows) the
    denominator holds exp(sink) once more.  scores [heads, t, t]."""
    scores = scores.masked_fill(~seen, float("-inf"))
    m = scores.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink[:, None, None])
    e = torch.exp(scores - m)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink[:, None, None] - m)
    return e / den


def attention_keys_values(h, w, p, mixer, eps):
    """The (normed) keys and the values that a layer's cache holds: [t, kv_heads, dim], [t, kv_heads, vdim]."""
    t = h.shape[0]
    k = rms_norm(h @ w[p + "k"].T, w[p + "k.norm"], eps)
    v = h @ w[p + "v"].T
    return k.view(t, mixer["kv_heads"], mixer["dim"]), v.view(t, mixer["kv_heads"], mixer["vdim"])


def attention_mixer(h, w, p, mixer, eps, keys_values):
    """h [t, width]; `keys_values`: this layer's own or, with kv_from, the named layer's."""
    t = h.shape[0]
    heads, kvh, dim, vdim = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    q = rms_norm(h @ w[p + "q"].T, w[p + "q.norm"], eps).view(t, heads, dim)
    k, v = keys_values
    rep = heads // kvh
    k = k.repeat_interleave(rep, dim=1)
    v = v.repeat_interleave(rep, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, k) * mixer["scale"]
    size = (mixer.get("mask") or {}).get("size")
    weights = softmax_with_sink(scores, chunk_mask(t, size))
    out = torch.einsum("hij,jhd->ihd", weights, v)
    gate = torch.sigmoid(h @ w[p + "g"].T)                 # [t, heads]
    out = out * gate[:, :, None]
    return out.reshape(t, heads * vdim) @ w[p + "o"].T


def latent_attention_mixer(h, w, p, mixer, eps):
    t = h.shape[0]
    heads, dim, vdim = mixer["heads"], mixer["dim"], mixer["vdim"]
    cq = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].T).view(t, heads, dim)
    c = rms_norm(h @ w[p + "dkv"].T, w[p + "dkv.norm"], eps)
    k = (c @ w[p + "uk"].T).view(t, heads, dim)
    v = (c @ w[p + "uv"].T).view(t, heads, vdim)
    scores = torch.einsum("ihd,jhd->hij", q, k) * mixer["scale"]
    weights = softmax_with_sink(scores, chunk_mask(t, None), w[p + "sink"])
    out = torch.einsum("hij,jhd->ihd", weights, v).reshape(t, heads * vdim)
    out = out * torch.sigmoid(h @ w[p + "g"].T)
    return out @ w[p + "o"].T


def causal_conv(u, weight, bias):
    """u [t, channels]; weight [channels, taps], the last column the current token's; zeros before
    the start."""
    t, taps = u.shape[0], weight.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, u.shape[1], dtype=u.dtype), u], dim=0)
    out = bias.expand(t, -1).clone()
    for k in range(taps):
        out = out + padded[k:k + t] * weight[:, k]
    return out


def state_space_recurrence(x, b, c, dt, a_log, d_skip, state=None):
    """x [t, heads, p]; b, c [t, groups, n]; dt [t, heads] (after softplus); a_log, d_skip [heads].
    S_t = exp(-exp(a_log) dt_t) S_(t-1) + dt_t B_t x_t^T;  y_t = S_t^T C_t + d_skip x_t.  Returns y [t, heads, p]
    and the last S [heads, n, p]; `state`: the S to start from (zeros if None)."""
    t, heads, p = x.shape
    per_group = heads // b.shape[1]
    decay = torch.exp(-torch.exp(a_log) * dt)
    s = torch.zeros(heads, b.shape[2], p, dtype=x.dtype) if state is None else state
    ys = []
    for i in range(t):
        bi = b[i].repeat_interleave(per_group, dim=0)      # [heads, n]
        ci = c[i].repeat_interleave(per_group, dim=0)
        s = decay[i][:, None, None] * s + dt[i][:, None, None] * bi[:, :, None] * x[i][:, None, :]
        ys.append(torch.einsum("hnp,hn->hp", s, ci) + d_skip[:, None] * x[i])
    return torch.stack(ys), s


def gated_group_norm(y, z, w, parts: int, eps):
    """y * silu(z), each of `parts` equal parts of a row divided by its own root mean square, times w."""
    t, width = y.shape
    v = (y * silu(z)).view(t, parts, width // parts)
    v = v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)
    return v.reshape(t, width) * w


def mamba2_mixer(h, w, p, mixer, eps):
    t = h.shape[0]
    heads, vdim, n, groups = mixer["heads"], mixer["vdim"], mixer["state"], mixer["groups"]
    inner = heads * vdim
    row = h @ w[p + "in"].T
    z, xbc, dt = row[:, :inner], row[:, inner:2 * inner + 2 * groups * n], row[:, 2 * inner + 2 * groups * n:]
    xbc = silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].view(t, heads, vdim)
    b = xbc[:, inner:inner + groups * n].view(t, groups, n)
    c = xbc[:, inner + groups * n:].view(t, groups, n)
    dt = softplus(dt + w[p + "dt_bias"])                   # [t, heads]
    y, _ = state_space_recurrence(x, b, c, dt, w[p + "A_log"], w[p + "D"])
    y = gated_group_norm(y.reshape(t, inner), z, w[p + "norm"], mixer["norm_groups"], eps)
    return y @ w[p + "o"].T


def dense_feed_forward(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def token_side(x, tokens, w, p, layer: int, dim: int, eps):
    e = w["side.embed"][tokens][:, layer * dim:(layer + 1) * dim]
    g = gelu_tanh(x @ w[p + "side.gate"].T) * e
    y = g @ w[p + "side.proj"].T
    return rms_norm(y, w[p + "side.norm"], eps)


def forward(config: dict, weights: dict, tokens, dtype=torch.float64, return_layers: bool = False):
    """Logits [t, vocab] of one whole sequence (and, if asked, the stream after every layer)."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = config["norm"]["eps"]
    side = config.get("token_side")
    x = w["embed"][tokens]
    kept = {}
    streams = []
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        mixer = layer["mixer"]
        h = layer_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "attention":
            src = mixer.get("kv_from")
            if src is None:
                kept[i] = attention_keys_values(h, w, p + "mix.", mixer, eps)
                src = i
            y = attention_mixer(h, w, p + "mix.", mixer, eps, kept[src])
        elif layer["type"] == "latent_attention":
            y = latent_attention_mixer(h, w, p + "mix.", mixer, eps)
        elif layer["type"] == "mamba2":
            y = mamba2_mixer(h, w, p + "mix.", mixer, eps)
        else:
            raise ValueError(layer["type"])
        x = x + layer_norm(y, w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = layer_norm(x, w[p + "norm2"], eps)
            x = x + layer_norm(dense_feed_forward(h, w, p + "mlp."), w[p + "norm2b"], eps)
        if side:
            x = x + token_side(x, tokens, w, p, i, side["dim"], eps)
        streams.append(x)
    logits = layer_norm(x, w["final.norm"], eps) @ w["embed"].T
    return (logits, torch.stack(streams)) if return_layers else logits
