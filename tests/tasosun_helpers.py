"""Shared by the Tasosun tests: small configurations that differ in every size and option, model
folders with random weights, and the comparison with the plain implementation."""
from __future__ import annotations

import copy

import torch

from plain import tasosun_plain
from wllm_amd.parts import write_random_model_from_config_json


def attention(heads, kv_heads, dim, *, rot=None, window=None, softcap=None, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale if scale is not None else dim ** -0.5}
    if rot is not None:
        dims, base, factor = rot
        m["rot"] = {"dims": dims, "base": base, "scaling": {"factor": factor}}
    if window is not None:
        m["mask"] = {"size": window}
    if softcap is not None:
        m["softcap"] = softcap
    return m


def layer(mixer, ff):
    return {"type": "attention", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def config(vocab, width, layers, *, loop=None, eps=1e-6, emb=1.0):
    c = {"architecture": "Tasosun", "vocab": vocab, "width": width, "embedding": {"scale": emb}, "norm": {"eps": eps},
         "layers": layers}
    if loop is not None:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    return c


# Head sizes 32 and 64 (the matrix-core kernels), a layer without a feed-forward, layers of unlike
# sizes, the whole head rotated in one layer and a quarter of it in the other, a span of two layers
# that runs three times after a layer that runs once.
MIXED = dict(page_size=16, seed=5, std=0.08, norm_std=0.2, config=config(160, 64, [
    layer(attention(4, 2, 32, rot=(32, 10000.0, 1.0), window=24, softcap=30.0, scale=0.4), 96),
    layer(attention(2, 1, 64, rot=(16, 500.0, 4.0), window=40, softcap=20.0), None),
    layer(attention(4, 4, 32, rot=(8, 3000.0, 1.5), window=9, softcap=12.0, scale=0.9), 48),
], loop=(1, 3, 3), eps=1e-5, emb=1.7))

# Head sizes the matrix-core kernels do not take (20 and 12), pages of 8, no loop at all, a window
# longer than any request of the tests, one key/value head a query head, a width that is no multiple of 32.
ODD = dict(page_size=8, seed=6, std=0.1, norm_std=0.1, config=config(97, 48, [
    layer(attention(3, 3, 20, rot=(8, 77.0, 2.0), window=7, softcap=5.0, scale=1.3), 40),
    layer(attention(6, 2, 12, rot=(12, 10000.0, 8.0), window=500, softcap=8.0, scale=0.7), 72),
], eps=1e-6, emb=0.5))

# Attention so sharp that single keys decide (scores reach the cap): a key lost at a window's edge,
# a wrong page or a stale slot moves the logits by far more than any rounding.  All layers loop.
SHARP = dict(page_size=16, seed=7, std=0.1, norm_std=0.1, config=config(200, 96, [
    layer(attention(4, 1, 32, rot=(16, 100.0, 2.0), window=16, softcap=40.0, scale=2.5), 128),
    layer(attention(4, 1, 32, rot=(16, 100.0, 2.0), window=21, softcap=40.0, scale=2.5), 128),
    layer(attention(2, 2, 64, rot=(32, 100.0, 1.0), window=33, softcap=25.0, scale=1.5), 64),
], loop=(0, 3, 2), eps=1e-6, emb=3.0))

# A large head (160), a window of one (a token sees itself alone), no cap in one layer, a loop that is
# empty (start = stop), pages of 4.
WIDE = dict(page_size=4, seed=8, std=0.06, norm_std=0.1, config=config(120, 80, [
    layer(attention(2, 2, 160, rot=(40, 50000.0, 1.0), window=1, softcap=15.0), 56),
    layer(attention(2, 1, 160, rot=(160, 50000.0, 3.0), window=130, scale=0.2), 56),
], loop=(1, 1, 4), eps=1e-4, emb=2.0))

# Heads of 6 and 10 elements (no multiple of four: the engine pads them), an odd width and vocabulary, every
# size 1 that can be (one head, one layer in the loop, a loop of one time).
SMALL = dict(page_size=16, seed=9, std=0.15, norm_std=0.1, config=config(53, 30, [
    layer(attention(1, 1, 6, rot=(4, 20.0, 1.0), window=5, softcap=9.0, scale=1.1), 22),
    layer(attention(4, 2, 10, rot=(10, 900.0, 16.0), window=64, softcap=11.0, scale=0.8), 34),
], loop=(1, 2, 1), eps=1e-6, emb=1.0))

CONFIGS = {"mixed": MIXED, "odd": ODD, "sharp": SHARP, "wide": WIDE, "small": SMALL}


def random_config(seed: int) -> dict:
    """A configuration drawn at random from what the design allows: sizes, head counts, order and sizes of the
    layers, windows, constants, the loop."""
    import random
    r = random.Random(seed)
    width = r.choice([24, 32, 48, 64, 72, 96, 128, 160])
    layers = []
    for _ in range(r.randint(1, 4)):
        kv = r.choice([1, 1, 2, 3, 4])
        heads = kv * r.choice([1, 1, 2, 3, 4, 8])
        dim = r.choice([6, 8, 12, 16, 20, 24, 32, 32, 40, 48, 64, 64, 96, 128])
        rot = None if r.random() < 0.1 else (2 * r.randint(1, dim // 2), r.choice([100.0, 10000.0, 1e6]), r.choice([1.0, 2.0, 8.0, 32.0]))
        window = None if r.random() < 0.1 else r.choice([1, 2, 5, 16, 17, 31, 32, 33, 64, 80, 200])
        softcap = None if r.random() < 0.1 else r.choice([5.0, 15.0, 30.0, 50.0])
        scale = dim ** -0.5 * r.choice([0.5, 1.0, 1.0, 4.0, 12.0])
        layers.append(layer(attention(heads, kv, dim, rot=rot, window=window, softcap=softcap, scale=scale),
                            None if r.random() < 0.2 else r.choice([24, 64, 100, 192, 256])))
    loop = None
    if r.random() < 0.8:
        start = r.randint(0, len(layers))
        stop = r.randint(start, len(layers))
        loop = (start, stop, r.randint(1, 3))
    return dict(page_size=16, seed=seed, std=r.choice([0.05, 0.1, 0.2]), norm_std=0.1,
                config=config(r.choice([50, 97, 256, 300, 1000]), width, layers, loop=loop, eps=r.choice([1e-6, 1e-5]),
                              emb=r.choice([0.5, 1.0, 3.0, 8.0])))


def middling_config(seed: int) -> dict:
    """Layers of some hundred columns, windows of about a hundred keys, a loop: sizes at which a request of a
    thousand tokens crosses many windows, pages and chunks of keys."""
    import random
    r = random.Random(1000 + seed)
    width = r.choice([192, 256, 384, 512])
    kinds = []
    for _ in range(r.randint(1, 2)):        # one or two kinds of layer, repeated
        kv = r.choice([1, 2, 4])
        heads = kv * r.choice([1, 2, 3, 6, 12])
        dim = r.choice([48, 64, 80, 112, 128])
        kinds.append(layer(attention(heads, kv, dim, rot=(2 * r.randint(4, dim // 2), r.choice([10000.0, 500000.0]), r.choice([1.0, 4.0, 8.0])),
                                     window=r.choice([64, 65, 100, 127, 128, 160]), softcap=r.choice([20.0, 50.0]),
                                     scale=dim ** -0.5 * r.choice([1.0, 3.0])), r.choice([None, 256, 512, 640])))
    layers = [copy.deepcopy(kinds[i % len(kinds)]) for i in range(r.randint(3, 6))]
    start = r.randint(0, len(layers) - 1)
    return dict(page_size=16, seed=seed, std=0.06, norm_std=0.1,
                config=config(r.choice([300, 512, 777]), width, layers, loop=(start, r.randint(start + 1, len(layers)), r.randint(2, 3)),
                              eps=1e-6, emb=r.choice([1.0, 3.0])))


def write_folder(name, folder: str) -> str:
    c = CONFIGS[name] if isinstance(name, str) else name
    return write_random_model_from_config_json(folder, copy.deepcopy(c["config"]), c["seed"], std=c["std"],
                                               norm_std=c["norm_std"])


def random_ids(seed: int, length: int, vocab: int) -> list:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (length,), generator=g).tolist()


def requests_for(name, lengths) -> dict:
    vocab = (CONFIGS[name] if isinstance(name, str) else name)["config"]["vocab"]
    salt = len(name) if isinstance(name, str) else 3
    return {f"q{i}": random_ids(1000 * i + salt, n, vocab) for i, n in enumerate(lengths)}


def plain_logits(folder: str, requests: dict, dtype=torch.float64, round_to=None) -> dict:
    cfg = tasosun_plain.read_config(folder)
    w = tasosun_plain.read_weights(folder, dtype)
    return {rid: tasosun_plain.forward(cfg, w, toks, round_to=round_to) for rid, toks in requests.items()}


def _centred_rms(d: torch.Tensor) -> float:
    d = d.double()
    return (d - d.mean()).pow(2).mean().sqrt().item()


def compare_rows(collected: dict, exact: dict, rounded: dict = None, *, float32_relative: float = 2e-5) -> float:
    """Every collected row against the plain implementation's exact row.  A row's error is the root mean
    square of the difference with its mean taken off.  float32 (`rounded` None): the error may be
    `float32_relative` of the exact row's own root mean square.  bfloat16: three times what rounding
    alone does to the plain implementation (the farthest row of the same request, `rounded` against
    `exact`).  Returns the worst error in units of its bound and names the first row beyond it."""
    worst = 0.0
    for (rid, pos) in sorted(collected, key=lambda k: (str(k[0]), k[1])):
        got, ref = collected[(rid, pos)].double(), exact[rid][pos].double()
        assert torch.isfinite(got).all(), f"request {rid!r} position {pos}: logits are not finite"
        if rounded is None:
            bound = float32_relative * max(_centred_rms(ref), 1e-3)
        else:
            bound = 3.0 * max(_centred_rms(rounded[rid][p] - exact[rid][p]) for p in range(len(exact[rid])))
        err = _centred_rms(got - ref) / bound
        assert err <= 1.0, f"request {rid!r} position {pos}: {err:.2f} x the bound ({_centred_rms(got - ref):.3e} against {bound:.3e})"
        worst = max(worst, err)
    return worst
