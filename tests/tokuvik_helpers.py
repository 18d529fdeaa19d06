"""Shared by the Tokuvik tests: small configurations that differ in every size and option, model
folders whose weights make every mechanism count, and the comparison with the plain implementation."""
from __future__ import annotations

import copy
import json
import os

import torch

from plain import tokuvik_plain
from wllm_amd.parts import build_model
from wllm_amd.weights.safetensors_io import write_safetensors


def attention(heads, kv_heads, dim, vdim, *, chunk=None, scale=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if chunk is not None:
        m["mask"] = {"size": chunk}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def latent(heads, dim, vdim, q_rank, kv_rank, *, scale=None):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank,
                                                  "kv_rank": kv_rank, "scale": scale if scale is not None else dim ** -0.5}}


def mamba(heads, vdim, state, groups, conv, norm_groups):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}}


def layer(mixer, ff):
    return dict(mixer, mlp=None if ff is None else {"kind": "dense", "ff": ff})


def config(vocab, width, layers, *, side=None, eps=1e-6):
    c = {"architecture": "Tokuvik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if side is not None:
        c["token_side"] = {"dim": side}
    return c


# Matrix-core head sizes (the padded head is 32 or 64), all three mixers, a layer that reads the first
# layer's keys with the same chunks (pages go back chunk by chunk), a layer without a feed-forward.
TRIO = dict(page_size=16, seed=11, config=config(150, 64, [
    layer(attention(4, 2, 32, 16, chunk=24, scale=0.5), 96),
    layer(latent(4, 16, 24, 40, 32), 80),
    layer(mamba(4, 16, 16, 2, 4, 2), None),
    layer(attention(4, 2, 32, 16, chunk=24, scale=0.3, kv_from=0), 96),
    layer(mamba(2, 40, 24, 1, 3, 1), 64),
], side=8, eps=1e-5))

# Sizes no matrix-core kernel takes, pages of 8, a width that is no multiple of 32, no token input, values
# wider than keys, a layer that reads another's keys under another mask (the cache keeps everything), an
# attention layer without a mask, a convolution of two taps and one of one, groups and heads that are 1.
ODD = dict(page_size=8, seed=12, config=config(97, 48, [
    layer(attention(3, 3, 20, 28, chunk=7, scale=0.9), 40),
    layer(mamba(3, 10, 7, 3, 2, 3), 56),
    layer(attention(3, 3, 20, 28, chunk=19, scale=0.6, kv_from=0), None),
    layer(latent(3, 12, 20, 12, 20, scale=0.8), 40),
    layer(attention(6, 1, 12, 8), 40),
    layer(mamba(1, 36, 5, 1, 1, 1), None),
], eps=1e-6))

# Attention so sharp that single keys decide: a key lost or gained at a chunk's edge, a stale slot, a
# wrong page or a sink left out moves the logits by far more than rounding.
SHARP = dict(page_size=16, seed=13, sharp=True, config=config(200, 96, [
    layer(attention(4, 1, 32, 32, chunk=16, scale=6.0), 128),
    layer(latent(4, 32, 32, 48, 64, scale=1.5), 128),
    layer(attention(2, 2, 64, 32, chunk=21, scale=4.0), 64),
    layer(attention(4, 1, 32, 32, chunk=16, scale=6.0, kv_from=0), None),
    layer(mamba(6, 16, 32, 2, 4, 3), 64),
], side=16, eps=1e-6))

CONFIGS = {"trio": TRIO, "odd": ODD, "sharp": SHARP}


def middling_config(seed: int) -> dict:
    """Widths of some hundred and heads as a small real model has them: the sizes at which steps of a few hundred
    rows take the library's products, the tiled kernels and the matrix-core attention."""
    import random
    r = random.Random(seed)
    width = r.choice([256, 384, 512])
    kv = r.choice([1, 2])
    dim, vdim = r.choice([(64, 96), (128, 64), (64, 64)])
    chunk = r.choice([130, 200, 333])
    heads = kv * r.choice([2, 4])
    groups = r.choice([1, 2])
    layers = [
        layer(attention(heads, kv, dim, vdim, chunk=chunk, scale=dim ** -0.5), r.choice([768, 1024])),
        layer(latent(r.choice([4, 8]), r.choice([32, 48]), r.choice([32, 64]), r.choice([96, 192]), r.choice([96, 128, 160])), 768),
        layer(mamba(groups * r.choice([4, 6]), r.choice([32, 64]), r.choice([32, 64, 100]), groups, 4, groups), r.choice([None, 768])),
        layer(attention(heads * 2, kv, dim, vdim, chunk=r.choice([chunk, None]), scale=dim ** -0.5, kv_from=0), 768),
    ]
    r.shuffle(layers)
    # the reader must come behind the layer it reads: put the owner first again
    owner = next(i for i, l in enumerate(layers) if l["type"] == "attention" and "kv_from" not in l["mixer"])
    reader = next(i for i, l in enumerate(layers) if l["mixer"].get("kv_from") is not None)
    if reader < owner:
        layers[owner], layers[reader] = layers[reader], layers[owner]
        owner = reader
    for l in layers:
        if l["mixer"].get("kv_from") is not None:
            l["mixer"]["kv_from"] = owner
    return dict(page_size=16, seed=seed, config=config(r.choice([1000, 2048]), width, layers, side=r.choice([16, 32]), eps=1e-6))


def random_config(seed: int) -> dict:
    """A configuration drawn from what the design allows: any order of mixers, any sizes."""
    import random
    r = random.Random(seed)
    width = r.choice([32, 48, 64, 80])
    layers, owners = [], []
    for i in range(r.randint(2, 5)):
        kind = r.choice(["attention", "attention", "latent", "mamba"])
        ff = r.choice([None, 32, 72])
        if kind == "attention":
            if owners and r.random() < 0.4:
                src = r.choice(owners)
                m = layers[src]["mixer"]
                group = r.choice([g for g in (1, 2, 3) if True])
                layers.append(layer(attention(m["kv_heads"] * group, m["kv_heads"], m["dim"], m["vdim"],
                                              chunk=r.choice([None, 5, 16, 33]), scale=r.choice([0.3, 1.0]), kv_from=src), ff))
            else:
                kv = r.choice([1, 2, 3])
                layers.append(layer(attention(kv * r.choice([1, 2, 4]), kv, r.choice([8, 20, 32, 64]), r.choice([4, 16, 32, 40]),
                                              chunk=r.choice([None, 5, 16, 33]), scale=r.choice([0.3, 1.0])), ff))
                owners.append(i)
        elif kind == "latent":
            layers.append(layer(latent(r.choice([1, 2, 5]), r.choice([8, 16, 24]), r.choice([8, 12, 32]), r.choice([8, 24, 40]),
                                       r.choice([8, 20, 32, 64])), ff))
        else:
            groups = r.choice([1, 2])
            heads = groups * r.choice([1, 2, 3])
            vdim = r.choice([4, 16, 24, 72])
            ng = r.choice([g for g in (1, 2, heads) if (heads * vdim) % g == 0])
            layers.append(layer(mamba(heads, vdim, r.choice([3, 16, 40]), groups, r.choice([1, 2, 4, 5]), ng), ff))
    return dict(page_size=r.choice([4, 8, 16]), seed=seed,
                config=config(r.choice([64, 130, 300]), width, layers, side=r.choice([None, 4, 12]), eps=r.choice([1e-6, 1e-5])))


def _draw(name: str, shape: tuple, seed: int, sharp: bool) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    n = torch.randn(shape, generator=g)
    last = name.rsplit(".", 1)[-1]
    if name.endswith(("norm1", "norm2", "norm1b", "norm2b", "final.norm", "side.norm", "mix.norm")) or name.endswith(".norm"):
        t = 1.0 + 0.3 * n                       # plain weights around one
    elif last == "A_log":
        t = -0.5 + 0.8 * n                      # decays from almost 1 to almost 0 over a few tokens
    elif last == "dt_bias":
        t = 0.3 * n
    elif last == "D":
        t = 1.0 + 0.3 * n
    elif last == "sink":
        t = (16.0 if sharp else 0.5) + n        # a sink that carries weight beside the sharpest scores
    elif last == "conv":
        t = 0.5 * n
    elif last == "b":
        t = 0.2 * n
    elif name in ("embed", "side.embed"):
        t = n
    else:
        t = n * (shape[-1] ** -0.5)             # a projection keeps its input's size
    return t.to(torch.bfloat16)


def write_folder(name, folder: str) -> str:
    """A model folder for one of CONFIGS (or a dict of the same form): config.json and weights that make
    every part count (norm weights around one, decays between 0 and 1, a sink of some weight)."""
    c = CONFIGS[name] if isinstance(name, str) else name
    raw = copy.deepcopy(c["config"])
    # (a generator keyed by a stable hash of the seed and the tensor's name: the python hash of a string differs from run to run)
    import hashlib
    expected = build_model(copy.deepcopy(raw)).expected_tensors()
    tensors = {}
    for tensor_name, exp in expected.items():
        stable = int.from_bytes(hashlib.sha256(f"{c['seed']}:{tensor_name}".encode()).digest()[:4], "little")
        tensors[tensor_name] = _draw(tensor_name, tuple(exp.shape), stable, bool(c.get("sharp")))
    os.makedirs(folder, exist_ok=True)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors, metadata={"format": "pt"})
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(raw, f, indent=1, sort_keys=True)
    return folder


def read_folder(folder: str, dtype=torch.float64):
    from wllm_amd.weights.checkpoint import Checkpoint
    with open(os.path.join(folder, "config.json"), encoding="utf-8") as f:
        raw = json.load(f)
    ck = Checkpoint(folder)
    try:
        weights = {n: ck.tensor(n).to(dtype).clone() for n in ck.names()}
    finally:
        ck.close()
    return raw, weights


def random_ids(seed: int, length: int, vocab: int) -> list:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (length,), generator=g).tolist()


def requests_for(name, lengths) -> dict:
    c = CONFIGS[name] if isinstance(name, str) else name
    return {f"q{i}": random_ids(1000 * i + c["seed"], n, c["config"]["vocab"]) for i, n in enumerate(lengths)}


def plain_logits(folder: str, requests: dict, dtype=torch.float64) -> dict:
    raw, weights = read_folder(folder, dtype)
    return {rid: tokuvik_plain.forward(raw, weights, toks, dtype) for rid, toks in requests.items()}


def _centred_rms(d: torch.Tensor) -> float:
    d = d.double()
    return (d - d.mean()).pow(2).mean().sqrt().item()


def compare_rows(collected: dict, exact: dict, *, relative: float, outliers: float = 0.0, ceiling: float = 1.0) -> float:
    """Every collected row against the plain implementation's: the root mean square of the difference,
    its mean taken off, may be `relative` of the exact row's own.  bfloat16 rounding now and then decides
    between two keys of almost equal score, and the row is then far off though nothing is wrong: a share
    `outliers` of the rows may lie beyond the bound, up to `ceiling` times it.  Returns the worst error in
    units of the bound and names the first row beyond what is allowed."""
    errors = {}
    for (rid, pos) in sorted(collected, key=lambda k: (str(k[0]), k[1])):
        got, ref = collected[(rid, pos)].double(), exact[rid][pos].double()
        assert torch.isfinite(got).all(), f"request {rid!r} position {pos}: logits are not finite"
        bound = relative * max(_centred_rms(ref), 1e-3)
        errors[(rid, pos)] = _centred_rms(got - ref) / bound
    beyond = {k: e for k, e in errors.items() if e > 1.0}
    worst = max(errors.values())
    assert len(beyond) <= outliers * len(errors), (
        f"{len(beyond)} of {len(errors)} rows beyond the bound; the first: request {next(iter(beyond))[0]!r} position "
        f"{next(iter(beyond))[1]}: {next(iter(beyond.values())):.2f} x the bound")
    assert worst <= max(ceiling, 1.0), f"a row is {worst:.2f} x the bound"
    return worst
