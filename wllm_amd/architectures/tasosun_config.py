"""Typed configuration of Tasosun, read from its config.json.

The file is nested where Gemma's is flat: `architecture` (one name), `vocab`, `width`,
`embedding.scale`, `norm.eps`, `layers` (a list; every entry has `type`, the sizes and
constants of its mixer under `mixer`, and its feed-forward under `mlp`, or null for none) and
`loop` (`start`, `stop`, `times`: the layers start .. stop-1 run `times` times in a row).
Every layer carries its own sizes, so two layers of one model may differ in all of them.
Nothing has a default that a model could rely on silently: a key the design needs and the
file lacks is an error.  A key that this code does not know is named in a warning
(`UnknownConfigKey`) and otherwise ignored: it may be a note of whoever wrote the file, or an
option of a later version of the design, which would then compute something else.
"""
from __future__ import annotations

import warnings
from dataclasses import dataclass
from typing import Optional

from wllm_amd.config.registry import ConfigError


class UnknownConfigKey(UserWarning):
    """config.json holds a key that the implementation does not read."""


def _positive_int(where: str, v) -> int:
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"{where} must be a positive integer, got {v!r}")
    return v


def _number(where: str, v, positive: bool = True) -> float:
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (positive and not v > 0) or v < 0:
        raise ConfigError(f"{where} must be a {'positive' if positive else 'non-negative'} number, got {v!r}")
    return float(v)


def _section(where: str, raw, required: tuple, optional: tuple = ()) -> dict:
    if not isinstance(raw, dict):
        raise ConfigError(f"{where} must be an object, got {raw!r}")
    missing = [k for k in required if k not in raw]
    if missing:
        raise ConfigError(f"{where} lacks required key(s): {', '.join(missing)}")
    unknown = sorted(set(raw) - set(required) - set(optional))
    if unknown:
        warnings.warn(f"{where} has key(s) this implementation does not read: {', '.join(unknown)}", UnknownConfigKey,
                      stacklevel=3)
    return raw


@dataclass(frozen=True)
class TasosunRotation:
    dims: int                       # the first `dims` elements of a head turn
    base: float
    scaling_factor: float = 1.0     # linear scaling: frequencies divided by it


@dataclass(frozen=True)
class TasosunAttention:
    heads: int
    kv_heads: int
    dim: int                        # query/key size of a head
    vdim: int                       # value size of a head (the values are the keys: equal to dim)
    scale: float
    softcap: Optional[float]
    window: Optional[int]           # mask.size: a position sees itself and the window - 1 before it
    rotation: Optional[TasosunRotation]

    @classmethod
    def from_dict(cls, where: str, raw) -> "TasosunAttention":
        raw = _section(where, raw, ("heads", "kv_heads", "dim", "vdim", "scale"), ("softcap", "mask", "rot"))
        heads, kv_heads = _positive_int(f"{where}.heads", raw["heads"]), _positive_int(f"{where}.kv_heads", raw["kv_heads"])
        dim, vdim = _positive_int(f"{where}.dim", raw["dim"]), _positive_int(f"{where}.vdim", raw["vdim"])
        if heads % kv_heads:
            raise ConfigError(f"{where}: heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        if vdim != dim:
            raise ConfigError(f"{where}: the values are the keys, so vdim ({vdim}) must equal dim ({dim})")
        window = None
        if raw.get("mask") is not None:
            window = _positive_int(f"{where}.mask.size", _section(f"{where}.mask", raw["mask"], ("size",))["size"])
        rotation = None
        if raw.get("rot") is not None:
            rot = _section(f"{where}.rot", raw["rot"], ("dims", "base"), ("scaling",))
            dims = _positive_int(f"{where}.rot.dims", rot["dims"])
            if dims % 2 or dims > dim:
                raise ConfigError(f"{where}.rot.dims must be even and at most dim ({dim}), got {dims}")
            factor = 1.0
            if rot.get("scaling") is not None:
                factor = _number(f"{where}.rot.scaling.factor",
                                 _section(f"{where}.rot.scaling", rot["scaling"], ("factor",))["factor"])
            rotation = TasosunRotation(dims, _number(f"{where}.rot.base", rot["base"]), factor)
        softcap = None if raw.get("softcap") is None else _number(f"{where}.softcap", raw["softcap"])
        return cls(heads, kv_heads, dim, vdim, _number(f"{where}.scale", raw["scale"]), softcap, window, rotation)


@dataclass(frozen=True)
class TasosunLayer:
    attention: TasosunAttention
    ff: Optional[int]               # width of the dense feed-forward, None for a layer without one


@dataclass(frozen=True)
class TasosunConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: tuple
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    raw: Optional[dict] = None      # the file's contents, written back as they were

    @classmethod
    def from_dict(cls, raw: dict) -> "TasosunConfig":
        raw = _section("config.json", raw, ("vocab", "width", "embedding", "norm", "layers"), ("architecture", "architectures", "loop"))
        layers = []
        if not isinstance(raw["layers"], list) or not raw["layers"]:
            raise ConfigError("config.json: layers must be a list with at least one layer")
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            entry = _section(where, entry, ("type", "mixer"), ("mlp",))
            if entry["type"] != "attention":
                raise ConfigError(f"{where}.type {entry['type']!r}: this design's mixers are: attention")
            ff = None
            if entry.get("mlp") is not None:
                mlp = _section(f"{where}.mlp", entry["mlp"], ("kind", "ff"))
                if mlp["kind"] != "dense":
                    raise ConfigError(f"{where}.mlp.kind {mlp['kind']!r}: this design's feed-forwards are: dense")
                ff = _positive_int(f"{where}.mlp.ff", mlp["ff"])
            layers.append(TasosunLayer(TasosunAttention.from_dict(f"{where}.mixer", entry["mixer"]), ff))
        start, stop, times = 0, 0, 1
        if raw.get("loop") is not None:
            loop = _section("loop", raw["loop"], ("start", "stop", "times"))
            start, stop, times = loop["start"], loop["stop"], loop["times"]
            for k, v in (("start", start), ("stop", stop)):
                if isinstance(v, bool) or not isinstance(v, int) or not 0 <= v <= len(layers):
                    raise ConfigError(f"loop.{k} must be an integer from 0 to the number of layers, got {v!r}")
            _positive_int("loop.times", times)
            if stop < start:
                raise ConfigError(f"loop.stop ({stop}) lies before loop.start ({start})")
        return cls(
            vocab=_positive_int("vocab", raw["vocab"]), width=_positive_int("width", raw["width"]),
            embedding_scale=_number("embedding.scale", _section("embedding", raw["embedding"], ("scale",))["scale"]),
            norm_eps=_number("norm.eps", _section("norm", raw["norm"], ("eps",))["eps"], positive=False),
            layers=tuple(layers), loop_start=start, loop_stop=stop, loop_times=times, raw=raw)

    def runs(self) -> list:
        """[(layer, whether the embedding output is added before this run)] in the order the layers run."""
        out = [(i, False) for i in range(self.loop_start)]
        for t in range(self.loop_times if self.loop_stop > self.loop_start else 1):
            out += [(i, t > 0 and i == self.loop_start) for i in range(self.loop_start, self.loop_stop)]
        return out + [(i, False) for i in range(self.loop_stop, len(self.layers))]

    def to_dict(self) -> dict:
        """The config.json of this configuration."""
        if self.raw is not None:
            return dict(self.raw)
        layers = []
        for layer in self.layers:
            a = layer.attention
            mixer = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale}
            if a.softcap is not None:
                mixer["softcap"] = a.softcap
            if a.window is not None:
                mixer["mask"] = {"size": a.window}
            if a.rotation is not None:
                mixer["rot"] = {"dims": a.rotation.dims, "base": a.rotation.base,
                                "scaling": {"factor": a.rotation.scaling_factor}}
            layers.append({"type": "attention", "mixer": mixer,
                           "mlp": None if layer.ff is None else {"kind": "dense", "ff": layer.ff}})
        return {"architecture": "Tasosun", "vocab": self.vocab, "width": self.width,
                "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps}, "layers": layers,
                "loop": {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}}
