"""Typed configuration of Tokuvik, read from its config.json.

The file is nested: `architecture`, `vocab`, `width`, `norm.eps`, `token_side.dim` (absent or null: the
layers have no token input) and `layers`, a list whose entries carry `type` (which mixer: `attention`,
`latent_attention` or `mamba2`), the mixer's sizes and constants under `mixer`, and the feed-forward
under `mlp` (`kind` = `dense` with `ff`), or null for a layer without one.  Every layer carries its own
sizes, so two layers of one model may differ in all of them, and the order of the mixers is the
file's.  A key the design needs and the file lacks is an error; a key this code does not read is
named in a warning (`UnknownConfigKey`).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from wllm_amd.architectures.tasosun_config import _number, _positive_int, _section
from wllm_amd.config.registry import ConfigError

MIXER_TYPES = ("attention", "latent_attention", "mamba2")


@dataclass(frozen=True)
class TokuvikAttention:
    heads: int
    kv_heads: int
    dim: int                    # query/key size of a head
    vdim: int                   # value size of a head
    scale: float
    chunk: Optional[int]        # mask.size: a position sees the earlier positions of its own chunk; None: all earlier
    kv_from: Optional[int]      # the layer whose keys and values this layer reads instead of making its own

    @classmethod
    def from_dict(cls, where: str, raw) -> "TokuvikAttention":
        raw = _section(where, raw, ("heads", "kv_heads", "dim", "vdim", "scale"), ("mask", "kv_from"))
        heads, kv_heads = _positive_int(f"{where}.heads", raw["heads"]), _positive_int(f"{where}.kv_heads", raw["kv_heads"])
        if heads % kv_heads:
            raise ConfigError(f"{where}: heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        chunk = None
        if raw.get("mask") is not None:
            chunk = _positive_int(f"{where}.mask.size", _section(f"{where}.mask", raw["mask"], ("size",))["size"])
        kv_from = raw.get("kv_from")
        if kv_from is not None and (isinstance(kv_from, bool) or not isinstance(kv_from, int) or kv_from < 0):
            raise ConfigError(f"{where}.kv_from must be the index of an earlier layer, got {kv_from!r}")
        return cls(heads, kv_heads, _positive_int(f"{where}.dim", raw["dim"]), _positive_int(f"{where}.vdim", raw["vdim"]),
                   _number(f"{where}.scale", raw["scale"]), chunk, kv_from)

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.chunk is not None:
            out["mask"] = {"size": self.chunk}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class TokuvikLatentAttention:
    heads: int
    dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float

    @classmethod
    def from_dict(cls, where: str, raw) -> "TokuvikLatentAttention":
        raw = _section(where, raw, ("heads", "dim", "vdim", "q_rank", "kv_rank", "scale"))
        return cls(*[_positive_int(f"{where}.{k}", raw[k]) for k in ("heads", "dim", "vdim", "q_rank", "kv_rank")],
                   _number(f"{where}.scale", raw["scale"]))

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "q_rank": self.q_rank, "kv_rank": self.kv_rank,
                "scale": self.scale}


@dataclass(frozen=True)
class TokuvikStateSpace:
    heads: int
    vdim: int                   # the size of a head
    state: int                  # N
    groups: int
    conv: int                   # taps of the convolution
    norm_groups: int

    @classmethod
    def from_dict(cls, where: str, raw) -> "TokuvikStateSpace":
        keys = ("heads", "vdim", "state", "groups", "conv", "norm_groups")
        raw = _section(where, raw, keys)
        out = cls(*[_positive_int(f"{where}.{k}", raw[k]) for k in keys])
        if out.heads % out.groups:
            raise ConfigError(f"{where}: heads ({out.heads}) must be a multiple of groups ({out.groups})")
        if (out.heads * out.vdim) % out.norm_groups:
            raise ConfigError(f"{where}: norm_groups ({out.norm_groups}) must divide heads * vdim ({out.heads * out.vdim})")
        return out

    def to_dict(self) -> dict:
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups, "conv": self.conv,
                "norm_groups": self.norm_groups}


_MIXERS = {"attention": TokuvikAttention, "latent_attention": TokuvikLatentAttention, "mamba2": TokuvikStateSpace}


@dataclass(frozen=True)
class TokuvikLayer:
    type: str
    mixer: object
    ff: Optional[int]           # width of the dense feed-forward, None for a layer without one


@dataclass(frozen=True)
class TokuvikConfig:
    vocab: int
    width: int
    norm_eps: float
    side_dim: Optional[int]     # token_side.dim; None: no token input
    layers: tuple
    raw: Optional[dict] = None

    @classmethod
    def from_dict(cls, raw: dict) -> "TokuvikConfig":
        raw = _section("config.json", raw, ("vocab", "width", "norm", "layers"), ("architecture", "architectures", "token_side"))
        if not isinstance(raw["layers"], list) or not raw["layers"]:
            raise ConfigError("config.json: layers must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            entry = _section(where, entry, ("type", "mixer"), ("mlp",))
            if entry["type"] not in _MIXERS:
                raise ConfigError(f"{where}.type {entry['type']!r}: this design's mixers are: {', '.join(MIXER_TYPES)}")
            mixer = _MIXERS[entry["type"]].from_dict(f"{where}.mixer", entry["mixer"])
            ff = None
            if entry.get("mlp") is not None:
                mlp = _section(f"{where}.mlp", entry["mlp"], ("kind", "ff"))
                if mlp["kind"] != "dense":
                    raise ConfigError(f"{where}.mlp.kind {mlp['kind']!r}: this design's feed-forwards are: dense")
                ff = _positive_int(f"{where}.mlp.ff", mlp["ff"])
            layers.append(TokuvikLayer(entry["type"], mixer, ff))
        for i, layer in enumerate(layers):
            src = getattr(layer.mixer, "kv_from", None)
            if src is None:
                continue
            where = f"layers[{i}].mixer.kv_from"
            if src >= i or layers[src].type != "attention" or layers[src].mixer.kv_from is not None:
                raise ConfigError(f"{where} = {src}: it must name an earlier attention layer that has keys and values of its own")
            theirs, mine = layers[src].mixer, layer.mixer
            if (theirs.kv_heads, theirs.dim, theirs.vdim) != (mine.kv_heads, mine.dim, mine.vdim):
                raise ConfigError(f"{where} = {src}: kv_heads, dim and vdim of the two layers must be equal")
        side_dim = None
        if raw.get("token_side") is not None:
            side_dim = _positive_int("token_side.dim", _section("token_side", raw["token_side"], ("dim",))["dim"])
        return cls(vocab=_positive_int("vocab", raw["vocab"]), width=_positive_int("width", raw["width"]),
                   norm_eps=_number("norm.eps", _section("norm", raw["norm"], ("eps",))["eps"], positive=False),
                   side_dim=side_dim, layers=tuple(layers), raw=raw)

    def to_dict(self) -> dict:
        """The config.json of this configuration."""
        if self.raw is not None:
            return dict(self.raw)
        out = {"architecture": "Tokuvik", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "layers": [{"type": layer.type, "mixer": layer.mixer.to_dict(),
                           "mlp": None if layer.ff is None else {"kind": "dense", "ff": layer.ff}} for layer in self.layers]}
        if self.side_dim is not None:
            out["token_side"] = {"dim": self.side_dim}
        return out
