"""Tasosun as a plan of parts.

A decoder of parallel blocks: h = norm(x), x += attention(h) + feed_forward(h), with one
(1 + w) RMS norm a layer.  The attention has biases on its query, key and output projections,
no value projection (a key head as projected is the value head), a rotation of interleaved
pairs over the first elements of a head with linearly scaled positions, a unit norm of every
query and key head after the rotation, scores bent under a cap, a sliding window, and a
sigmoid gate from a projection of its own on the concatenated heads.  The feed-forward is
gated with silu.  A span of the layers may run several times with the same weights, each run
with a cache of its own, and the embedding output is added to the stream before every pass of
the span but the first.  The embedding table is multiplied by a constant of the file; the head
is a matrix of its own after the model's (1 + w) norm.  Tensor names: `embed`, `head`,
`final.norm`, and per layer i `l<i>.norm1`, `l<i>.mix.{q,k,g,o}` with biases `.b` on q, k, o,
`l<i>.mlp.{gate,up,down}`.
"""
from __future__ import annotations

from wllm_amd.architectures.tasosun_config import TasosunConfig
from wllm_amd.config.registry import register_architecture
from wllm_amd.parts.specs import (
    AttentionSpec,
    BlockSpec,
    EmbeddingSpec,
    GatedMLPSpec,
    HeadSpec,
    ModelPlan,
    NormSpec,
    PositionSpec,
    ScheduleEntry,
)

# the design names no longest sequence: a request is as long as the cache lets it be
NO_POSITION_LIMIT = 1 << 30


def tasosun_plan(cfg: TasosunConfig) -> ModelPlan:
    def norm(name: str) -> NormSpec:
        return NormSpec(size=cfg.width, eps=cfg.norm_eps, weight=name, weight_offset=1.0)

    layers = []
    for i, layer in enumerate(cfg.layers):
        a, p = layer.attention, f"l{i}."
        rot = a.rotation
        position = PositionSpec(kind="none") if rot is None else PositionSpec(
            kind="rope", rotary_dim=rot.dims, theta=rot.base, pairing="interleaved", scaling_factor=rot.scaling_factor)
        layers.append(BlockSpec(
            arrangement="parallel",
            mixer=AttentionSpec(
                hidden_size=cfg.width, num_heads=a.heads, num_kv_heads=a.kv_heads, head_dim=a.dim, scale=a.scale,
                window=a.window, position=position,
                q_weight=p + "mix.q", k_weight=p + "mix.k", o_weight=p + "mix.o", gate_weight=p + "mix.g",
                q_bias=p + "mix.q.b", k_bias=p + "mix.k.b", o_bias=p + "mix.o.b",
                softcap=a.softcap, qk_norm_eps=cfg.norm_eps, values_are_keys=True, weights_in_float32=True),
            feed_forward=None if layer.ff is None else GatedMLPSpec(
                hidden_size=cfg.width, intermediate_size=layer.ff, activation="silu",
                gate_weight=p + "mlp.gate", up_weight=p + "mlp.up", down_weight=p + "mlp.down"),
            mixer_norm=norm(p + "norm1"),
            feed_forward_norm=None,
        ))
    return ModelPlan(
        embedding=EmbeddingSpec(vocab_size=cfg.vocab, hidden_size=cfg.width, weight="embed", scale=cfg.embedding_scale),
        layers=tuple(layers),
        schedule=tuple(ScheduleEntry(layer=i, adds_embedding=again) for i, again in cfg.runs()),
        final_norm=norm("final.norm"),
        head=HeadSpec(vocab_size=cfg.vocab, hidden_size=cfg.width, weight="head"),
        max_positions=NO_POSITION_LIMIT,
    )


register_architecture("Tasosun", TasosunConfig.from_dict, tasosun_plan)
