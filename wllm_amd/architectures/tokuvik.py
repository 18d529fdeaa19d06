"""Tokuvik as a plan of parts.

A decoder of "sandwich" layers: x += norm1b(mixer(norm1(x))), then (if the layer has a feed-forward)
x += norm2b(ff(norm2(x))), all four layer norms with a weight and no bias, then a per-layer token
input x += rms(W_proj (gelu_tanh(W_gate x) * e)) * w with e the layer's band of the token's row of a
shared table.  The file picks each layer's mixer: attention inside chunks of the sequence, with an RMS
norm over the whole query and key projections, value heads of a size of their own, no rotation, one
sigmoid gate a head, and optionally the keys and values of an earlier layer (`kv_from`); latent
attention over one cached compressed vector a token, with a sink in the softmax and an elementwise
gate; or the state-space recurrence of Mamba-2.  Feed-forwards are gated with silu.  The head is the
embedding table after the model's norm; the embedding has no factor.  Tensor names: `embed`,
`side.embed`, `final.norm`, and per layer i `l<i>.norm1`, `.norm1b`, `.norm2`, `.norm2b`,
`l<i>.mix.*`, `l<i>.mlp.{gate,up,down}`, `l<i>.side.{gate,proj,norm}`.
"""
from __future__ import annotations

from wllm_amd.architectures.tokuvik_config import TokuvikConfig
from wllm_amd.config.registry import register_architecture
from wllm_amd.parts.specs import (
    AttentionSpec,
    BlockSpec,
    EmbeddingSpec,
    GatedMLPSpec,
    HeadSpec,
    LatentAttentionSpec,
    ModelPlan,
    NormSpec,
    PositionSpec,
    ScheduleEntry,
    StateSpaceSpec,
    TokenSideSpec,
)

# the design names no longest sequence: a request is as long as the cache lets it be
NO_POSITION_LIMIT = 1 << 30


def tokuvik_plan(cfg: TokuvikConfig) -> ModelPlan:
    def norm(name: str, kind: str = "layer") -> NormSpec:
        return NormSpec(size=cfg.width, eps=cfg.norm_eps, weight=name, kind=kind)

    # the masks of all layers that read one cache: its pages go back by the chunk only if they all agree
    readers = {}
    for i, layer in enumerate(cfg.layers):
        if layer.type == "attention":
            owner = i if layer.mixer.kv_from is None else layer.mixer.kv_from
            readers.setdefault(owner, set()).add(layer.mixer.chunk)
    layers = []
    for i, layer in enumerate(cfg.layers):
        m, p = layer.mixer, f"l{i}.mix."
        if layer.type == "attention":
            owns = m.kv_from is None
            masks = readers[i if owns else m.kv_from]
            mixer = AttentionSpec(
                hidden_size=cfg.width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim,
                scale=m.scale, chunk=m.chunk, release_chunk=m.chunk if len(masks) == 1 else None,
                position=PositionSpec(kind="none"), q_weight=p + "q", k_weight=p + "k" if owns else "",
                v_weight=p + "v" if owns else "", o_weight=p + "o", gate_weight=p + "g", gate_per_head=True,
                q_norm_weight=p + "q.norm", k_norm_weight=p + "k.norm" if owns else None, band_norm_eps=cfg.norm_eps,
                owns_cache=owns, weights_in_float32=True)
        elif layer.type == "latent_attention":
            mixer = LatentAttentionSpec(
                hidden_size=cfg.width, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim, q_rank=m.q_rank,
                kv_rank=m.kv_rank, scale=m.scale, norm_eps=cfg.norm_eps, dq_weight=p + "dq", dq_norm_weight=p + "dq.norm",
                uq_weight=p + "uq", dkv_weight=p + "dkv", dkv_norm_weight=p + "dkv.norm", uk_weight=p + "uk",
                uv_weight=p + "uv", sink_weight=p + "sink", gate_weight=p + "g", o_weight=p + "o")
        else:
            mixer = StateSpaceSpec(
                hidden_size=cfg.width, num_heads=m.heads, head_dim=m.vdim, state_size=m.state, groups=m.groups,
                conv_taps=m.conv, norm_groups=m.norm_groups, norm_eps=cfg.norm_eps, in_weight=p + "in",
                conv_weight=p + "conv", conv_bias=p + "conv.b", dt_bias=p + "dt_bias", a_log=p + "A_log", d_skip=p + "D",
                norm_weight=p + "norm", o_weight=p + "o")
        q = f"l{i}."
        side = None
        if cfg.side_dim is not None:
            side = TokenSideSpec(
                hidden_size=cfg.width, vocab_size=cfg.vocab, dim=cfg.side_dim, table="side.embed",
                table_width=cfg.side_dim * len(cfg.layers), offset=i * cfg.side_dim, activation="gelu_tanh",
                gate_weight=q + "side.gate", proj_weight=q + "side.proj", norm=norm(q + "side.norm", kind="rms"))
        has_ff = layer.ff is not None
        layers.append(BlockSpec(
            arrangement="sandwich", mixer=mixer,
            feed_forward=GatedMLPSpec(hidden_size=cfg.width, intermediate_size=layer.ff, activation="silu",
                                      gate_weight=q + "mlp.gate", up_weight=q + "mlp.up",
                                      down_weight=q + "mlp.down") if has_ff else None,
            mixer_norm=norm(q + "norm1"), mixer_post_norm=norm(q + "norm1b"),
            feed_forward_norm=norm(q + "norm2") if has_ff else None,
            feed_forward_post_norm=norm(q + "norm2b") if has_ff else None, side=side))
    # a layer that reads another layer's keys and values: its run reads the cache of that layer's run
    schedule = tuple(ScheduleEntry(layer=i, reads_cache_of=getattr(layer.mixer, "kv_from", None))
                     for i, layer in enumerate(cfg.layers))
    return ModelPlan(
        embedding=EmbeddingSpec(vocab_size=cfg.vocab, hidden_size=cfg.width, weight="embed"),
        layers=tuple(layers), schedule=schedule, final_norm=norm("final.norm"),
        head=HeadSpec(vocab_size=cfg.vocab, hidden_size=cfg.width), max_positions=NO_POSITION_LIMIT,
        # a layer without a feed-forward needs neither of its norms; a file may still carry them
        ignored_tensor_suffixes=tuple(f"l{i}.{n}" for i, layer in enumerate(cfg.layers) if layer.ff is None
                                      for n in ("norm2", "norm2b")))


register_architecture("Tokuvik", TokuvikConfig.from_dict, tokuvik_plan)
