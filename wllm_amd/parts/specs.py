"""Descriptions of a model as data: which parts each layer is made of, with every
size and constant as a field, and the order in which layers run.

A specification names a part kind (the key of a registry in
`wllm_amd.parts.registry`) and carries that part's parameters and the names of
its tensors in the checkpoint.  No part, and nothing in here, knows which model
it belongs to: an architecture is a function from its configuration to a
`ModelPlan`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional


@dataclass(frozen=True)
class NormSpec:
    """kind "rms": y = x * rsqrt(mean(x^2) + eps) * (weight_offset + w); kind "layer": y = (x - mean(x)) *
    rsqrt(mean((x - mean(x))^2) + eps) * (weight_offset + w), a layer norm without a bias.  Computed in float32."""
    size: int
    eps: float
    weight: str                    # tensor name
    weight_offset: float = 0.0     # 1.0: the weight is stored as an offset from one
    kind: str = "rms"


@dataclass(frozen=True)
class PositionSpec:
    """How positions enter a mixer.  kind "rope": rotation of query and key by
    angles position * theta^(-2j/rotary_dim) / scaling_factor, pairing element j with
    j + rotary_dim/2 ("half") or element 2j with 2j + 1 ("interleaved"); elements of a head
    beyond rotary_dim pass unchanged.  kind "none": nothing."""
    kind: str = "rope"
    rotary_dim: int = 0
    theta: float = 10000.0
    pairing: str = "half"
    scaling_factor: float = 1.0     # linear scaling: every frequency is divided by it


@dataclass(frozen=True)
class MixerSpec:
    """Base of token-mixer specifications; `kind` selects the implementation."""
    kind: str = ""


@dataclass(frozen=True)
class AttentionSpec(MixerSpec):
    """Softmax attention of each query over the earlier keys of its request,
    read from the paged cache.  Query head h uses key/value head
    h // (num_heads // num_kv_heads).  `window` = W limits a query at position p
    to keys p-W+1..p; None is all keys.

    Options beyond the plain form, each off by default.  `softcap` c: the scaled score s becomes
    c * tanh(s / c) before the softmax.  `qk_norm_eps`: after the rotation every query and key
    head is divided by sqrt(mean of its squares + eps) (a norm without a weight).
    `values_are_keys`: there is no value projection; a key head as projected (with its bias,
    before rotation and norm) is also the value head.  `gate_weight`: the concatenated heads are
    multiplied by sigmoid(W_gate h) before the output projection.  `o_bias`: a bias of the output
    projection.  `weights_in_float32`: the softmax weights are not rounded to the values' type before
    they weigh the values (a design that wants its attention weights in 32-bit).
    `value_dim`: the size of a value head where it is not head_dim.  `chunk` c (instead of a window): a
    query sees the earlier keys of its own chunk of c positions counted from 0.  `release_chunk`: the
    chunk by which the cache gives pages back (the owner of a cache that layers with other masks read
    keeps what the widest of them needs; None with `chunk` set: keep everything).  `q_norm_weight` /
    `k_norm_weight` with `band_norm_eps`: an RMS norm with a weight over the whole query projection
    (all heads at once) and over the whole key projection, before the heads are split.
    `gate_per_head`: the gate's projection has one row a head, and its sigmoid multiplies the whole head.
    `owns_cache` False: the layer has no key and value projections (nor their norms); it reads the cache
    of the schedule entry its run names."""
    kind: str = "attention"
    hidden_size: int = 0
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    scale: float = 1.0
    window: Optional[int] = None
    position: PositionSpec = field(default_factory=PositionSpec)
    q_weight: str = ""
    k_weight: str = ""
    v_weight: str = ""
    o_weight: str = ""
    q_bias: Optional[str] = None
    k_bias: Optional[str] = None
    v_bias: Optional[str] = None
    softcap: Optional[float] = None
    qk_norm_eps: Optional[float] = None
    values_are_keys: bool = False
    gate_weight: Optional[str] = None
    o_bias: Optional[str] = None
    weights_in_float32: bool = False
    value_dim: Optional[int] = None
    chunk: Optional[int] = None
    release_chunk: Optional[int] = None
    q_norm_weight: Optional[str] = None
    k_norm_weight: Optional[str] = None
    band_norm_eps: Optional[float] = None
    gate_per_head: bool = False
    owns_cache: bool = True


@dataclass(frozen=True)
class LatentAttentionSpec(MixerSpec):
    """Causal softmax attention whose keys and values are expanded from one compressed vector a token
    (`kv_rank` numbers, the only thing cached), without positions: c_q = rms(W_dq h) * w_dqn, q = W_uq c_q;
    c = rms(W_dkv h) * w_dkvn; per head k = W_uk c, v = W_uv c; score = q.k * scale; with `sink_weight` the
    softmax's denominator holds exp(sink_h) once more; the concatenated heads are multiplied by
    sigmoid(W_g h) and projected by W_o."""
    kind: str = "latent_attention"
    hidden_size: int = 0
    num_heads: int = 0
    head_dim: int = 0           # query/key size of a head
    value_dim: int = 0
    q_rank: int = 0
    kv_rank: int = 0
    scale: float = 1.0
    norm_eps: float = 1e-6
    dq_weight: str = ""
    dq_norm_weight: str = ""
    uq_weight: str = ""
    dkv_weight: str = ""
    dkv_norm_weight: str = ""
    uk_weight: str = ""
    uv_weight: str = ""
    sink_weight: Optional[str] = None
    gate_weight: Optional[str] = None
    o_weight: str = ""


@dataclass(frozen=True)
class StateSpaceSpec(MixerSpec):
    """The selective state-space mixer of Mamba-2.  W_in h is [z: inner | x: inner | B: groups*N | C: groups*N |
    dt: heads] with inner = heads * head_dim; x, B and C pass a causal convolution per channel (`conv_taps`
    taps, a bias) and silu; dt = softplus(dt + dt_bias); per head S = exp(-exp(A_log) dt) S + dt B x^T,
    y = S^T C + D x; y * silu(z) is RMS-normed in `norm_groups` equal parts, times a weight, and projected.
    A request carries S (float32) and the convolution's last taps - 1 inputs."""
    kind: str = "state_space"
    hidden_size: int = 0
    num_heads: int = 0
    head_dim: int = 0
    state_size: int = 0
    groups: int = 1
    conv_taps: int = 4
    norm_groups: int = 1
    norm_eps: float = 1e-6
    in_weight: str = ""
    conv_weight: str = ""
    conv_bias: str = ""
    dt_bias: str = ""
    a_log: str = ""
    d_skip: str = ""
    norm_weight: str = ""
    o_weight: str = ""


@dataclass(frozen=True)
class TokenSideSpec:
    """A per-layer token input behind the feed-forward: e = table[token][offset : offset + dim];
    g = act(W_gate x) * e; y = W_proj g; x += rms(y) * w_norm.  The table [vocab, D] is shared by
    the layers, each reading its own band of columns."""
    hidden_size: int = 0
    vocab_size: int = 0
    dim: int = 0
    table: str = ""
    table_width: int = 0
    offset: int = 0
    activation: str = "gelu_tanh"
    gate_weight: str = ""
    proj_weight: str = ""
    norm: Optional[NormSpec] = None


@dataclass(frozen=True)
class FeedForwardSpec:
    kind: str = ""


@dataclass(frozen=True)
class GatedMLPSpec(FeedForwardSpec):
    """down(act(gate(x)) * up(x)) without biases; `activation` names the
    nonlinearity ("gelu_tanh")."""
    kind: str = "gated_mlp"
    hidden_size: int = 0
    intermediate_size: int = 0
    activation: str = "gelu_tanh"
    gate_weight: str = ""
    up_weight: str = ""
    down_weight: str = ""


@dataclass(frozen=True)
class BlockSpec:
    """One layer: a mixer and a feed-forward with their norms, and how they are
    arranged around the residual stream.  "pre_norm": x += mixer(norm(x));
    x += ffn(norm(x)).  "parallel": h = mixer_norm(x); x += mixer(h) + ffn(h): one norm, both
    sublayers read it (`feed_forward_norm` is None, and `feed_forward` may be None: then the
    layer is its mixer alone).  "sandwich": x += post(mixer(pre(x))); x += post(ffn(pre(x))) with the
    two norms behind the sublayers in `mixer_post_norm` and `feed_forward_post_norm` (a layer without a
    feed-forward has neither of its norms), then the layer's token input (`side`), if it has one."""
    mixer: MixerSpec
    feed_forward: Optional[FeedForwardSpec]
    mixer_norm: NormSpec
    feed_forward_norm: Optional[NormSpec]
    arrangement: str = "pre_norm"
    mixer_post_norm: Optional[NormSpec] = None
    feed_forward_post_norm: Optional[NormSpec] = None
    side: Optional[TokenSideSpec] = None


@dataclass(frozen=True)
class EmbeddingSpec:
    """x = table[id] * scale.  `scale_in_model_dtype`: the factor is rounded to
    the model's dtype before use, as a buffer cast with the model would be."""
    vocab_size: int
    hidden_size: int
    weight: str
    scale: float = 1.0
    scale_in_model_dtype: bool = False


@dataclass(frozen=True)
class HeadSpec:
    """logits = hidden @ W^T; W is the embedding table when `weight` is None.  `tied_checkpoint_name`:
    the name under which a checkpoint of tied weights may still store the head; such a tensor is
    accepted if it equals the table."""
    vocab_size: int
    hidden_size: int
    weight: Optional[str] = None
    tied_checkpoint_name: Optional[str] = None


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  `layer` indexes ModelPlan.layers (the same layer may
    be named by several entries: its weights are shared, each run has a cache
    of its own).  `reads_cache_of` = index of an earlier schedule entry whose
    cache this run reads instead of writing one.  `adds_embedding`: before this run the
    embedding output (the stream as it was before the first run) is added to the stream, as
    a model does that sends the stream through a span of its layers several times."""
    layer: int
    reads_cache_of: Optional[int] = None
    adds_embedding: bool = False


@dataclass(frozen=True)
class ModelPlan:
    embedding: EmbeddingSpec
    layers: tuple
    schedule: tuple
    final_norm: NormSpec
    head: HeadSpec
    max_positions: int
    # tensor names that may appear in a checkpoint and are ignored
    ignored_tensor_suffixes: tuple = ()

    def __post_init__(self):
        n = len(self.layers)
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < n:
                raise ValueError(f"schedule entry {i} names layer {e.layer}, the plan has {n}")
            if e.reads_cache_of is not None:
                j = e.reads_cache_of
                if not 0 <= j < i:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {j}, which is not an earlier entry")
                if self.schedule[j].reads_cache_of is not None:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {j}, which owns none")
