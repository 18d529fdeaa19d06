"""The selective state-space mixer of Mamba-2 on the step's flat batch.

    [z | x | B | C | dt] = W_in h                       inner = heads * head_dim; B, C: groups * N each
    [x | B | C] = silu(conv(x | B | C))                 a causal convolution per channel, `conv_taps` taps
    dt = softplus(dt + dt_bias)
    S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T    per head, S [N, head_dim], float32
    y_t = S_t^T C_t + D x_t
    out = W_o (rms_in_groups(y * silu(z)) * w)

A request carries S and the convolution's last taps - 1 inputs from step to step in one float32 state
row of the cache manager ([heads * N * head_dim] then [(taps - 1) * channels]; zeroed at admission, which
is both the zero state and the zeros before a sequence's start).  The kernels walk every segment's
tokens in order from that row and leave it for the next step, so a prompt may be cut anywhere, and a
decoded token is a segment of one.  Everything the kernels read of the step lies in device arrays, so a
decode step can be captured in a graph.
"""
from __future__ import annotations

from typing import Optional

import torch

from wllm_amd.kernels import ops
from wllm_amd.parts.common import Product, load_matrix
from wllm_amd.parts.registry import register_mixer
from wllm_amd.parts.specs import StateSpaceSpec
from wllm_amd.weights.checkpoint import ExpectedTensor


@register_mixer("state_space")
class StateSpaceMixer:
    graph_capturable = True

    def __init__(self, spec: StateSpaceSpec):
        for name in ("hidden_size", "num_heads", "head_dim", "state_size", "groups", "conv_taps", "norm_groups"):
            if getattr(spec, name) <= 0:
                raise ValueError(f"{name} must be positive, got {getattr(spec, name)}")
        if spec.num_heads % spec.groups:
            raise ValueError(f"num_heads ({spec.num_heads}) must be a multiple of groups ({spec.groups})")
        if (spec.num_heads * spec.head_dim) % spec.norm_groups:
            raise ValueError(f"norm_groups ({spec.norm_groups}) must divide heads * head_dim")
        if spec.state_size > 256:
            raise ValueError(f"state_size {spec.state_size}: the recurrence's kernel keeps at most 256 rows a head")
        self.spec = spec
        self.inner = spec.num_heads * spec.head_dim
        self.channels = self.inner + 2 * spec.groups * spec.state_size        # what the convolution runs over
        self.in_width = self.inner + self.channels + spec.num_heads
        self.recurrent_size = spec.num_heads * spec.state_size * spec.head_dim
        self.w_in = self.t_in = self.w_o = self.t_o = None
        self.conv_w = self.conv_b = self.dt_bias = self.a_log = self.d_skip = self.norm_w = None

    def expected_tensors(self) -> dict:
        s = self.spec
        vector = dict(role="vector", init="norm")
        return {
            s.in_weight: ExpectedTensor((self.in_width, s.hidden_size)),
            s.conv_weight: ExpectedTensor((self.channels, s.conv_taps), role="vector"),
            s.conv_bias: ExpectedTensor((self.channels,), **vector),
            s.dt_bias: ExpectedTensor((s.num_heads,), **vector),
            s.a_log: ExpectedTensor((s.num_heads,), **vector),
            s.d_skip: ExpectedTensor((s.num_heads,), **vector),
            s.norm_weight: ExpectedTensor((self.inner,), **vector),
            s.o_weight: ExpectedTensor((s.hidden_size, self.inner)),
        }

    def load(self, fetch) -> None:
        s = self.spec
        self.w_in, self.t_in = load_matrix(fetch, fetch.matrix(s.in_weight))
        self.w_o, self.t_o = load_matrix(fetch, fetch.matrix(s.o_weight))
        # everything that enters the recurrence, and the convolution's taps, is kept in float32
        self.conv_w = fetch.to_device(fetch.vector(s.conv_weight))
        self.conv_b = fetch.to_device(fetch.vector(s.conv_bias))
        self.dt_bias = fetch.to_device(fetch.vector(s.dt_bias))
        self.a_log = fetch.to_device(fetch.vector(s.a_log))
        self.d_skip = fetch.to_device(fetch.vector(s.d_skip))
        self.norm_w = fetch.to_device(fetch.vector(s.norm_weight))

    def cache_need(self):
        return None

    def state_shape(self):
        return (self.recurrent_size + (self.spec.conv_taps - 1) * self.channels,)

    def flops(self, tokens: int, keys: float = 0.0) -> float:
        s = self.spec
        return 2.0 * tokens * (s.hidden_size * (self.in_width + self.inner) + self.channels * s.conv_taps
                               + 3 * s.num_heads * s.state_size * s.head_dim)

    def forward(self, ctx, entry: int, h: torch.Tensor, product_input: Optional[torch.Tensor] = None):
        s = self.spec
        n = h.shape[0]
        row = ctx.buffer("ssm_in", (n, self.in_width), h.dtype)
        ops.linear(h, self.w_in, row, self.t_in)
        state = ctx.state(entry)
        xbc = ctx.buffer("ssm_xbc", (n, self.channels), h.dtype)
        ops.causal_conv(row[:, self.inner:self.inner + self.channels], self.conv_w, self.conv_b, state, self.recurrent_size,
                        ctx.token_segment, ctx.seg_q_start, ctx.seg_q_len, ctx.state_slots, xbc)
        y = ctx.buffer("ssm_y", (n, self.inner), torch.float32)
        ops.ssm_scan(xbc, row[:, self.inner + self.channels:], self.dt_bias, self.a_log, self.d_skip, state,
                     ctx.seg_q_start, ctx.seg_q_len, ctx.state_slots, y, heads=s.num_heads, groups=s.groups,
                     state_size=s.state_size, head_dim=s.head_dim,
                     steps=ctx.buffer("ssm_steps", (2, n, s.num_heads), torch.float32))
        out = ctx.buffer("ssm_out", (n, self.inner), h.dtype)
        ops.gated_group_norm(y, row[:, :self.inner], self.norm_w, out, s.norm_groups, s.norm_eps)
        if product_input is not None:
            ops.copy_columns(out, product_input)
            out = product_input
        return Product("mixer_out", out, self.w_o, self.t_o)
