"""A per-layer token input: every layer looks its tokens up in a band of columns of one shared table
and lets a small projection of the stream gate the entry:

    e = table[token][offset : offset + dim];  g = act(W_gate x) * e;  y = W_proj g;  x += rms(y) * w

x is the residual stream itself (no norm before the gate's projection); the norm behind the part is an
RMS norm with a plain weight, whatever the model's other norms are.  The table lies on the device once,
however many layers read it.
"""
from __future__ import annotations

import torch

from wllm_amd.kernels import ops
from wllm_amd.parts.common import Product, load_matrix
from wllm_amd.parts.registry import build_norm
from wllm_amd.parts.specs import TokenSideSpec
from wllm_amd.weights.checkpoint import ExpectedTensor


class TokenSide:
    lookup_tables = ("table",)      # read a row a token, not whole: no part of the weights a step streams

    def __init__(self, spec: TokenSideSpec):
        if spec.activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation {spec.activation!r} is not implemented; known: {ops.ACTIVATIONS}")
        if not 0 <= spec.offset <= spec.table_width - spec.dim:
            raise ValueError(f"columns {spec.offset}..{spec.offset + spec.dim} do not lie in a table of {spec.table_width}")
        self.spec = spec
        self.norm = build_norm(spec.norm)
        self.table = None
        self.w_gate = self.t_gate = None
        self.w_proj = self.t_proj = None

    def expected_tensors(self) -> dict:
        s = self.spec
        out = {
            s.table: ExpectedTensor((s.vocab_size, s.table_width)),
            s.gate_weight: ExpectedTensor((s.dim, s.hidden_size)),
            s.proj_weight: ExpectedTensor((s.hidden_size, s.dim)),
        }
        out.update(self.norm.expected_tensors())
        return out

    def load(self, fetch) -> None:
        s = self.spec
        # the table is one tensor for all layers: whoever loads first puts it on the device
        shared = fetch.__dict__.setdefault("_shared_tables", {})
        if s.table not in shared:
            shared[s.table] = fetch.to_device(fetch.matrix(s.table))
        self.table = shared[s.table]
        self.w_gate, self.t_gate = load_matrix(fetch, fetch.matrix(s.gate_weight))
        self.w_proj, self.t_proj = load_matrix(fetch, fetch.matrix(s.proj_weight))
        self.norm.load(fetch)

    def forward(self, ctx, x: torch.Tensor) -> Product:
        """x: the stream in the activation type [n, hidden].  Returns the part's last product; the block
        puts it under `self.norm` as it adds it."""
        s = self.spec
        n = x.shape[0]
        gate = ctx.buffer("side_gate", (n, s.dim), ctx.dtype)
        ops.linear(x, self.w_gate, gate, self.t_gate)
        g = ctx.buffer("side_in", (n, s.dim), ctx.dtype)
        ops.gated_lookup(gate, ctx.token_ids, self.table, s.offset, g, s.activation)
        return Product("side_out", g, self.w_proj, self.t_proj)
