"""The attention mixer: q/k/v projection as one product, rotation and cache write
as one kernel, attention over the request's pages, output projection.

It follows the reference's attention (src/wllm/models/llama.py:82-115 for the
formulas, :143-247 for the cached forms) with one code path for all of them: a
flat batch of segments, each the next tokens of some request, a decoded token
being a segment of one.  Head h of the q/k/v rows is columns h*head_dim ..
(h+1)*head_dim of the projection (llama.py:103-105).  The three projection
matrices are stacked at load so that one product makes the [n, (nh+2nkv)*d]
row the kernels read.

The specification's options widen the row and the steps between projection and attention
(`ops.head_prepare` then stands where `ops.rope_and_cache_write` stands for the plain form): a
rotation of interleaved pairs or of a part of the head, a unit norm of queries and keys, values
that are the keys as projected (the row has no value heads), a cap on the scores, and an output
gate whose projection is stacked behind the heads (row: queries, keys, [values], [gate]) and
multiplied into the attention's result before the output projection, which may have a bias.
"""
from __future__ import annotations

from typing import Optional

import torch

from wllm_amd.cache.manager import CacheNeed
from wllm_amd.kernels import ops
from wllm_amd.parts.common import Product, load_matrix, project
from wllm_amd.parts.registry import build_position, register_mixer
from wllm_amd.parts.specs import AttentionSpec
from wllm_amd.weights.checkpoint import ExpectedTensor


@register_mixer("attention")
class PagedAttention:
    graph_capturable = True     # everything it does reads the step's device arrays

    def __init__(self, spec: AttentionSpec):
        if spec.num_heads % spec.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if spec.window is not None and spec.window <= 0:
            raise ValueError(f"window must be positive or None, got {spec.window}")
        plain = not (spec.softcap or spec.qk_norm_eps is not None or spec.values_are_keys or spec.gate_weight
                     or spec.position.pairing == "interleaved")
        if (plain and spec.head_dim % ops.HEAD_DIM_STEP) or not 0 < spec.head_dim <= ops.MAX_HEAD_DIM:
            raise ValueError(f"head_dim {spec.head_dim}: the attention kernels take multiples of "
                             f"{ops.HEAD_DIM_STEP} up to {ops.MAX_HEAD_DIM}")
        if spec.values_are_keys and (spec.v_weight or spec.v_bias):
            raise ValueError("values_are_keys: there is no value projection to name")
        if spec.softcap is not None and not spec.softcap > 0:
            raise ValueError(f"softcap must be positive or None, got {spec.softcap}")
        if spec.qk_norm_eps is not None and spec.qk_norm_eps < 0:
            raise ValueError(f"qk_norm_eps must not be negative, got {spec.qk_norm_eps}")
        self.spec = spec
        self.position = build_position(spec.position)
        self.w_qkv = None
        self.b_qkv = None
        self.w_o = None
        self.b_o = None
        # the plain form runs the kernels that were written for it; anything else the general ones
        self.plain = plain
        # The kernels take heads of a multiple of four elements.  A head of another size is padded at load with
        # rows of zeros in its projections (and columns of zeros in the output projection): the padding is zero
        # in queries, keys and values, adds nothing to a score or a result, and the unit norm divides by the
        # true size.  Only the general path does this.
        self.dim = spec.head_dim if plain else -(-spec.head_dim // ops.HEAD_DIM_STEP) * ops.HEAD_DIM_STEP

    @property
    def qkv_width(self) -> int:
        """Columns of the projected row: queries, keys, values (unless they are the keys), gate."""
        s = self.spec
        heads = s.num_heads + (1 if s.values_are_keys else 2) * s.num_kv_heads + (s.num_heads if s.gate_weight else 0)
        return heads * self.dim

    @property
    def gate_offset(self) -> int:
        s = self.spec
        return (s.num_heads + (1 if s.values_are_keys else 2) * s.num_kv_heads) * self.dim

    def expected_tensors(self) -> dict:
        s = self.spec
        q, kv = s.num_heads * s.head_dim, s.num_kv_heads * s.head_dim
        out = {
            s.q_weight: ExpectedTensor((q, s.hidden_size)),
            s.k_weight: ExpectedTensor((kv, s.hidden_size)),
            s.o_weight: ExpectedTensor((s.hidden_size, q)),
        }
        if not s.values_are_keys:
            out[s.v_weight] = ExpectedTensor((kv, s.hidden_size))
        if s.gate_weight:
            out[s.gate_weight] = ExpectedTensor((q, s.hidden_size))
        for name, width in ((s.q_bias, q), (s.k_bias, kv), (s.v_bias, kv), (s.o_bias, s.hidden_size)):
            if name is not None:
                out[name] = ExpectedTensor((width,), role="vector")
        if hasattr(self.position, "expected_tensors"):      # a position encoding with tensors of its own
            out.update(self.position.expected_tensors())
        return out

    def load(self, fetch) -> None:
        s = self.spec
        names = [s.q_weight, s.k_weight] + ([] if s.values_are_keys else [s.v_weight]) + ([s.gate_weight] if s.gate_weight else [])
        pad = self.dim - s.head_dim

        def heads_padded(t: torch.Tensor, axis: int) -> torch.Tensor:
            """`t` with every head of `axis` (heads * head_dim long) followed by `pad` zeros."""
            if not pad:
                return t
            shape = list(t.shape)
            heads = shape[axis] // s.head_dim
            t = t.unflatten(axis, (heads, s.head_dim))
            zeros = torch.zeros(shape[:axis] + [heads, pad] + shape[axis + 1:], dtype=t.dtype, device=t.device)
            return torch.cat([t, zeros], dim=axis + 1).flatten(axis, axis + 1)

        w = torch.cat([heads_padded(fetch.matrix(name), 0) for name in names], dim=0)
        self.w_qkv, self.t_qkv = load_matrix(fetch, w)        # the matrix and its tile-major copy
        self.w_o, self.t_o = load_matrix(fetch, heads_padded(fetch.matrix(s.o_weight), 1))
        if s.o_bias is not None:
            self.b_o = fetch.to_device(fetch.vector(s.o_bias))
        if s.q_bias is not None or s.k_bias is not None or s.v_bias is not None:
            q, kv = s.num_heads * s.head_dim, s.num_kv_heads * s.head_dim
            biases = [(s.q_bias, q), (s.k_bias, kv)] + ([] if s.values_are_keys else [(s.v_bias, kv)])
            # (the gate's projection, behind the heads in the row, has none: the bias is shorter than the row)
            found = [fetch.vector(name) if name is not None else None for name, _ in biases]
            where = next(v.device for v in found if v is not None)      # a fetcher may make its tensors on the device
            parts = [heads_padded(v if v is not None else torch.zeros(width, device=where), 0)
                     for v, (_, width) in zip(found, biases)]
            self.b_qkv = fetch.to_device(torch.cat(parts))
        if hasattr(self.position, "load"):
            self.position.load(fetch)
        self.position.prepare(fetch.device)

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed(self.spec.num_kv_heads, self.dim, self.spec.window)

    def state_shape(self):
        return None

    def flops(self, tokens: int, keys: float) -> float:
        """Floating-point operations of `tokens` tokens whose queries see `keys` keys in all (what a
        measurement divides by its time)."""
        s = self.spec
        return 2.0 * tokens * s.hidden_size * (self.qkv_width + s.num_heads * s.head_dim) + 4.0 * s.num_heads * s.head_dim * keys

    def _work_items(self, ctx, page_size: int):
        """The step's work items for attention of this shape: made once a step, shared by all
        layers of the shape; of fixed shape and rewritten in place in a captured graph."""
        s = self.spec
        # (the plan depends on these alone: layers that differ in their rows' width or cap share it)
        shape = dict(num_heads=s.num_heads, num_kv_heads=s.num_kv_heads, head_dim=self.dim, page_size=page_size,
                     window=s.window or 0)

        def build(c):
            if c.captured:
                return ops.static_attention_plan(c.num_segments, max_context=c.capture_max_context,
                                                 max_total_keys=c.capture_max_tokens, dtype=c.dtype, device=c.device, **shape)
            return ops.plan_paged_attention(c.host_q_len, c.host_ctx_len, dtype=c.dtype, device=c.device, **shape)

        def refresh(plan, c):
            plan.update(c.host_q_len, c.host_ctx_len)

        return ctx.plan(("attention",) + tuple(shape.values()), build, refresh)

    def forward(self, ctx, entry: int, h: torch.Tensor, product_input: Optional[torch.Tensor] = None):
        """`product_input`: a band of columns [n, heads * head_dim] of a wider buffer into which the
        input of the output projection is to be written (a block that makes one product of several
        parts' last products asks for it); the returned `Product` then names that band."""
        s = self.spec
        n = h.shape[0]
        qkv = ctx.buffer("qkv", (n, self.qkv_width), h.dtype)
        pages = ctx.pages(entry)
        slots, storage = (pages.slots, pages.storage) if pages.writes else (None, None)
        # What the position encoding asks for: a table of frequencies that the rotation kernels turn
        # queries and keys by (`inv_freq`, or None), and/or a step of its own on the projected rows
        # before they are cached and read (`apply`).
        inv_freq = self.position.inv_freq
        apply = getattr(self.position, "apply", None)
        rotary_dim = 2 * inv_freq.shape[0] if inv_freq is not None else s.head_dim
        if not self.plain:
            if apply is not None:
                raise NotImplementedError("a position encoding with a step of its own beside the attention's options")
            projected = project(ctx, "qkv", h, self.w_qkv, qkv, tiles=self.t_qkv)
            ops.head_prepare(
                qkv, self.b_qkv, ctx.positions, inv_freq, slots, storage, num_heads=s.num_heads,
                num_kv_heads=s.num_kv_heads, head_dim=self.dim, page_size=pages.page_size,
                interleaved=getattr(self.position, "interleaved", False), norm_eps=s.qk_norm_eps,
                values_are_keys=s.values_are_keys, parts=projected if projected.dim() == 3 else None,
                norm_dim=s.head_dim)
        elif apply is not None:
            ops.linear(h, self.w_qkv, qkv, self.t_qkv)
            if self.b_qkv is not None:
                qkv += self.b_qkv.to(qkv.dtype)
            apply(ctx, qkv, num_heads=s.num_heads, num_kv_heads=s.num_kv_heads, head_dim=s.head_dim)
            ops.rope_and_cache_write(
                qkv, None, ctx.positions, inv_freq, slots, storage,
                num_heads=s.num_heads, num_kv_heads=s.num_kv_heads, head_dim=s.head_dim, page_size=pages.page_size)
        elif ops.qkv_rope_takes(n, h.dtype, h.shape[1], s.head_dim, rotary_dim):
            # a decode step: projection, rotation and cache write in one kernel
            ops.qkv_rope(h, self.w_qkv, qkv, self.b_qkv, ctx.positions, inv_freq, slots, storage,
                         num_heads=s.num_heads, num_kv_heads=s.num_kv_heads, head_dim=s.head_dim,
                         page_size=pages.page_size, tiles=self.t_qkv)
        else:
            # where the product kernel splits its sums, the rotation kernel adds them as it reads
            projected = project(ctx, "qkv", h, self.w_qkv, qkv, tiles=self.t_qkv)
            parts = projected if projected.dim() == 3 else None
            ops.rope_and_cache_write(
                qkv, self.b_qkv, ctx.positions, inv_freq, slots, storage,
                num_heads=s.num_heads, num_kv_heads=s.num_kv_heads, head_dim=s.head_dim, page_size=pages.page_size,
                parts=parts)
        attn = ctx.buffer("attn", (n, s.num_heads * self.dim), h.dtype)
        ops.paged_attention(
            qkv, pages.storage, pages.block_tables, ctx.token_segment, ctx.seg_q_start, ctx.seg_q_len,
            ctx.seg_ctx_len, attn, num_heads=s.num_heads, num_kv_heads=s.num_kv_heads, head_dim=self.dim,
            page_size=pages.page_size, scale=s.scale, window=s.window or 0,
            max_q_len=ctx.max_q_len, max_ctx_len=ctx.max_ctx_len,
            plan=self._work_items(ctx, pages.page_size), softcap=s.softcap or 0.0, exact_weights=s.weights_in_float32)
        if s.gate_weight:
            # the gate's columns lie behind the heads in the projected row
            gate = qkv[:, self.gate_offset:self.gate_offset + s.num_heads * self.dim]
            target = product_input if product_input is not None else attn
            ops.sigmoid_gate(attn, gate, target)
            attn = target
        elif product_input is not None:
            ops.copy_columns(attn, product_input)
            attn = product_input
        # the stream adds the output projection: at once, or through the next norm, partial sums and all
        return Product("mixer_out", attn, self.w_o, self.t_o, bias=self.b_o)
