"""Norms.  "rms": y = x * rsqrt(mean(x^2) + eps) * (weight_offset + w) in float32,
cast after the multiply.  With weight_offset 1 this is the reference's
GemmaRMSNorm (src/wllm/models/gemma.py:41-51); with 0 the plain RMSNorm.  The
kernel also adds a pending contribution to the residual stream before it
normalises, which saves one pass over the stream per norm.
"layer": y = (x - mean) * rsqrt(variance + eps) * (weight_offset + w), a layer norm with a weight and
no bias; it runs on the general norm kernel, which can also put the pending contribution under a norm
of its own before it adds it (`delta_norm`: a norm behind a sublayer).  Any norm gives its `recipe()`
to stand behind a sublayer in that way."""
from __future__ import annotations

import torch

from wllm_amd.kernels import ops
from wllm_amd.parts.registry import register_norm
from wllm_amd.parts.specs import NormSpec
from wllm_amd.weights.checkpoint import ExpectedTensor


@register_norm("rms")
class RMSNorm:
    def __init__(self, spec: NormSpec):
        self.spec = spec
        self.weight = None

    def expected_tensors(self) -> dict:
        return {self.spec.weight: ExpectedTensor((self.spec.size,), role="vector", init="norm")}

    def load(self, fetch) -> None:
        self.weight = fetch.to_device(fetch.vector(self.spec.weight))

    def forward(self, x: torch.Tensor, out: torch.Tensor, delta=None, rows=None, delta_bias=None,
                delta_norm=None) -> torch.Tensor:
        """`delta_norm` (an `ops.NormRecipe`): the pending contribution is normalised by it before it is added."""
        if delta_norm is not None:
            if delta_bias is not None:
                raise NotImplementedError("a pending contribution with a bias under a norm of its own")
            ops.norm_add(x, delta=delta, delta_norm=delta_norm, out=out, out_norm=self.recipe(), rows=rows)
            return out
        ops.rms_norm(x, self.weight, self.spec.eps, self.spec.weight_offset, out, delta=delta, rows=rows,
                     delta_bias=delta_bias)
        return out

    takes_delta_norm = True

    def recipe(self) -> "ops.NormRecipe":
        return ops.NormRecipe("rms", self.weight, self.spec.eps, self.spec.weight_offset)

    def on_load(self, residual: torch.Tensor, sumsq: torch.Tensor, dtype: torch.dtype):
        """This norm of `residual` as a recipe for a kernel that applies it while it reads."""
        return ops.NormOnLoad(residual, sumsq, self.weight, self.spec.eps, self.spec.weight_offset, dtype)


@register_norm("layer")
class LayerNorm:
    """A layer norm with a weight and no bias, in float32, on the general norm kernel."""
    takes_delta_norm = True

    def __init__(self, spec: NormSpec):
        self.spec = spec
        self.weight = None

    def expected_tensors(self) -> dict:
        return {self.spec.weight: ExpectedTensor((self.spec.size,), role="vector", init="norm")}

    def load(self, fetch) -> None:
        self.weight = fetch.to_device(fetch.vector(self.spec.weight))

    def recipe(self) -> "ops.NormRecipe":
        return ops.NormRecipe("layer", self.weight, self.spec.eps, self.spec.weight_offset)

    def forward(self, x: torch.Tensor, out: torch.Tensor, delta=None, rows=None, delta_bias=None,
                delta_norm=None) -> torch.Tensor:
        if delta_bias is not None:
            raise NotImplementedError("a pending contribution with a bias before a layer norm")
        ops.norm_add(x, delta=delta, delta_norm=delta_norm, out=out, out_norm=self.recipe(), rows=rows)
        return out
