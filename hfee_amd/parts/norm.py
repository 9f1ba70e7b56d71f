"""RMSNorm (/root/reference/internal/ggml/ops.go:124-134): y = x / sqrt(mean(x^2) + eps) * w,
the sum in float32, x the float32 residual stream, y in the engine's dtype (with the parameter
`weight_offset` the stored weight lies around zero and the norm multiplies by offset + w: the sum
is made once, in float32, when the weight is bound); "layernorm": y = (x - mean) / sqrt(variance + eps) * w
with the variance as the mean of the squared deviations and no bias; and "none" for a
place where a model has no norm (the rows as they are, in the engine's dtype)."""
from __future__ import annotations

import torch

from ..config.specs import NormSpec
from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import Norm, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, spec: NormSpec, name: str):
        self.width, self.eps, self.name = spec.width, spec.eps, name
        self.offset = float(dict(spec.params).get("weight_offset", 0.0))
        self.weight = None

    def tensor_specs(self):
        return [TensorSpec(self.name, (self.width,), role="vector",
                           init=("normal",) if self.offset else ("one_plus_normal",))]

    def bind(self, tensors):
        self.weight = tensors[self.name]
        if self.offset:
            self.weight = (self.weight.to(torch.float32) + self.offset).contiguous()

    def fused_form(self):
        return self.weight, self.eps

    def fused_form_f32(self):
        """(weight as float32, eps), for the launches that take their weights in float32 only."""
        if self.weight.dtype == torch.float32:
            return self.weight, self.eps
        if getattr(self, "_weight_f32", None) is None:
            self._weight_f32 = self.weight.to(torch.float32).contiguous()
        return self._weight_f32, self.eps

    def forward(self, ctx, out, x, rows=None):
        ops.rmsnorm(out, x, self.weight, self.eps, rows)


@register_norm("layernorm")
class LayerNorm(Norm):
    """The mean taken off, then the root mean square of what is left: not of the form that products
    fold into their first or last step (no `fused_form`), so it always runs as a launch of its own."""
    graph_safe = True

    def __init__(self, spec: NormSpec, name: str):
        self.width, self.eps, self.name = spec.width, spec.eps, name
        self.weight = None

    def tensor_specs(self):
        return [TensorSpec(self.name, (self.width,), role="vector", init=("one_plus_normal",))]

    def bind(self, tensors):
        self.weight = tensors[self.name].contiguous()

    def forward(self, ctx, out, x, rows=None):
        ops.layernorm(out, x, self.weight, self.eps, rows)


@register_norm("none")
class NoNorm(Norm):
    """Stands where an arrangement expects a norm and the model has none (no final norm before
    the head, a block whose sub-layers read the stream as it is): no tensor, nothing to fold into
    a product; the rows go to the part behind it rounded to the engine's dtype."""
    graph_safe = True

    def __init__(self, spec: NormSpec, name: str):
        self.width = spec.width

    def forward(self, ctx, out, x, rows=None):
        ops.cast_rows(out, x, rows)
