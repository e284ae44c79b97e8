"""RMSNorm (/root/reference/internal/ggml/ops.go:124-134): y = x / sqrt(mean(x^2) + eps) * w,
the sum in float32, x the float32 residual stream, y in the engine's dtype; and "none" for a
place where a model has no norm (the rows as they are, in the engine's dtype)."""
from __future__ import annotations

from ..config.specs import NormSpec
from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import Norm, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, spec: NormSpec, name: str):
        self.width, self.eps, self.name = spec.width, spec.eps, name
        self.weight = None

    def tensor_specs(self):
        return [TensorSpec(self.name, (self.width,), role="vector", init=("one_plus_normal",))]

    def bind(self, tensors):
        self.weight = tensors[self.name]

    def fused_form(self):
        return self.weight, self.eps

    def forward(self, ctx, out, x, rows=None):
        ops.rmsnorm(out, x, self.weight, self.eps, rows)


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
