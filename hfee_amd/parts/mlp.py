"""The gated feed-forward (/root/reference/internal/llm/forward.go:110-114,
/root/reference/internal/ggml/ops.go:159-165): down(silu(gate(h)) * up(h)), added to
the residual stream.  gate and up run as one product over the concatenated weight
[gate rows; up rows]."""
from __future__ import annotations

import torch

from ..config.specs import FeedForwardSpec
from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import FeedForward, register_feed_forward


@register_feed_forward("gated_mlp")
class GatedMLP(FeedForward):
    graph_safe = True

    def __init__(self, spec: FeedForwardSpec, prefix: str, dtype: torch.dtype):
        self.hidden = spec.get("hidden")
        self.intermediate = spec.get("intermediate")
        act = spec.get("activation", "silu")
        if act != "silu":
            raise ValueError(f"the gated feed-forward is built for 'silu', got {act!r}")
        self.prefix, self.dtype = prefix, dtype
        self.w_gate_up = self.w_down = None

    def tensor_specs(self):
        p = self.prefix
        return [TensorSpec(p + "gate_proj.weight", (self.intermediate, self.hidden)),
                TensorSpec(p + "up_proj.weight", (self.intermediate, self.hidden)),
                TensorSpec(p + "down_proj.weight", (self.hidden, self.intermediate))]

    def bind(self, tensors):
        p = self.prefix
        self.w_gate_up = torch.cat([tensors.pop(p + "gate_proj.weight"), tensors.pop(p + "up_proj.weight")],
                                   dim=0).contiguous()
        self.w_down = tensors.pop(p + "down_proj.weight").contiguous()

    def forward_add(self, ctx, x, h):
        F = self.intermediate
        gate_up = ctx.rows("mlp.gate_up", 2 * F)
        ops.linear(gate_up, h, self.w_gate_up)
        act = ctx.rows("mlp.act", F)
        ops.swiglu(act, gate_up[:, :F], gate_up[:, F:])
        ops.linear(x, act, self.w_down, accumulate=True)
