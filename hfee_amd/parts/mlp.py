"""The gated feed-forward (/root/reference/internal/llm/forward.go:110-114,
/root/reference/internal/ggml/ops.go:159-165): down(activation(gate(h)) * up(h)), added to
the residual stream; the reference's activation is the SiLU, and which one it is is a
parameter of the part (`activation`: one of `ops.GATE_ACTIVATIONS`).  gate and up run as
one product over a weight whose rows alternate gate_j, up_j, so that the gate is the
product's epilogue (and a step of at most 64 tokens folds the norm in front of it into
the same launch)."""
from __future__ import annotations

import torch

from ..config.specs import FeedForwardSpec
from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import FeedForward, LazyNorm, register_feed_forward


@register_feed_forward("gated_mlp")
class GatedMLP(FeedForward):
    graph_safe = True
    takes_lazy_norm = True
    emits_norm = True
    second_half_rows = ops.SKINNY_MAX_ROWS

    def __init__(self, spec: FeedForwardSpec, prefix: str, dtype: torch.dtype):
        self.hidden = spec.get("hidden")
        self.intermediate = spec.get("intermediate")
        self.activation = spec.get("activation", "silu")
        if self.activation not in ops.GATE_ACTIVATIONS:
            raise ValueError(f"the gated feed-forward has the activations {sorted(ops.GATE_ACTIVATIONS)}, "
                             f"not {self.activation!r}")
        self.prefix, self.dtype = prefix, dtype
        self.w_gate_up = self.w_down = None

    def tensor_specs(self):
        p = self.prefix
        return [TensorSpec(p + "gate_proj.weight", (self.intermediate, self.hidden)),
                TensorSpec(p + "up_proj.weight", (self.intermediate, self.hidden)),
                TensorSpec(p + "down_proj.weight", (self.hidden, self.intermediate))]

    def bind(self, tensors):
        p = self.prefix
        self.w_gate_up = torch.stack([tensors.pop(p + "gate_proj.weight"), tensors.pop(p + "up_proj.weight")],
                                     dim=1).reshape(2 * self.intermediate, self.hidden).contiguous()
        self.w_down = tensors.pop(p + "down_proj.weight").contiguous()
        # a second copy in tiles for steps of up to 64 rows, whose products stream the weights
        self.aligned = self.dtype == torch.bfloat16 and self.hidden % 8 == 0 and self.intermediate % 8 == 0
        tiles = ops.tile_weights_if_room(self.w_gate_up, self.w_down) if self.aligned else None
        self.streams = tiles is not None
        self.w_gate_up_tiles, self.w_down_tiles = tiles if tiles else (None, None)
        if not self.streams:      # (nobody finishes a norm here that the part before has begun)
            self.second_half_rows = 0

    def forward_add(self, ctx, x, h, then=None):
        F, n = self.intermediate, ctx.n
        act = ctx.rows("mlp.act", F)
        aligned = self.aligned
        lazy = isinstance(h, LazyNorm)
        if self.streams and n <= ops.SKINNY_MAX_ROWS:        # both products stream the weights' tiles
            w = self.w_gate_up_tiles
            halves = h.row_scale() if lazy else None     # (offered for few rows only)
            norm = None
            if halves is None and lazy and n <= ops.FUSED_NORM_MAX_ROWS and ops.norm_fusion_pays(*w.shape):
                norm = h.fusable()
            # the gate as the product's epilogue, where it is the reference's; another activation is a
            # kernel of its own over the product's alternating columns (the kernels for few rows have
            # no register to spare for a choice in their loops)
            silu = self.activation == "silu"
            out, epilogue = (act, "swiglu") if silu else (ctx.rows("mlp.gate_up", 2 * F), "bf16")
            if halves:        # the norm's first half came with the product before; both projections and the gate
                ops.linear_fused(out, halves[0], w, epilogue, row_scale=halves[1], **ctx.workspace.product_scratch(n, w))
            elif norm:        # norm, both projections and the gate in one launch
                ops.linear_fused(out, h.x, w, epilogue, norm_weight=norm[0], eps=norm[1])
            else:
                ops.linear_fused(out, h.tensor() if lazy else h, w, epilogue, **ctx.workspace.product_scratch(n, w))
            if not silu:
                ops.swiglu(act, out[:, 0::2], out[:, 1::2], activation=self.activation)
            # the down projection adds into x and, if asked, begins the norm that follows
            emit = then.offer() if then is not None else None
            ops.linear_fused(x, act, self.w_down_tiles, "add", emit=emit,
                             **ctx.workspace.product_scratch(n, self.w_down_tiles))
            return
        hn = h.tensor() if lazy else h
        if aligned:   # the gate in the product's epilogue
            ops.linear(act, hn, self.w_gate_up, gate=True, activation=self.activation)
        else:
            gate_up = ctx.rows("mlp.gate_up", 2 * F)
            ops.linear(gate_up, hn, self.w_gate_up)
            ops.swiglu(act, gate_up[:, 0::2], gate_up[:, 1::2], activation=self.activation)
        # the down projection adds into x and, if asked, goes on with the norm that follows
        # (where its K is cut over workgroups: the kernel that adds the cuts up has the row at hand)
        cut = ctx.workspace.split_scratch(n, self.w_down)
        after = then.offer_whole() if then is not None and aligned and cut else None
        if after:
            ops.linear_add_norm(x, act, self.w_down, after["out"], after["weight"], after["eps"], **cut)
        else:
            ops.linear(x, act, self.w_down, accumulate=True, **cut)
