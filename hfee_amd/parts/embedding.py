"""Token embedding and the output head.

Embedding: a row gather into the float32 residual stream, no scaling
(/root/reference/internal/llm/forward.go:75-77).  Head: final norm and the
vocabulary product only for the rows whose logits are wanted
(/root/reference/internal/llm/forward.go:117-141); it shares the embedding table
when the model has no separate head (/root/reference/internal/llm/model.go:118-121).
"""
from __future__ import annotations

import torch

from ..config.specs import EmbeddingSpec, HeadSpec
from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import Part, register_embedding, register_head


@register_embedding("lookup")
class Embedding(Part):
    """constructor of every embedding kind: (spec, tensor name, vocabulary, width, engine dtype);
    `table` is what a head without a matrix of its own shares."""
    graph_safe = True

    def __init__(self, spec: EmbeddingSpec, name: str, vocab: int, hidden: int, dtype: torch.dtype = None):
        self.name, self.vocab, self.hidden = name, vocab, hidden
        self.table = None

    def tensor_specs(self):
        return [TensorSpec(self.name, (self.vocab, self.hidden))]

    def bind(self, tensors):
        self.table = tensors[self.name].contiguous()

    # forward takes the normed input of the first block as `then` (a LazyNorm), and may do
    # the first half of that norm on its way
    emits_norm = True

    def forward(self, ctx, x, then=None):
        emit = None
        if then is not None and ops.can_embed_emit(self.table, ctx.n):
            emit = then.offer(blocks=ops.embed_emit_blocks(self.hidden))
        ops.embed(x, self.table, ctx.token_ids, emit=emit)


@register_head("norm_linear")
class Head(Part):
    """constructor of every head kind: (spec, the final norm part, tensor name or None to share
    the embedding's table, vocabulary, width, the embedding part, engine dtype)."""
    graph_safe = True

    def __init__(self, spec: HeadSpec, norm, name, vocab: int, hidden: int, embedding, dtype: torch.dtype):
        self.norm, self.name, self.vocab, self.hidden = norm, name, vocab, hidden
        self.embedding, self.dtype = embedding, dtype
        self.weight = None

    def parts(self):
        return [self.norm, self]

    def tensor_specs(self):
        specs = self.norm.tensor_specs()
        if self.name is not None:
            specs.append(TensorSpec(self.name, (self.vocab, self.hidden)))
        return specs

    def bind(self, tensors):
        self.norm.bind(tensors)
        self.weight = tensors[self.name].contiguous() if self.name is not None else self.embedding.table
        # a second copy in tiles for up to 64 wanted rows, whose product streams the weights (of a
        # table shared with the embedding too: the lookup reads rows as they lie); like every second
        # copy only while it leaves room, else the wanted rows go through the kernels for rows
        self.weight_tiles = None
        if self.dtype == torch.bfloat16 and self.weight.dtype == torch.bfloat16 and self.hidden % 8 == 0:
            tiles = ops.tile_weights_if_room(self.weight)
            self.weight_tiles = tiles[0] if tiles else None
        self.streams = self.weight_tiles is not None

    def forward(self, ctx, logits, x, rows):
        """logits[i] = head(norm(x[rows[i]])); logits float32 [len(rows), vocab]."""
        w = logits.shape[0]
        fused = getattr(self.norm, "fused_form", lambda: None)()
        if self.streams and w <= ops.SKINNY_MAX_ROWS:
            if fused and w <= ops.FUSED_NORM_MAX_ROWS and ops.norm_fusion_pays(self.vocab, self.hidden):
                ops.linear_fused(logits, x, self.weight_tiles, "f32", norm_weight=fused[0], eps=fused[1], rows=rows, m=w)
                return
            normed = ctx.rows("head.normed", self.hidden, n=w)
            self.norm.forward(ctx, normed, x, rows)
            ops.linear_fused(logits, normed, self.weight_tiles, "f32", **ctx.workspace.product_scratch(w, self.weight_tiles))
            return
        normed = ctx.rows("head.normed", self.hidden, n=w)
        self.norm.forward(ctx, normed, x, rows)
        ops.linear(logits, normed, self.weight)
