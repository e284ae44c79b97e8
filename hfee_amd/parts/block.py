"""How a layer's parts are arranged around the residual stream.

"prenorm" is the reference's block (/root/reference/internal/llm/forward.go:79-115):
x += mixer(norm(x)); x += feed_forward(norm(x)).
"""
from __future__ import annotations

import torch

from ..config.specs import LayerSpec
from .base import LazyNorm, Part, lookup, register_block


@register_block("prenorm")
class PreNormBlock(Part):
    def __init__(self, spec: LayerSpec, dtype: torch.dtype):
        self.spec, self.dtype = spec, dtype
        self.mixer_norm = lookup("norm", spec.mixer_norm.kind)(
            spec.mixer_norm, spec.name_of("mixer_norm", "mixer_norm.") + "weight")
        self.mixer = lookup("mixer", spec.mixer.kind)(spec.mixer, spec.name_of("mixer", "mixer."), dtype)
        self.feed_forward_norm = lookup("norm", spec.feed_forward_norm.kind)(
            spec.feed_forward_norm, spec.name_of("feed_forward_norm", "feed_forward_norm.") + "weight")
        self.feed_forward = lookup("feed_forward", spec.feed_forward.kind)(
            spec.feed_forward, spec.name_of("feed_forward", "feed_forward."), dtype)
        self.hidden = spec.hidden

    def parts(self):
        # (each with the parts it is made of itself: a mixer lists a step behind its projections)
        return [q for p in self._own() for q in p.parts()]

    def _own(self):
        return [self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward]

    # the layer of the paged cache that a run of this block is given belongs to its mixer
    def cache_spec(self):
        return self.mixer.cache_spec()

    def key_layout(self):
        return getattr(self.mixer, "key_layout", lambda: None)()

    def tensor_specs(self):
        return [s for p in self._own() for s in p.tensor_specs()]

    def bind(self, tensors):
        for p in self._own():
            p.bind(tensors)

    # forward takes the normed input that the block before may have begun, and that of
    # the block after, which this block's last part may begin (the engine makes both with
    # `begin` for blocks that say so)
    chains_norms = True

    def begin(self, ctx, x):
        """The block's normed input, not yet computed."""
        return LazyNorm(ctx, self.mixer_norm, x, self.mixer.second_half_rows)

    def forward(self, ctx, x, entry, h_in=None, h_next=None):
        h = h_in if h_in is not None else self.begin(ctx, x)
        h2 = LazyNorm(ctx, self.feed_forward_norm, x, self.feed_forward.second_half_rows)
        self._run(self.mixer, ctx, x, h, h2, entry.cache, entry.writes_cache)
        self._run(self.feed_forward, ctx, x, h2, h_next)

    @staticmethod
    def _run(part, ctx, x, h, then, *args):
        h = h if part.takes_lazy_norm else h.tensor()
        if then is not None and part.emits_norm:
            part.forward_add(ctx, x, h, *args, then=then)
        else:
            part.forward_add(ctx, x, h, *args)
