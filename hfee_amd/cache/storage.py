"""Device memory behind the cache manager: the pages of each group and the
state slots.

A group's pages are one tensor [cache layers, pages, page_size * elements a token adds]
in the engine's dtype; how a page is arranged inside is up to the parts that use the
layer, which ask for it under the shape they want (attention: [2, kv_heads,
page_size * head_dim], keys of a (page, head) as [slot][head_dim], values transposed as
[head_dim][slot], the layout its kernels read).  State slots are
tensors [max_requests, ...] that parts with per-request state of fixed size ask
for; a slot is cleared when a request is admitted.
"""
from __future__ import annotations

import torch

from .manager import CacheError


class CacheStorage:
    def __init__(self, groups, page_size: int, pages_per_group, max_requests: int,
                 dtype: torch.dtype, device):
        self.groups = tuple(groups)
        self.page_size = page_size
        self.dtype = dtype
        self.device = device
        self.max_requests = max_requests
        if isinstance(pages_per_group, int):
            pages_per_group = [pages_per_group] * len(self.groups)
        self.pages = []
        self._where = {}
        for g, (spec, n) in enumerate(zip(self.groups, pages_per_group)):
            t = torch.zeros((len(spec.cache_layers), n, page_size * spec.token_elements), dtype=dtype, device=device)
            self.pages.append(t)
            for i, layer in enumerate(spec.cache_layers):
                if layer in self._where:
                    raise CacheError(f"cache layer {layer} is in two groups")
                self._where[layer] = (g, i)
        self.states: dict = {}
        self._views: dict = {}

    def group_of(self, cache_layer: int) -> int:
        return self._where[cache_layer][0]

    def layer(self, cache_layer: int, page_shape=None) -> torch.Tensor:
        """One cache layer: [pages, page_size * elements a token adds], or with page_shape
        (which must have as many elements) [pages, *page_shape]."""
        key = (cache_layer, page_shape)
        view = self._views.get(key)
        if view is None:
            g, i = self._where[cache_layer]
            view = self.pages[g][i]
            if page_shape is not None:
                view = view.view(view.shape[0], *page_shape)       # (raises if the sizes do not match)
            self._views[key] = view
        return view

    def add_state(self, name: str, shape, dtype: torch.dtype) -> torch.Tensor:
        """A per-request state of fixed size: [max_requests, *shape], indexed by slot."""
        if name in self.states:
            raise CacheError(f"state {name!r} is registered twice")
        t = torch.zeros((self.max_requests, *shape), dtype=dtype, device=self.device)
        self.states[name] = t
        return t

    def clear_slot(self, slot: int) -> None:
        for t in self.states.values():
            t[slot].zero_()

    def bytes_per_page(self, group: int) -> int:
        t = self.pages[group]
        return t.shape[0] * t[0, 0].numel() * t.element_size()


def bytes_per_token(groups, dtype: torch.dtype) -> int:
    size = torch.empty((), dtype=dtype).element_size()
    return sum(len(g.cache_layers) * g.token_elements * size for g in groups)
