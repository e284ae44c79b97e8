"""A model: embedding, the layers in the order the schedule gives, final norm and
head, built from a ModelSpec by looking every part up in the registries.

It mirrors the reference's Model (/root/reference/internal/llm/model.go:35-48:
embedding, output norm, output matrix, layers) and its build
(/root/reference/internal/llm/model.go:115-141), with the layer list and the run
order as data.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ..cache.manager import CacheGroupSpec
from ..config.registry import config_from_folder, model_spec_of
from ..config.specs import ModelSpec
from ..parts import lookup
from ..weights.loader import bind_tensors, engine_dtype, load_tensors
from ..weights.random_init import random_tensors


@dataclass
class EngineInfo:
    """What parts may need to know of the engine before the first step."""
    num_positions: int
    device: object
    dtype: torch.dtype
    page_size: int
    max_requests: int
    storage: object = None


class Model:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype):
        self.spec, self.dtype = spec, dtype
        self.embedding = lookup("embedding", spec.embedding.kind)(spec.embedding, spec.embedding_name, spec.vocab,
                                                                  spec.hidden, dtype)
        self.blocks = [lookup("block", ls.arrangement)(ls, dtype) for ls in spec.layers]
        final_norm = lookup("norm", spec.final_norm.kind)(spec.final_norm, spec.final_norm_name)
        self.head = lookup("head", spec.head.kind)(spec.head, final_norm, spec.head_name, spec.vocab, spec.hidden,
                                                   self.embedding, dtype)
        self.schedule = tuple(spec.schedule)
        for e in self.schedule:
            if not 0 <= e.layer < len(self.blocks):
                raise ValueError(f"the schedule names layer {e.layer}, the model has {len(self.blocks)}")
        self.bound = False

    # ---- tensors
    def tensor_specs(self):
        specs = self.embedding.tensor_specs()
        for b in self.blocks:
            specs += b.tensor_specs()
        specs += self.head.tensor_specs()
        return specs

    def bind(self, tensors: dict):
        self.embedding.bind(tensors)
        for b in self.blocks:
            b.bind(tensors)
        self.head.bind(tensors)
        self.bound = True

    # ---- parts
    def parts(self):
        """Every part of the model once, in running order: the embedding, each layer's
        parts, the head's.  Whatever a part asks of the engine (state, preparation, a
        step's metadata, graph capture) is collected over this list."""
        out, seen = [], set()
        for owner in [self.embedding, *self.blocks, self.head]:
            for p in owner.parts():
                if id(p) not in seen:
                    seen.add(id(p))
                    out.append(p)
        return out

    # ---- cache
    def cache_groups(self):
        """Cache layers with the same needs share a group.  A cache layer's needs are
        those of the block that writes it (a block answers for the part of it that uses
        the cache)."""
        needs: dict = {}
        for e in self.schedule:
            need = self.blocks[e.layer].cache_spec()
            if need is None:
                continue
            if e.writes_cache:
                if e.cache in needs and needs[e.cache] != need:
                    raise ValueError(f"cache layer {e.cache} is written by layers with different needs")
                needs[e.cache] = need
        for e in self.schedule:
            need = self.blocks[e.layer].cache_spec()
            if need is not None and not e.writes_cache:
                if e.cache not in needs:
                    raise ValueError(f"layer {e.layer} reads cache layer {e.cache}, which no layer writes")
                writer = next(w for w in self.schedule if w.cache == e.cache and w.writes_cache)
                mine = getattr(self.blocks[e.layer], "key_layout", lambda: None)()
                theirs = getattr(self.blocks[writer.layer], "key_layout", lambda: None)()
                theirs_need = needs[e.cache]
                if (theirs_need.token_shape, theirs_need.layout) != (need.token_shape, need.layout) or mine != theirs:
                    raise ValueError(f"layer {e.layer} cannot read cache layer {e.cache}: its keys are laid out "
                                     f"differently from those that layer {writer.layer} writes")
        by_need: dict = {}
        for layer, need in sorted(needs.items()):
            by_need.setdefault(need, []).append(layer)
        return [CacheGroupSpec(kind=n.kind, token_shape=tuple(n.token_shape), window=n.window, layout=n.layout,
                               cache_layers=tuple(layers))
                for n, layers in by_need.items()]

    def state_specs(self):
        return [s for p in self.parts() for s in p.state_specs()]

    def prepare(self, info: EngineInfo):
        for p in self.parts():
            p.prepare(info)

    def plan(self, plan):
        for p in self.parts():
            p.plan(plan)

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in self.parts())


def declared_tensors(config):
    """Every tensor the architecture's parts declare for this configuration."""
    return Model(model_spec_of(config), torch.float32).tensor_specs()


def load_model(model_dir: str, dtype="bfloat16", device="cuda:0"):
    """config.json chooses the architecture; the safetensors are bound by name."""
    dtype = engine_dtype(dtype)
    config = config_from_folder(model_dir)
    spec = model_spec_of(config)
    model = Model(spec, dtype)
    tensors = load_tensors(model_dir, model.tensor_specs(), dtype, device, spec.ignored_tensor_suffixes)
    model.bind(tensors)
    return model, config


def random_model(config, seed: int = 0, dtype="bfloat16", device="cuda:0", std: float = 0.02,
                 norm_init=None):
    """The model with seeded random weights made on the device (no folder written)."""
    dtype = engine_dtype(dtype)
    spec = model_spec_of(config)
    model = Model(spec, dtype)
    specs = model.tensor_specs()
    tensors = random_tensors(specs, seed, std, dtype, device, norm_init)
    model.bind(bind_tensors(tensors, specs, dtype, device, "random weights", spec.ignored_tensor_suffixes))
    return model
