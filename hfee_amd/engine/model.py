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
from ..parts import Embedding, Head, lookup
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
        self.embedding = Embedding(spec.embedding_name, spec.vocab, spec.hidden)
        self.blocks = [lookup("block", ls.arrangement)(ls, dtype) for ls in spec.layers]
        final_norm = lookup("norm", spec.final_norm.kind)(spec.final_norm, spec.final_norm_name)
        self.head = Head(final_norm, spec.head_name, spec.vocab, spec.hidden, self.embedding, dtype)
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

    # ---- cache
    def cache_groups(self):
        """Cache layers with the same needs share a group.  A cache layer's needs
        are those of the mixer that writes it."""
        needs: dict = {}
        for e in self.schedule:
            spec = self.blocks[e.layer].mixer.cache_spec()
            if spec is None:
                continue
            if e.writes_cache:
                if e.cache in needs and needs[e.cache] != spec:
                    raise ValueError(f"cache layer {e.cache} is written by mixers with different needs")
                needs[e.cache] = spec
        for e in self.schedule:
            spec = self.blocks[e.layer].mixer.cache_spec()
            if spec is not None and not e.writes_cache:
                if e.cache not in needs:
                    raise ValueError(f"layer {e.layer} reads cache layer {e.cache}, which no layer writes")
                writer = next(w for w in self.schedule if w.cache == e.cache and w.writes_cache)
                mine = getattr(self.blocks[e.layer].mixer, "key_layout", lambda: None)()
                theirs = getattr(self.blocks[writer.layer].mixer, "key_layout", lambda: None)()
                if needs[e.cache][1:3] != spec[1:3] or mine != theirs:
                    raise ValueError(f"layer {e.layer} cannot read cache layer {e.cache}: its keys are laid out "
                                     f"differently from those that layer {writer.layer} writes")
        by_need: dict = {}
        for layer, spec in sorted(needs.items()):
            by_need.setdefault(spec, []).append(layer)
        return [CacheGroupSpec(kind=k, kv_heads=kv, head_dim=hd, window=w, cache_layers=tuple(layers))
                for (k, kv, hd, w), layers in by_need.items()]

    def mixers(self):
        return [b.mixer for b in self.blocks]

    def prepare(self, info: EngineInfo):
        for m in self.mixers():
            m.prepare(info)


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
