"""Descriptions of the parts a model is put together from.

An architecture turns its configuration into a `ModelSpec`: a list of
`LayerSpec`s (each naming its mixer, feed-forward and norms with all their sizes
and constants), the order in which the layers run (`ScheduleEntry`), and the
embedding / final norm / head.  Nothing in here knows any particular model; the
part classes in `hfee_amd.parts` are chosen by the `kind` strings, layer by layer.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional


@dataclass(frozen=True)
class NormSpec:
    kind: str            # key in the norm registry, e.g. "rmsnorm"
    width: int
    eps: float
    params: tuple = ()   # extra (name, value) pairs for other kinds


@dataclass(frozen=True)
class PositionSpec:
    kind: str            # key in the position-encoding registry, e.g. "rope"
    params: tuple = ()   # (name, value) pairs; see each kind's part

    def get(self, name: str, default: Any = None):
        return dict(self.params).get(name, default)


@dataclass(frozen=True)
class MixerSpec:
    kind: str            # key in the mixer registry, e.g. "attention"
    params: tuple = ()
    position: Optional[PositionSpec] = None

    def get(self, name: str, default: Any = None):
        return dict(self.params).get(name, default)


@dataclass(frozen=True)
class FeedForwardSpec:
    kind: str            # key in the feed-forward registry, e.g. "gated_mlp"
    params: tuple = ()

    def get(self, name: str, default: Any = None):
        return dict(self.params).get(name, default)


@dataclass(frozen=True)
class EmbeddingSpec:
    kind: str = "lookup"      # key in the embedding registry
    params: tuple = ()

    def get(self, name: str, default: Any = None):
        return dict(self.params).get(name, default)


@dataclass(frozen=True)
class HeadSpec:
    kind: str = "norm_linear"   # key in the head registry: final norm, then the vocabulary product
    params: tuple = ()

    def get(self, name: str, default: Any = None):
        return dict(self.params).get(name, default)


@dataclass(frozen=True)
class CacheNeed:
    """What one cache layer of a part needs of the paged cache.  token_shape: the elements
    that a token adds to the layer (keys and values of attention: (2, kv_heads, head_dim); a
    latent vector: (width,)); how they are arranged inside a page is the part's own affair
    (`layout` names it: two parts may share a cache layer only if they agree on it).  Cache
    layers with equal needs share a group of pages."""
    kind: str                 # "full": every token is kept; "window": the last `window` tokens
    token_shape: tuple
    window: int = 0
    layout: str = ""


@dataclass(frozen=True)
class LayerSpec:
    """One block: how norm, mixer, feed-forward and the residual stream are arranged."""
    arrangement: str     # key in the block registry, e.g. "prenorm"
    hidden: int
    mixer: MixerSpec
    feed_forward: FeedForwardSpec
    mixer_norm: NormSpec
    feed_forward_norm: NormSpec
    prefix: str          # tensor-name prefix of this layer, e.g. "model.layers.3."
    names: tuple = ()    # (role, tensor-name suffix) pairs overriding the parts' defaults

    def name_of(self, role: str, default: str) -> str:
        return self.prefix + dict(self.names).get(role, default)


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  `cache` is the cache layer whose keys/values (or other
    growing memory) the mixer reads; `writes_cache` is False for a layer that only
    reads what another entry has written."""
    layer: int
    cache: int
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden: int
    vocab: int
    layers: tuple            # of LayerSpec
    schedule: tuple          # of ScheduleEntry
    final_norm: NormSpec
    embedding_name: str
    final_norm_name: str
    head_name: Optional[str]   # None: the head shares the embedding table
    max_positions: int
    eos_token_ids: tuple = ()
    bos_token_id: Optional[int] = None
    ignored_tensor_suffixes: tuple = ()   # names in a checkpoint that are not weights
    embedding: EmbeddingSpec = EmbeddingSpec()
    head: HeadSpec = HeadSpec()


def params(**kw) -> tuple:
    """Helper: keyword arguments to the sorted (name, value) tuple the specs hold."""
    return tuple(sorted(kw.items()))
