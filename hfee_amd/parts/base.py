"""What every part has in common: how it names its tensors, how it is registered,
and what a step hands it.

A part gets all its sizes and constants through its spec; it never learns which
model it is in.  Eight kinds, each with a registry from the spec's `kind` string to
a class:

  embedding       forward(ctx, x): the residual stream's first value from the token ids
                  (with `emits_norm = True`: forward(ctx, x, then=None), see LazyNorm)
  norm            forward(ctx, out, x, rows=None)
  position        prepare(num_positions, device); applied by the mixer that owns it
  mixer           forward_add(ctx, x, h, cache_layer, writes_cache): x += mix(h)
  projection_step forward(ctx, q, k, v): what a mixer does to its projections before it applies
                  the position (a bias, a norm over each head); named by the attention
                  mixer's `after_projection` parameter, see ProjectionStep
  feed_forward    forward_add(ctx, x, h):                            x += ffn(h)
  block           forward(ctx, x, entry): one layer's arrangement of the above
  head            forward(ctx, logits, x, rows): logits of the wanted rows

Every part, whatever its kind, may also ask for per-request state of fixed size
(state_specs), prepare itself before the first step (prepare), add int32 metadata to
every step (plan), and, through its block, for a layer of the paged cache (cache_spec):
the engine collects these from all parts of the model alike.

`x` is the residual stream, float32 [n, hidden]; `h` is a normed copy in the
engine's dtype.  Every part also has tensor_specs() -> [TensorSpec] and
bind(tensors) (take your tensors out of the dict by full name).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import torch


_REGISTRIES: dict[str, dict] = {"norm": {}, "position": {}, "mixer": {}, "feed_forward": {}, "block": {},
                                "embedding": {}, "head": {}, "projection_step": {}}


def _register(family: str, kind: str, cls):
    _REGISTRIES[family][kind] = cls
    return cls


def register_norm(kind: str, cls=None):
    return _register("norm", kind, cls) if cls else (lambda c: _register("norm", kind, c))


def register_position(kind: str, cls=None):
    return _register("position", kind, cls) if cls else (lambda c: _register("position", kind, c))


def register_mixer(kind: str, cls=None):
    return _register("mixer", kind, cls) if cls else (lambda c: _register("mixer", kind, c))


def register_feed_forward(kind: str, cls=None):
    return _register("feed_forward", kind, cls) if cls else (lambda c: _register("feed_forward", kind, c))


def register_block(kind: str, cls=None):
    return _register("block", kind, cls) if cls else (lambda c: _register("block", kind, c))


def register_embedding(kind: str, cls=None):
    return _register("embedding", kind, cls) if cls else (lambda c: _register("embedding", kind, c))


def register_projection_step(kind: str, cls=None):
    return _register("projection_step", kind, cls) if cls else (lambda c: _register("projection_step", kind, c))


def register_head(kind: str, cls=None):
    return _register("head", kind, cls) if cls else (lambda c: _register("head", kind, c))


def lookup(family: str, kind: str):
    try:
        return _REGISTRIES[family][kind]
    except KeyError:
        known = ", ".join(sorted(_REGISTRIES[family])) or "none"
        raise KeyError(f"no {family} part is registered under {kind!r} (known: {known})") from None


class Part:
    """Base of all parts."""

    # True if forward reads nothing from the host that changes between steps (only
    # device tensors of the context), so that a decode step may be captured once as
    # a HIP graph and replayed.  A part that leaves it False keeps its model eager.
    graph_safe = False
    # True if forward_add accepts a LazyNorm in place of the normed tensor.
    takes_lazy_norm = False
    # True if forward_add accepts `then=` (the LazyNorm of the norm that follows this
    # part) and may do that norm's first half in its last product.
    emits_norm = False
    # Up to how many rows in a step forward_add finishes a norm whose first half a part
    # before it has done (LazyNorm.row_scale); 0: never.
    second_half_rows = 0

    def tensor_specs(self) -> list:
        return []

    def bind(self, tensors: dict) -> None:
        pass

    def parts(self) -> list:
        """The parts this one is made of, itself included if it has hooks of its own (a
        block lists its norms, mixer and feed-forward)."""
        return [self]

    def cache_spec(self):
        """None, or a CacheNeed: the growing memory that one cache layer of this part
        needs.  The engine asks a layer's block, which answers for the part of it that
        reads and writes the cache layer named by the schedule."""
        return None

    def state_specs(self) -> list:
        """Per-request states of fixed size: [(name, shape, dtype)].  The engine keeps
        one tensor [max_requests, *shape] per name (info.storage.states[name], indexed
        by a request's slot) and clears a slot when a request is admitted."""
        return []

    def prepare(self, engine_info) -> None:
        """Called once before the first step (tables, state tensors...)."""

    def plan(self, plan) -> None:
        """Called once per step before the metadata goes to the device; may add
        int32 arrays with plan.add(key, array) (they arrive as ctx.extra[key]) and
        host values with plan.host[key] = value."""


class Mixer(Part):
    """Mixes information between the tokens of a sequence."""

    def forward_add(self, ctx, x, h, cache_layer: int, writes_cache: bool) -> None:
        raise NotImplementedError


class ProjectionStep(Part):
    """What stands between a mixer's projections and the position encoding: a bias on q, k
    and v, a norm over each head of q and k, anything that works row by row.  The attention
    mixer builds one from its `after_projection` parameter, a (kind, params) pair, with the
    constructor (params, prefix, num_heads, kv_heads, head_dim, dtype); a mixer that has one
    runs its projections, this step and the rotation as launches of their own (the fused
    epilogues know nothing of it)."""

    def bind(self, tensors: dict, order=None) -> None:
        """order: the attention mixer keeps the rows of a q or k head in an order of its own
        (rotation pairs side by side); element j of a head as this step sees it is element
        order[j] of the head in the checkpoint.  Per-dimension tensors of q and k must follow."""

    def forward(self, ctx, q, k, v) -> None:
        """In place: q [n, num_heads * head_dim], k and v [n, kv_heads * head_dim] (None where
        this run of the layer reads another run's cache), in the engine's dtype."""
        raise NotImplementedError


class FeedForward(Part):
    def forward_add(self, ctx, x, h) -> None:
        raise NotImplementedError


class Norm(Part):
    def forward(self, ctx, out, x, rows=None) -> None:
        raise NotImplementedError


class LazyNorm:
    """A normed copy of the residual stream that is made only when someone asks for
    it.  A part that sets `takes_lazy_norm = True` gets one of these instead of a
    tensor and may fold the norm into its first product (`fusable()`), or call
    `tensor()` for the materialised rows.

    The norm may also be done in two halves around it, without a launch of its own: a
    part whose last step adds into the residual stream (`emits_norm = True`) is handed
    the LazyNorm of what follows it as `then`; if `then.offer()` returns arguments, its
    adding product also writes bfloat16(x_new * weight) and the rows' sums of squares
    (`ops.linear_fused(..., emit=...)`).  The part that consumes the norm then finds
    `pending` set and gives it to its first product as `row_scale`.  An embedding with
    `emits_norm = True` is handed the first block's LazyNorm in the same way."""

    def __init__(self, ctx, norm, x, second_half_rows: int = 0):
        self.ctx, self.norm, self.x = ctx, norm, x
        self.second_half_rows = second_half_rows      # of the part that will consume this norm
        self._tensor = None
        self.pending = None      # dict(out, shares, blocks, eps) once a producer has done the first half

    def fusable(self):
        """(weight, eps) if the norm is y = x / sqrt(mean(x^2) + eps) * weight, else None."""
        return getattr(self.norm, "fused_form", lambda: None)()

    def offer(self, blocks: int | None = None):
        """For the part that writes x last: the `emit` arguments of its adding product, or None
        if this norm cannot be split (then nothing changes for anybody).  blocks: in how many
        shares the producer leaves a row's sum of squares (one for every 16 columns unless it
        says otherwise)."""
        form = self.fusable()
        if form is None or self.x.dtype != torch.float32 or self.ctx.n > self.second_half_rows:
            return None
        weight, eps = form
        width = self.x.shape[1]
        most = (width + 15) // 16
        blocks = blocks or most
        out = self.ctx.rows("block.emitted", width, torch.bfloat16)
        # (one size for every producer: the buffer is made once)
        shares = self.ctx.workspace.flat("block.emitted_shares", max(blocks, most) * 64, torch.float32)[:blocks * 64]
        self.pending = dict(out=out, shares=shares, blocks=blocks, eps=eps)
        return dict(weight=weight, out=out, shares=shares)

    def offer_whole(self):
        """For the part that adds into x last with bfloat16 operands: dict(out, weight, eps) if
        its adding product may also write the whole norm of the new rows into `out`
        (`ops.linear_add_norm`); the part that takes the offer has to fill `out`.  None if this
        norm is not of that form (then nothing changes for anybody)."""
        form = self.fusable()
        if form is None or self.x.dtype != torch.float32 or self._tensor is not None or self.pending is not None:
            return None
        out = self.ctx.rows("block.normed", self.x.shape[1])
        if out.dtype != torch.bfloat16:
            return None
        self._tensor = out
        return dict(out=out, weight=form[0], eps=form[1])

    def row_scale(self):
        """For the consuming part: (emitted tensor, `row_scale` arguments) if a producer has
        done the first half, else None."""
        if self.pending is None:
            return None
        p = self.pending
        return p["out"], dict(shares=p["shares"], blocks=p["blocks"], eps=p["eps"])

    def tensor(self):
        if self._tensor is None:       # (also after an offer: x is complete, the whole norm is always right)
            self._tensor = self.ctx.rows("block.normed", self.x.shape[1])
            self.norm.forward(self.ctx, self._tensor, self.x)
        return self._tensor


@dataclass
class Segment:
    """One request's share of a step (host side)."""
    request_id: object
    slot: int        # state slot
    start: int       # tokens already in the cache
    length: int      # new tokens in this step
    row0: int        # first row of the segment in the flattened batch


class Workspace:
    """Scratch buffers by name, allocated once for `capacity` rows and reused by
    every step (the reference allocates its scratch per call,
    /root/reference/internal/llm/forward.go:66-73)."""

    def __init__(self, capacity: int, device):
        self.capacity = capacity
        self.device = device
        self._buffers: dict = {}
        self._retired: list = []     # outgrown buffers stay alive: captured graphs may still point at them

    def rows(self, name: str, n: int, width: int, dtype: torch.dtype) -> torch.Tensor:
        """A [n, width] view of the buffer `name` ([capacity, width])."""
        if n > self.capacity:
            raise ValueError(f"a step of {n} tokens exceeds the workspace of {self.capacity}")
        key = (name, width, dtype)
        buf = self._buffers.get(key)
        if buf is None:
            buf = self._buffers[key] = torch.empty((self.capacity, width), dtype=dtype, device=self.device)
        return buf[:n]

    def flat(self, name: str, count: int, dtype: torch.dtype) -> torch.Tensor:
        key = (name, "flat", dtype)
        buf = self._buffers.get(key)
        if buf is None or buf.numel() < count:
            if buf is not None:
                self._retired.append(buf)
            buf = self._buffers[key] = torch.empty((count,), dtype=dtype, device=self.device)
        return buf[:count]

    def product_scratch(self, n_rows: int, weight: torch.Tensor) -> dict:
        """The `scratch` argument of `ops.linear_fused` for a product of n_rows rows with
        this weight (empty where it has no use for it)."""
        from ..kernels import ops
        words = ops.mid_rows_scratch(n_rows, weight.shape[0], weight.shape[1])
        if not words:
            return {}
        return dict(scratch=self.flat("product.partial", words, torch.float32))

    def split_scratch(self, n_rows: int, weight: torch.Tensor) -> dict:
        """The `scratch` argument of `ops.linear` for a bfloat16 product of n_rows rows with
        this weight (empty where it has no use for it)."""
        from ..kernels import ops
        if weight.dtype != torch.bfloat16:
            return {}
        words = ops.linear_scratch(n_rows, weight.shape[0], weight.shape[1])
        return dict(scratch=self.flat("product.partial", words, torch.float32)) if words else {}

    def counters(self, name: str, count: int) -> torch.Tensor:
        """`count` int32 that are zero, for kernels whose workgroups count themselves
        (the one that finishes last does a final piece of work and sets the counter
        back to zero, so the buffer is zero again whenever a kernel has run)."""
        key = (name, "counters", torch.int32)
        buf = self._buffers.get(key)
        if buf is None or buf.numel() < count:
            if buf is not None:
                self._retired.append(buf)
            buf = self._buffers[key] = torch.zeros((max(count, 256),), dtype=torch.int32, device=self.device)
        return buf[:count]


@dataclass
class StepContext:
    """What a step hands to the parts.  Device tensors are int32."""
    n: int
    dtype: torch.dtype
    device: object
    segments: list                      # of Segment (host)
    token_ids: torch.Tensor             # [n]
    positions: torch.Tensor             # [n] absolute position of each token
    token_segment: torch.Tensor         # [n] index of the token's segment
    segment_slots: torch.Tensor         # [segments] state slot of each segment
    segment_starts: torch.Tensor        # [segments] tokens cached before this step
    segment_lengths: torch.Tensor       # [segments]
    segment_rows: torch.Tensor          # [segments] first row in the batch
    block_tables: list                  # per cache group: [segments, blocks] page ids
    max_position: int                   # largest position in the step (host)
    storage: object                     # CacheStorage
    workspace: Workspace
    page_size: int
    extra: dict = field(default_factory=dict)   # arrays that parts planned: key -> device tensor
    host: dict = field(default_factory=dict)    # host-side values that parts planned

    def rows(self, name: str, width: int, dtype: Optional[torch.dtype] = None, n: Optional[int] = None):
        return self.workspace.rows(name, self.n if n is None else n, width, dtype or self.dtype)
