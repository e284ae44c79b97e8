"""Attention over the paged cache, with grouped KV heads and an optional window.

The reference's layer (/root/reference/internal/llm/forward.go:83-107): project to
q, k, v; rotate q and k at the token's position; write k (rotated) and v to the
cache; each token attends to the keys of its own sequence up to its position, head
h reading KV head h // (heads / kv_heads), scores scaled by `scale`; project back
and add to the residual stream.

The three projections run as one product over the concatenated weight.  In
bfloat16, portions of prompts go through the tiled matrix-core kernel (tiles of 32
positions), single decoded tokens through the split-key kernel; in float32 every
token goes through the plain kernel.

Rotation pairs are made adjacent when the weights are bound: for the pairing
(i, i + half) the rows of the q and k projections are reordered inside each head to
(2i, 2i + 1).  Scores are dot products over the head, so reordering q and k alike
changes nothing (the reference states the same relation between its two pairings,
/root/reference/internal/llm/forward.go:187-190), and adjacent pairs let a step of at
most 64 tokens do norm, projections, rotation and the cache write in one launch.
"""
from __future__ import annotations

import numpy as np
import torch

from ..config.specs import CacheNeed, MixerSpec
from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import LazyNorm, Mixer, lookup, register_mixer

_TILE = 32            # query rows per workgroup of the prefill kernel, keys per tile
_DECODE_WAVES = 4     # waves of a decode workgroup; each takes every 4th key tile
_TILES_PER_WAVE = 16  # beyond this many tiles per wave the keys are always split over workgroups
_DECODE_WORKGROUPS = 256   # with fewer (segment, KV head) pairs than this the keys are split to fill the chip


@register_mixer("attention")
class Attention(Mixer):
    graph_safe = True
    takes_lazy_norm = True
    emits_norm = True
    second_half_rows = ops.SKINNY_MAX_ROWS

    def __init__(self, spec: MixerSpec, prefix: str, dtype: torch.dtype):
        self.hidden = spec.get("hidden")
        self.num_heads = spec.get("num_heads")
        self.kv_heads = spec.get("num_kv_heads", self.num_heads)
        self.head_dim = spec.get("head_dim")
        self.scale = float(spec.get("scale", self.head_dim ** -0.5))
        self.window = int(spec.get("window", 0) or 0)
        if self.num_heads % self.kv_heads:
            raise ValueError(f"{self.num_heads} heads are not a multiple of {self.kv_heads} kv heads")
        if dtype == torch.bfloat16 and (self.head_dim % 16 or not 16 <= self.head_dim <= 256):
            raise ValueError(f"the bfloat16 attention kernels take head sizes 16..256 in steps of 16, "
                             f"not {self.head_dim}")
        if self.head_dim > 256:
            raise ValueError(f"head sizes above 256 are not built, got {self.head_dim}")
        self.prefix, self.dtype = prefix, dtype
        self.position = lookup("position", spec.position.kind)(spec.position) if spec.position else None
        # an optional step between the projections and the rotation: (kind, params)
        step = spec.get("after_projection")
        self.after_projection = None
        if step is not None:
            self.after_projection = lookup("projection_step", step[0])(dict(step[1]), prefix, self.num_heads, self.kv_heads,
                                                                       self.head_dim, dtype)
            self.second_half_rows = 0      # (the product that would finish a norm's second half is the fused one)
        self.q_width = self.num_heads * self.head_dim
        self.kv_width = self.kv_heads * self.head_dim
        self.w_qkv = self.w_o = None

    # ---- weights
    def tensor_specs(self):
        p = self.prefix
        return [TensorSpec(p + "q_proj.weight", (self.q_width, self.hidden)),
                TensorSpec(p + "k_proj.weight", (self.kv_width, self.hidden)),
                TensorSpec(p + "v_proj.weight", (self.kv_width, self.hidden)),
                TensorSpec(p + "o_proj.weight", (self.hidden, self.q_width))] + \
            (self.after_projection.tensor_specs() if self.after_projection else [])

    def parts(self):
        return [self] + (self.after_projection.parts() if self.after_projection else [])

    def _pair_order(self, device):
        """Row order inside a head that puts rotation pairs side by side."""
        pos = self.position
        order = torch.arange(self.head_dim, device=device)
        if pos is not None and pos.pairing == 0:
            half = pos.rotary_dim // 2
            order[0:2 * half:2] = torch.arange(half, device=device)
            order[1:2 * half:2] = torch.arange(half, device=device) + half
        return order

    def bind(self, tensors):
        p = self.prefix
        wq, wk = tensors.pop(p + "q_proj.weight"), tensors.pop(p + "k_proj.weight")
        order = self._pair_order(wq.device)
        wq = wq.view(self.num_heads, self.head_dim, self.hidden)[:, order].reshape(self.q_width, self.hidden)
        wk = wk.view(self.kv_heads, self.head_dim, self.hidden)[:, order].reshape(self.kv_width, self.hidden)
        self.w_qkv = torch.cat([wq, wk, tensors.pop(p + "v_proj.weight")], dim=0).contiguous()
        self.w_o = tensors.pop(p + "o_proj.weight").contiguous()
        if self.after_projection is not None:
            self.after_projection.bind(tensors, order)
        self.pairing = 1          # pairs are (2i, 2i + 1) from here on
        # a second copy in tiles for steps of up to 64 rows, whose products stream the weights
        # (as rows they serve the tiled products of longer portions)
        self.streams = self.dtype == torch.bfloat16 and self.hidden % 8 == 0 and self.q_width % 8 == 0
        tiles = ops.tile_weights_if_room(self.w_qkv, self.w_o) if self.streams else None
        self.streams = tiles is not None
        self.w_qkv_tiles, self.w_o_tiles = tiles if tiles else (None, None)
        if not self.streams:      # (nobody finishes a norm here that the part before has begun)
            self.second_half_rows = 0
        # where the q/k/v product of a portion is cut along K, the rotation kernel can add the cuts up
        half = self.position.rotary_dim // 2 if self.position is not None else 0
        self.cuts_into_rotation = (self.dtype == torch.bfloat16 and self.hidden % 8 == 0 and self.head_dim % 8 == 0
                                   and half % 4 == 0)

    def key_layout(self):
        """What two layers must share to read one cache layer."""
        pos = self.position
        return (self.kv_heads, self.head_dim, None if pos is None else pos.signature())

    # ---- cache
    def cache_spec(self):
        # keys of a (page, head) as [slot][head_dim], values transposed: csrc/common.h's CacheLayout
        return CacheNeed("window" if self.window > 0 else "full", (2, self.kv_heads, self.head_dim), self.window,
                         layout="keys by slot, values by dimension")

    def _cache_layer(self, ctx, cache_layer):
        """The cache layer as the kernels take it: [pages, 2, kv_heads, page_size * head_dim]."""
        return ctx.storage.layer(cache_layer, (2, self.kv_heads, ctx.page_size * self.head_dim))

    def prepare(self, info):
        if self.position is not None:
            self.position.prepare(info.num_positions, info.device)

    def plan(self, plan):
        if self.dtype != torch.bfloat16 or "attention.tiles" in plan.arrays:
            return
        tiles, runs, d_rows, d_pos, d_tab = [], [], [], [], []
        for s, seg in enumerate(plan.segments):
            if seg.length == 1:
                d_rows.append(seg.row0)
                d_pos.append(seg.start)
                d_tab.append(s)
            else:
                for off in range(0, seg.length, _TILE):
                    tiles.append((seg.row0 + off, min(_TILE, seg.length - off), seg.start + off, s))
        # (runs of row tiles of a portion that follow one another: for heads that share no keys with another)
        runs = ops.attention_runs(tiles, self.head_dim)
        plan.add("attention.tiles", np.asarray(tiles, dtype=np.int32).reshape(-1, 4))
        plan.add("attention.runs", np.asarray(runs, dtype=np.int32).reshape(-1, 2))
        plan.add("attention.decode_rows", np.asarray(d_rows, dtype=np.int32))
        plan.add("attention.decode_positions", np.asarray(d_pos, dtype=np.int32))
        plan.add("attention.decode_tables", np.asarray(d_tab, dtype=np.int32))
        plan.host["attention.prefill_kernel"] = ops.prefill_attention_kernel(tiles, self.window, self.kv_heads,
                                                                             self.num_heads // self.kv_heads, self.head_dim)
        plan.host["attention.decode_max_position"] = max(d_pos) if d_pos else 0
        # (a step of decoding requests only: segment i is row i and has block table i)
        plan.host["attention.decode_in_order"] = d_rows == list(range(len(d_rows))) and d_tab == d_rows

    # ---- the layer
    def forward_add(self, ctx, x, h, cache_layer: int, writes_cache: bool, then=None):
        H, K, hd = self.num_heads, self.kv_heads, self.head_dim
        n = ctx.n
        group = ctx.storage.group_of(cache_layer)
        cache = self._cache_layer(ctx, cache_layer)
        tables = ctx.block_tables[group]
        pos = self.position
        cos, sin = (pos.cos, pos.sin) if pos else (None, None)
        # (the tiled kernels have the same epilogue for more rows, but there the rotation
        # as a kernel of its own, spread over the whole chip, measured faster than as the
        # tail of 256 x 256 tiles with one wave a SIMD: 135 us against 156 us a layer at
        # 2,048 rows)
        fused = self.streams and n <= ops.SKINNY_MAX_ROWS and self.after_projection is None
        qkv = ctx.rows("attention.qkv", self.q_width + 2 * self.kv_width)
        q = qkv[:, :self.q_width]
        if fused:
            # norm, projections, rotation and the cache write in one launch
            few = n <= ops.FUSED_NORM_MAX_ROWS
            halves = h.row_scale() if isinstance(h, LazyNorm) else None     # first half done before
            norm = h.fusable() if (halves is None and few and isinstance(h, LazyNorm)
                                   and ops.norm_fusion_pays(*self.w_qkv.shape)) else None
            a = halves[0] if halves else h.x if norm else (h.tensor() if isinstance(h, LazyNorm) else h)
            ops.linear_fused(q, a, self.w_qkv_tiles, "qkv", norm_weight=norm[0] if norm else None,
                             eps=norm[1] if norm else 0.0, row_scale=halves[1] if halves else None,
                             qkv=dict(positions=ctx.positions, token_segment=ctx.token_segment, block_tables=tables,
                                      cos=cos, sin=sin, cache_layer=cache if writes_cache else None,
                                      num_heads=H, kv_heads=K, head_dim=hd, page_size=ctx.page_size),
                             **ctx.workspace.product_scratch(n, self.w_qkv_tiles))
        else:
            hn = h.tensor() if isinstance(h, LazyNorm) else h
            portions = self.dtype != torch.bfloat16 or ctx.extra["attention.tiles"].shape[0] > 0
            cuts = 0
            if writes_cache and self.cuts_into_rotation and self.after_projection is None:
                # a product of few tiles, cut along K: the rotation adds the cuts up on its way
                scratch = ctx.workspace.split_scratch(n, self.w_qkv).get("scratch")
                cuts = ops.linear_cuts(hn, self.w_qkv, scratch)
                if cuts:
                    ops.rope_cache_write_cuts(q, scratch, cuts, ctx.positions, ctx.token_segment, tables, cos, sin,
                                              cache, H, K, hd, ctx.page_size, ctx.max_position, portions=portions)
            if not cuts:
                if writes_cache:
                    ops.linear(qkv, hn, self.w_qkv, **ctx.workspace.split_scratch(n, self.w_qkv))
                    k = qkv[:, self.q_width:self.q_width + self.kv_width]
                    v = qkv[:, self.q_width + self.kv_width:]
                else:   # this run of the layer reads keys and values that another run wrote
                    ops.linear(q, hn, self.w_qkv[:self.q_width])
                    k = v = None
                if self.after_projection is not None:
                    self.after_projection.forward(ctx, q, k, v)
                ops.rope_cache_write(q, k, v, ctx.positions, ctx.token_segment, tables, cos, sin, self.pairing,
                                     cache if writes_cache else None, H, K, hd, ctx.page_size, ctx.max_position,
                                     portions=portions)
        att = ctx.rows("attention.out", self.q_width)
        if self.dtype == torch.float32:
            ops.attention_plain(att, q, cache, ctx.positions, ctx.token_segment, tables, H, K, hd,
                                ctx.page_size, self.scale, self.window)
        else:
            tiles = ctx.extra["attention.tiles"]
            if tiles.shape[0]:
                kernel = ctx.host.get("attention.prefill_kernel", 0)
                if kernel == 3 and not ops.attention_halves_fit(hd, H // K, cache):
                    kernel = 0          # (the plan knew the step's row tiles, not the size of the layer)
                ops.attention_bf16_prefill(att, q, cache, tiles, tables, H, K, hd, ctx.page_size,
                                           self.scale, self.window, runs=ctx.extra["attention.runs"] if H == K else None,
                                           kernel=kernel)
            rows = ctx.extra["attention.decode_rows"]
            if rows.numel():
                nseg = rows.numel()
                # under a captured graph the split count is fixed for the whole width of the block table
                span = ctx.host.get("graph.max_context", ctx.host["attention.decode_max_position"] + 1)
                if self.window > 0:
                    span = min(span, self.window + _TILE)
                key_tiles = (span + _TILE - 1) // _TILE
                splits = max(-(-key_tiles // (_DECODE_WAVES * _TILES_PER_WAVE)),
                             min(_DECODE_WORKGROUPS // max(1, nseg * K), -(-key_tiles // _DECODE_WAVES)), 1)
                partial = counters = None
                if splits > 1:
                    partial = ctx.workspace.flat("attention.partial", nseg * H * splits * (hd + 2), torch.float32)
                    counters = ctx.workspace.counters("attention.splits", nseg * K)
                in_order = ctx.host.get("attention.decode_in_order", False)
                ops.attention_bf16_decode(att, q, cache, None if in_order else rows,
                                          ctx.extra["attention.decode_positions"],
                                          None if in_order else ctx.extra["attention.decode_tables"], tables, H, K, hd,
                                          ctx.page_size, self.scale, self.window, partial, splits, _DECODE_WAVES,
                                          counters)
        if fused:      # the output projection adds into x and, if asked, begins the norm that follows
            emit = then.offer() if then is not None else None
            ops.linear_fused(x, att, self.w_o_tiles, "add", emit=emit, **ctx.workspace.product_scratch(n, self.w_o_tiles))
        else:
            cut = ctx.workspace.split_scratch(n, self.w_o)
            after = then.offer_whole() if then is not None and self.dtype == torch.bfloat16 and cut else None
            if after:      # ... goes on with the whole norm that follows, where its K is cut over workgroups
                ops.linear_add_norm(x, att, self.w_o, after["out"], after["weight"], after["eps"], **cut)
            else:
                ops.linear(x, att, self.w_o, accumulate=True, **cut)
