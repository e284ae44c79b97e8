"""The step function: one batch of (request, its next tokens) through the model.

It is the reference's Model.Forward (/root/reference/internal/llm/forward.go:41-142):
every entry brings any number >= 1 of consecutive new tokens of one sequence,
starting at that sequence's cached length; portions of prompts sit beside single
decoded tokens; all rows run through the layers together; keys and values go to the
cache; the final norm and the head run only for the rows whose logits are wanted.
Unlike the reference, logits can be asked for at any of an entry's tokens, not only
its last, and the cache is paged.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..cache import CacheManager, CacheStorage, OutOfPages, bytes_per_token, capacity
from ..parts.base import Segment, StepContext, Workspace
from .model import EngineInfo, Model


@dataclass
class StepEntry:
    request_id: object
    tokens: list
    want: list = field(default_factory=list)    # indices into `tokens` whose logits are wanted


class StepError(ValueError):
    """The batch breaks the step function's contract."""


class StepPlan:
    """Host side of a step: the segments and every int32 array that goes to the device."""

    def __init__(self, segments):
        self.segments = segments
        self.arrays: dict = {}
        self.host: dict = {}
        self.packed = None        # set by the engine once the arrays lie in a pinned buffer

    def add(self, key: str, array: np.ndarray):
        if key in self.arrays:
            raise StepError(f"step metadata {key!r} is planned twice")
        self.arrays[key] = np.ascontiguousarray(array, dtype=np.int32)


class Engine:
    """Model + cache + workspace on one GPU, and step()."""

    takes_device_tokens = True      # step(..., tokens_from=) is there

    def __init__(self, model: Model, *, num_pages=None, cache_tokens=None, page_size: int = 16,
                 max_requests: int = 64, max_batch_tokens: int = 2048, num_positions: int | None = None,
                 device="cuda:0", use_graphs: bool = True, keep_prefixes: bool = False):
        if not model.bound:
            raise ValueError("the model has no weights bound")
        if not torch.cuda.is_available():
            raise RuntimeError("hfee_amd runs on a GPU only; no GPU is visible")
        self.model, self.dtype, self.device = model, model.dtype, torch.device(device)
        self.page_size = page_size
        self.max_requests = max_requests
        self.max_batch_tokens = max_batch_tokens
        self.num_positions = min(num_positions or model.spec.max_positions, model.spec.max_positions)
        self.vocab = model.spec.vocab
        self.groups = model.cache_groups()
        # The pool: as many pages as were asked for (by number or by tokens), or what every slot at
        # its full context takes; never more than the device's free memory holds beside the
        # workspace of the largest step and a reserve (the weights are there already).
        wanted = None
        if num_pages is not None:
            wanted = num_pages
        elif cache_tokens is not None:
            wanted = (cache_tokens + page_size - 1) // page_size
        at_most = max_requests * ((self.num_positions + page_size - 1) // page_size)
        if isinstance(wanted, (list, tuple)):          # a number for every group
            need = sum(n * page_size * bytes_per_token([g], self.dtype) for n, g in zip(wanted, self.groups))
            capacity.require_room(need + self._state_bytes(), f"the cache of {list(wanted)} pages in its groups",
                                  *self._memory(), self._workspace_estimate())
            num_pages = list(wanted)
        else:
            num_pages = capacity.choose_pages(wanted, at_most, *self._memory(), self._workspace_estimate(),
                                              page_size * bytes_per_token(self.groups, self.dtype),
                                              self._state_bytes())
        self.num_pages = num_pages
        # (a finished request's full pages wait for a request that begins alike: only where every
        # group keeps every token and no part has state that cannot be cut back)
        keep_prefixes = bool(keep_prefixes) and all(g.kind == "full" for g in self.groups) and not model.state_specs()
        self.cache = CacheManager(self.groups, page_size, num_pages, max_requests, keep_prefixes=keep_prefixes)
        self.storage = CacheStorage(self.groups, page_size, num_pages, max_requests, self.dtype, self.device)
        self.workspace = Workspace(max_batch_tokens, self.device)
        info = EngineInfo(self.num_positions, self.device, self.dtype, page_size, max_requests, self.storage)
        for name, shape, dt in model.state_specs():
            self.storage.add_state(name, shape, dt)
        model.prepare(info)
        self._meta_capacity = 0
        self._meta_views: dict = {}        # layout of a step's metadata -> (offsets, views of the device buffer)
        self._prepared = None              # (signature, plan) of a step planned ahead
        self._meta_ring, self._meta_device = [], None
        self.steps_run = 0
        # decode-only steps are replayed as captured HIP graphs, one per
        # (batch size, block-table width, wanted rows): launch gaps would otherwise
        # cost more than the kernels at small batches
        self.use_graphs = use_graphs and model.graph_safe
        self._graphs: dict = {}
        self._graph_seen: dict = {}        # shape -> how often it has come without a recording
        self.graph_replays = 0

    # ------------------------------------------------------------ memory
    def _memory(self):
        """(free, total) bytes of the device; what torch holds in its pool without using it counts as free."""
        free, total = torch.cuda.mem_get_info(self.device)
        idle = torch.cuda.memory_reserved(self.device) - torch.cuda.memory_allocated(self.device)
        return free + max(0, idle), total

    def _workspace_estimate(self) -> int:
        widest = max([s.shape[0] for s in self.model.tensor_specs() if len(s.shape) == 2 and s.shape[0] != self.vocab]
                     or [self.model.spec.hidden])
        return capacity.workspace_bytes(self.max_batch_tokens, self.vocab, max(widest, self.model.spec.hidden))

    def _state_bytes(self) -> int:
        total = 0
        for _, shape, dt in self.model.state_specs():
            n = self.max_requests
            for d in shape:
                n *= d
            total += n * torch.empty((), dtype=dt).element_size()
        return total

    # ------------------------------------------------------------ requests
    def admit(self, request_id, tokens=None):
        """tokens: the request's prompt; with kept prefixes the request starts with the pages
        that hold its beginning (`.length` of what is returned: tokens that need not be run)."""
        rc = self.cache.admit(request_id, tokens)
        self.storage.clear_slot(rc.slot)
        self._prepared = None
        return rc

    def release(self, request_id, tokens=None):
        """tokens: what the request's cache holds, position by position (prompt and generated
        tokens); with kept prefixes its full pages stay behind for a request that begins alike."""
        self.cache.release(request_id, tokens)
        self._prepared = None

    def is_live(self, request_id) -> bool:
        return request_id in self.cache.requests

    def cached_length(self, request_id) -> int:
        return self.cache.get(request_id).length

    # ---------------------------------------------------------------- step
    def _check(self, entries):
        if not entries:
            raise StepError("an empty step")
        seen = set()
        total = 0
        for e in entries:
            if e.request_id in seen:
                raise StepError(f"request {e.request_id!r} appears twice in one step")
            seen.add(e.request_id)
            if len(e.tokens) < 1:
                raise StepError(f"request {e.request_id!r} brings no tokens")
            rc = self.cache.get(e.request_id)
            if rc.length + len(e.tokens) > self.num_positions:
                raise StepError(f"request {e.request_id!r} would reach position "
                                f"{rc.length + len(e.tokens) - 1}, the context holds {self.num_positions}")
            if min(e.tokens) < 0 or max(e.tokens) >= self.vocab:
                raise StepError(f"a token id of request {e.request_id!r} is outside the vocabulary of {self.vocab}")
            if e.want and (min(e.want) < 0 or max(e.want) >= len(e.tokens)):
                raise StepError(f"request {e.request_id!r} wants logits outside its {len(e.tokens)} tokens")
            total += len(e.tokens)
        if total > self.max_batch_tokens:
            raise StepError(f"{total} tokens in one step, the engine was made for {self.max_batch_tokens}")

    def _reserve(self, entries):
        ps = self.page_size
        if all(len(t) * ps >= rc.length + len(e.tokens)
               for e in entries for rc in (self.cache.requests[e.request_id],) for t in rc.tables):
            return                      # every token already has a place (the scheduler reserved it)
        need = [0] * len(self.groups)
        for e in entries:
            for g, k in enumerate(self.cache.pages_needed(e.request_id, len(e.tokens))):
                need[g] += k
        free = self.cache.free_pages()
        for g in range(len(self.groups)):
            if need[g] > free[g]:
                raise OutOfPages(f"the step needs {need[g]} pages in cache group {g}, {free[g]} are free")
        for e in entries:
            self.cache.reserve(e.request_id, len(e.tokens))

    def _pack(self, plan: StepPlan) -> None:
        """Lays the planned arrays out in the pinned buffer of the coming step."""
        layout = tuple((key, a.shape) for key, a in plan.arrays.items())
        total = max(sum((a.size + 3) // 4 * 4 for a in plan.arrays.values()), 4)
        if total > self._meta_capacity:
            cap = max(total * 2, self._meta_bound())
            # a ring of pinned buffers: the copy of step k may still be in flight
            # while the host fills the buffer of step k+1
            self._meta_ring = [(torch.empty(cap, dtype=torch.int32, pin_memory=True), torch.cuda.Event())
                               for _ in range(4)]
            self._meta_device = torch.empty(cap, dtype=torch.int32, device=self.device)
            self._meta_capacity = cap
            self._meta_views.clear()
            self._graphs.clear()      # captured graphs point into the old buffer
            self._graph_seen.clear()
        views = self._meta_views.get(layout)
        if views is None:             # where each array lies, and its view of the device buffer
            if len(self._meta_views) > 256:
                self._meta_views.clear()
            offsets, dev, at = {}, {}, 0
            for key, a in plan.arrays.items():
                offsets[key] = at
                dev[key] = self._meta_device[at:at + a.size].view(a.shape)
                at += (a.size + 3) // 4 * 4
            views = self._meta_views[layout] = (offsets, dev)
        offsets, dev = views
        pinned, event = self._meta_ring[self.steps_run % len(self._meta_ring)]
        event.synchronize()
        host = pinned.numpy()
        for key, a in plan.arrays.items():
            host[offsets[key]:offsets[key] + a.size] = a.reshape(-1)
        plan.packed = (self.steps_run, self._meta_device, pinned, event, total, dev, host[offsets["token_ids"]:])

    def _upload(self, plan: StepPlan, tokens, tokens_from=None) -> dict:
        """All planned arrays in one pinned buffer, one copy to the device.  tokens_from: the
        token ids are (or will be, by the stream's order) on the device: if they lie where the
        step looks for them, the copy leaves that place alone; else they are copied there."""
        if plan.packed is None or plan.packed[0] != self.steps_run or plan.packed[1] is not self._meta_device:
            self._pack(plan)
        _, _, pinned, event, total, dev, token_place = plan.packed
        place = dev["token_ids"]
        first = 0
        if tokens_from is None:
            token_place[:len(tokens)] = tokens
        elif tokens_from.data_ptr() == place.data_ptr():
            first = (place.numel() + 3) // 4 * 4              # (token_ids is the first array of the layout)
        self._meta_device[first:total].copy_(pinned[first:total], non_blocking=True)
        if tokens_from is not None and first == 0:
            place.copy_(tokens_from[:place.numel()])           # on the stream, behind the metadata
        event.record()
        return dev

    @property
    def token_place(self):
        """Where a step of single tokens looks for its token ids on the device (None before
        the first step): a sampler that leaves its ids here saves the next step a copy."""
        return None if self._meta_device is None else self._meta_device[:self.max_requests]

    def _plan(self, shape) -> StepPlan:
        """The metadata of a step whose entries are `shape`: (request id, number of tokens,
        wanted places) each; everything but the token ids themselves.  The requests' pages
        are reserved already."""
        segments, logit_rows = [], []
        row = 0
        for rid, count, want in shape:
            rc = self.cache.get(rid)
            segments.append(Segment(rid, rc.slot, rc.length, count, row))
            logit_rows += [row + w for w in want]
            row += count
        n = row
        starts = np.fromiter((s.start for s in segments), dtype=np.int32, count=len(segments))
        lengths = np.fromiter((s.length for s in segments), dtype=np.int32, count=len(segments))
        rows0 = np.fromiter((s.row0 for s in segments), dtype=np.int32, count=len(segments))
        token_segment = np.repeat(np.arange(len(segments), dtype=np.int32), lengths)
        positions = np.arange(n, dtype=np.int32) - np.repeat(rows0 - starts, lengths)

        plan = StepPlan(segments)
        plan.add("token_ids", np.zeros(n, dtype=np.int32))
        plan.add("positions", positions)
        plan.add("token_segment", token_segment)
        plan.add("segment_slots", np.fromiter((s.slot for s in segments), dtype=np.int32, count=len(segments)))
        plan.add("segment_starts", starts)
        plan.add("segment_lengths", lengths)
        plan.add("segment_rows", rows0)
        plan.add("logit_rows", np.asarray(logit_rows))
        decode_only = self.use_graphs and all(s.length == 1 for s in segments)
        widths = []
        for g in range(len(self.groups)):
            tables = [self.cache.get(s.request_id).table_array(g) for s in segments]
            width = max(1, max(len(t) for t in tables))
            if decode_only:      # few distinct widths, so that few graphs are captured
                width = min(max(8, 1 << (width - 1).bit_length()), max(width, self._max_blocks()))
            widths.append(width)
            bt = np.zeros((len(segments), width), dtype=np.int32)
            for i, t in enumerate(tables):
                bt[i, :len(t)] = t          # blocks that a window has given back hold 0 and are never read
            plan.add(f"block_tables.{g}", bt)
        if decode_only:
            plan.host["graph.max_context"] = max(widths) * self.page_size
        self.model.plan(plan)
        plan.n, plan.wanted, plan.max_position = n, len(logit_rows), int(positions.max())
        plan.graph_key = None
        if decode_only:
            plan.graph_key = (n, tuple(widths), plan.wanted, tuple(sorted((k, a.shape) for k, a in plan.arrays.items())))
        return plan

    def _signature(self, shape) -> tuple:
        """What a plan depends on beside the pages that its requests hold."""
        return tuple((rid, self.cache.get(rid).length, count, tuple(want)) for rid, count, want in shape)

    def prepare(self, shape) -> bool:
        """For a caller that knows the shape of its next step before it knows the tokens
        (a scheduler, while the GPU still runs the step before): reserves the pages and
        plans the step now, so that begin() has only the tokens left to fill in.  shape:
        (request id, number of tokens, wanted places) for each entry.  Nothing is lost if
        the next step turns out differently: begin() then plans anew (pages that were
        reserved stay with their requests).  False if the pages do not suffice."""
        self._prepared = None
        shape = [(rid, count, list(want)) for rid, count, want in shape]
        need = [0] * len(self.groups)
        for rid, count, _ in shape:
            if rid not in self.cache.requests or self.cache.get(rid).length + count > self.num_positions:
                return False
            for g, k in enumerate(self.cache.pages_needed(rid, count)):
                need[g] += k
        free = self.cache.free_pages()
        if any(need[g] > free[g] for g in range(len(self.groups))):
            return False
        for rid, count, _ in shape:
            self.cache.reserve(rid, count)
        plan = self._plan(shape)
        self._pack(plan)
        self._prepared = (self._signature(shape), plan)
        return True

    def begin(self, entries, tokens_from=None):
        """Checks the entries, takes their pages, sends the step's metadata to the
        device and returns (context, number of wanted rows, key for graph capture or
        None).  step() is begin + the model + commit; tests of single parts call
        begin() themselves.  tokens_from: see step()."""
        entries = list(entries)
        self._check(entries)
        self._reserve(entries)

        shape = [(e.request_id, len(e.tokens), e.want) for e in entries]
        prepared, self._prepared = self._prepared, None
        if prepared is not None and prepared[0] == self._signature(shape):
            plan = prepared[1]
        else:
            plan = self._plan(shape)
        tokens = entries[0].tokens if len(entries) == 1 else [t for e in entries for t in e.tokens]
        if tokens_from is not None and (tokens_from.dtype != torch.int32 or tokens_from.device != self.device
                                        or tokens_from.numel() < plan.n):
            raise StepError("tokens_from must be int32 on the engine's device, one id a row of the step")
        dev = self._upload(plan, tokens, tokens_from)
        ctx = StepContext(
            n=plan.n, dtype=self.dtype, device=self.device, segments=plan.segments,
            token_ids=dev["token_ids"], positions=dev["positions"], token_segment=dev["token_segment"],
            segment_slots=dev["segment_slots"], segment_starts=dev["segment_starts"],
            segment_lengths=dev["segment_lengths"], segment_rows=dev["segment_rows"],
            block_tables=[dev[f"block_tables.{g}"] for g in range(len(self.groups))],
            max_position=plan.max_position, storage=self.storage, workspace=self.workspace,
            page_size=self.page_size, extra=dev, host=plan.host)
        return ctx, plan.wanted, plan.graph_key

    def commit(self, entries) -> None:
        for e in entries:
            self.cache.commit(e.request_id, len(e.tokens))
        self.steps_run += 1

    def step(self, entries, tokens_from=None) -> torch.Tensor:
        """Runs the entries as one batch; returns float32 logits [wanted, vocab] in the
        order of the entries and of each entry's `want` (None if nothing is wanted).
        The tensor is a view of the workspace: the next step overwrites it.

        tokens_from: an int32 tensor on the device that holds the step's token ids, one a
        row, when the step runs (work queued on the stream before this call may still be
        writing it); the entries' own tokens then only say how many there are.  For a
        caller that launches a step before the host has seen the tokens that the step
        before sampled."""
        entries = list(entries)
        ctx, w, key = self.begin(entries, tokens_from)
        n, dev = ctx.n, ctx.extra
        if key is not None:
            graph = self._graphs.get(key)
            if graph is None:
                logits = self._forward(ctx, n, w, dev)          # this step, eagerly; buffers get made
                # A shape is recorded when it comes a second time: recording takes as long as several
                # steps, and while requests end one after the other every step has a batch size of
                # its own that never comes again (128 requests at the 1B shape: a third of the run
                # went into recordings that were replayed once or never).
                self._graph_seen[key] = self._graph_seen.get(key, 0) + 1
                if self._graph_seen[key] >= 2:
                    captured = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(captured):
                        self._forward(ctx, n, w, dev)            # recorded, not run
                    self._graphs[key] = captured
            else:
                graph.replay()
                self.graph_replays += 1
                logits = self.workspace.rows("logits", w, self.vocab, torch.float32) if w else None
        else:
            logits = self._forward(ctx, n, w, dev)

        self.commit(entries)
        return logits

    def _forward(self, ctx, n: int, w: int, dev: dict):
        x = self.workspace.rows("residual", n, self.model.spec.hidden, torch.float32)
        schedule, blocks = self.model.schedule, self.model.blocks
        carried = None          # the next block's normed input, if what ran before has begun it
        first = blocks[schedule[0].layer] if schedule else None
        if getattr(self.model.embedding, "emits_norm", False) and getattr(first, "chains_norms", False):
            carried = first.begin(ctx, x)
            self.model.embedding.forward(ctx, x, then=carried)
        else:
            self.model.embedding.forward(ctx, x)
        for i, entry in enumerate(schedule):
            block = blocks[entry.layer]
            if getattr(block, "chains_norms", False):
                after = blocks[schedule[i + 1].layer] if i + 1 < len(schedule) else None
                following = after.begin(ctx, x) if getattr(after, "chains_norms", False) else None
                block.forward(ctx, x, entry, carried, following)
                carried = following
            else:
                block.forward(ctx, x, entry)
                carried = None
        if not w:
            return None
        logits = self.workspace.rows("logits", w, self.vocab, torch.float32)
        self.model.head.forward(ctx, logits, x, dev["logit_rows"])
        return logits

    def _max_blocks(self) -> int:
        return (self.num_positions + self.page_size - 1) // self.page_size

    def _meta_bound(self) -> int:
        """int32 words that the metadata of the largest step can take."""
        t, r = self.max_batch_tokens, self.max_requests
        return 8 * t + 16 * r + len(self.groups) * r * (self._max_blocks() + 4) + 4096
