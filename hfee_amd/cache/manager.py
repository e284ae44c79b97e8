"""The cache manager: pages, block tables and fixed-size state slots.

The reference gives every sequence one dense array per layer, all allocated up
front and never returned (/root/reference/internal/llm/forward.go:10-26), and only
its token count says how much of it is valid (forward.go:28-34, 121-123).  Here the
same memory is cut into pages of `page_size` tokens.  A request holds, for every
cache group, a block table (page ids by position // page_size) and one state slot.

Groups: layers whose caches have the same needs share a group and a page id
addresses the same place in each of the group's layers.  A "full" group keeps every
key; a "window" group keeps the last `window` keys, and pages that the window has
passed go back to the pool at commit time.  Pages come back when a request is
released and are handed out again at once (last freed, first reused).

Prefixes kept between requests.  The reference leaves a finished request's cache in its
slot and puts the next request into the slot whose tokens share the longest prefix with
it, so that only the rest of the prompt is run, and always at least one token
(/root/reference/internal/llm/runner.go:198-229).  With pages the same thing is done page
by page (`keep_prefixes`): the full pages of a released request stay behind, each under a
digest of all tokens up to its end; a new request takes over, from the first page on, the
kept pages whose digests its own prompt produces, as its own (a page is never shared:
it is free, kept, or owned by one request), and runs what is left.  Kept pages count as
free: when the free list is empty the oldest kept page is taken, the deepest page of a
chain before the pages in front of it.  Only models whose groups all keep every token can
do this (a window group has given pages back; fixed-size state cannot be cut back).

This file is bookkeeping only (no tensors); storage.py holds the device memory.
"""
from __future__ import annotations

import hashlib
from collections import OrderedDict
from dataclasses import dataclass, field

import numpy as np


class OutOfPages(RuntimeError):
    """A reservation needs more pages than the pool has free."""


class CacheError(RuntimeError):
    """The manager was used against its contract (unknown request, double release...)."""


@dataclass(frozen=True)
class CacheGroupSpec:
    """Cache layers with the same needs.  token_shape: the elements one token adds to one
    layer (attention: (2, kv_heads, head_dim)); the manager needs only its size, the
    arrangement inside a page (`layout`) is the business of the parts that use the layers."""
    kind: str                 # "full" or "window"
    token_shape: tuple
    cache_layers: tuple       # ids of the cache layers in this group
    window: int = 0           # keys kept per token for kind == "window"
    layout: str = ""

    def __post_init__(self):
        if self.kind not in ("full", "window"):
            raise CacheError(f"unknown cache group kind {self.kind!r}")
        if self.kind == "window" and self.window <= 0:
            raise CacheError("a window group needs a positive window")
        if not self.token_shape or any(int(n) < 1 for n in self.token_shape):
            raise CacheError(f"a token must add at least one element to a cache layer, got {self.token_shape!r}")

    @property
    def token_elements(self) -> int:
        n = 1
        for k in self.token_shape:
            n *= int(k)
        return n


KEPT = ("kept prefix",)      # the owner of pages that wait for a request with the same prefix


class PagePool:
    """The pages of one group.  LIFO free list; every page is free or owned by
    exactly one owner (a request, or KEPT)."""

    def __init__(self, num_pages: int):
        if num_pages < 1:
            raise CacheError("a page pool needs at least one page")
        self.num_pages = num_pages
        self._free = list(range(num_pages - 1, -1, -1))   # pop() hands out 0 first
        self._owner: list = [None] * num_pages
        self.reclaimable = lambda: 0        # pages that `reclaim` can still bring back
        self.reclaim = lambda: None         # brings at least one page back to the free list

    @property
    def num_free(self) -> int:
        """Pages that can be taken: the free ones and those a kept prefix would give up."""
        return len(self._free) + self.reclaimable()

    def take(self, owner) -> int:
        if not self._free and self.reclaimable():
            self.reclaim()
        if not self._free:
            raise OutOfPages("no free page")
        page = self._free.pop()
        assert self._owner[page] is None, "a free page had an owner"
        self._owner[page] = owner
        return page

    def give_back(self, page: int, owner) -> None:
        if not 0 <= page < self.num_pages:
            raise CacheError(f"page {page} does not exist")
        if self._owner[page] is None:
            raise CacheError(f"page {page} is freed twice")
        if self._owner[page] != owner:
            raise CacheError(f"page {page} belongs to {self._owner[page]!r}, not {owner!r}")
        self._owner[page] = None
        self._free.append(page)

    def owner_of(self, page: int):
        return self._owner[page]

    def hand_over(self, page: int, owner, new_owner) -> None:
        if self._owner[page] != owner or owner is None or new_owner is None:
            raise CacheError(f"page {page} belongs to {self._owner[page]!r}, not {owner!r}")
        self._owner[page] = new_owner


@dataclass
class RequestCache:
    request_id: object
    slot: int
    length: int = 0                                   # committed tokens
    reused: int = 0                                   # of these, taken over from a kept prefix at admission
    tables: list = field(default_factory=list)        # per group: page id per block, -1 once released
    first_live_block: list = field(default_factory=list)   # per group
    arrays: list = field(default_factory=list)        # per group: the table as int32 (released blocks read 0),
                                                      # kept in step with `tables` for the step's upload

    def table_array(self, group: int) -> np.ndarray:
        return self.arrays[group][:len(self.tables[group])]

    def _append(self, group: int, page: int) -> None:
        arr, n = self.arrays[group], len(self.tables[group])
        if n >= arr.shape[0]:
            grown = np.zeros(max(16, 2 * arr.shape[0]), dtype=np.int32)
            grown[:n] = arr[:n]
            self.arrays[group] = arr = grown
        arr[n] = page
        self.tables[group].append(page)


class CacheManager:
    def __init__(self, groups, page_size: int, pages_per_group, max_requests: int, keep_prefixes: bool = False):
        if page_size < 16 or page_size & (page_size - 1):
            raise CacheError(f"page_size must be a power of two >= 16, got {page_size}")
        self.groups = tuple(groups)
        if isinstance(pages_per_group, int):
            pages_per_group = [pages_per_group] * len(self.groups)
        if len(pages_per_group) != len(self.groups):
            raise CacheError("one page count per cache group is needed")
        self.page_size = page_size
        self.pools = [PagePool(n) for n in pages_per_group]
        self.max_requests = max_requests
        self._free_slots = list(range(max_requests - 1, -1, -1))
        self.requests: dict = {}
        if keep_prefixes and any(g.kind != "full" for g in self.groups):
            raise CacheError("prefixes can be kept only where every cache group keeps every token")
        self.keep_prefixes = bool(keep_prefixes) and bool(self.groups)
        # digest of the tokens up to a page's end -> (the page in every group, the page's own tokens);
        # the oldest entry first
        self._kept: OrderedDict = OrderedDict()
        self.prefix_hits = 0          # tokens taken over from kept prefixes so far
        for pool in self.pools:
            pool.reclaimable = lambda: len(self._kept)
            pool.reclaim = self._drop_oldest_kept

    # ------------------------------------------------------------ requests
    def admit(self, request_id, tokens=None) -> RequestCache:
        """A new request.  With `tokens` (its prompt) and kept prefixes, it takes over the kept
        pages that hold the beginning of the prompt, whole pages only and never the whole
        prompt: its `length` (= `reused`) says how many tokens need not be run."""
        if request_id in self.requests:
            raise CacheError(f"request {request_id!r} is already live")
        if not self._free_slots:
            raise CacheError(f"all {self.max_requests} state slots are in use")
        rc = RequestCache(request_id, self._free_slots.pop(),
                          tables=[[] for _ in self.groups], first_live_block=[0] * len(self.groups),
                          arrays=[np.zeros(16, dtype=np.int32) for _ in self.groups])
        self.requests[request_id] = rc
        if self.keep_prefixes and tokens is not None and self._kept:
            ps = self.page_size
            for b, digest in enumerate(self._digests(tokens, (len(tokens) - 1) // ps)):
                entry = self._kept.get(digest)
                if entry is None or entry[1] != tuple(tokens[b * ps:(b + 1) * ps]):
                    break
                del self._kept[digest]
                for g, page in enumerate(entry[0]):
                    self.pools[g].hand_over(page, KEPT, request_id)
                    rc._append(g, page)
                rc.length += ps
            rc.reused = rc.length
            self.prefix_hits += rc.reused
        return rc

    def get(self, request_id) -> RequestCache:
        try:
            return self.requests[request_id]
        except KeyError:
            raise CacheError(f"request {request_id!r} is not live") from None

    def release(self, request_id, tokens=None) -> None:
        """The request is over: its pages and its slot come back.  With `tokens` (what the
        positions of its cache hold, from the first on; it may know fewer or more than
        `length`) and kept prefixes, the full pages that these tokens cover stay behind for a
        request that begins alike."""
        rc = self.get(request_id)
        keep = 0
        if self.keep_prefixes and tokens is not None:
            keep = min(len(tokens), rc.length) // self.page_size
            digests = self._digests(tokens, keep)
            for b in range(keep - 1, -1, -1):           # the deepest page first: it is the first to go
                if digests[b] in self._kept:            # the same prefix is kept already: this copy is not needed
                    for g in range(len(self.groups)):
                        self.pools[g].give_back(rc.tables[g][b], request_id)
                    continue
                pages = tuple(rc.tables[g][b] for g in range(len(self.groups)))
                for g, page in enumerate(pages):
                    self.pools[g].hand_over(page, request_id, KEPT)
                self._kept[digests[b]] = (pages, tuple(tokens[b * self.page_size:(b + 1) * self.page_size]))
        for g, table in enumerate(rc.tables):
            for page in table[keep:]:
                if page >= 0:
                    self.pools[g].give_back(page, request_id)
        del self.requests[request_id]
        self._free_slots.append(rc.slot)

    # ------------------------------------------------------- kept prefixes
    def _digests(self, tokens, n_pages: int) -> list:
        """For each of the first n_pages pages, a digest of all tokens up to its end."""
        out, h, ps = [], hashlib.blake2b(digest_size=16), self.page_size
        for b in range(n_pages):
            h.update(np.asarray(tokens[b * ps:(b + 1) * ps], dtype=np.int64).tobytes())
            out.append(h.copy().digest())
        return out

    def _drop_oldest_kept(self) -> None:
        if not self._kept:
            return
        _, (pages, _) = self._kept.popitem(last=False)
        for g, page in enumerate(pages):
            self.pools[g].give_back(page, KEPT)

    def drop_kept(self) -> None:
        """Gives every kept page back (nothing is reused after this until requests end again)."""
        while self._kept:
            self._drop_oldest_kept()

    @property
    def num_kept_pages(self) -> int:
        return len(self._kept)

    @property
    def num_free_slots(self) -> int:
        return len(self._free_slots)

    # --------------------------------------------------------------- pages
    def _blocks_for(self, length: int) -> int:
        return (length + self.page_size - 1) // self.page_size

    def pages_needed(self, request_id, n_new: int) -> list:
        """Pages each group would have to take so that positions
        length .. length + n_new - 1 have a place."""
        rc = self.get(request_id)
        want = self._blocks_for(rc.length + n_new)
        return [max(0, want - len(t)) for t in rc.tables]

    def pages_for_tokens(self, n_tokens: int) -> list:
        """Pages per group that a fresh request of n_tokens holds at most at one time
        when it is run in one portion."""
        return [self._blocks_for(n_tokens)] * len(self.groups)

    def can_reserve(self, request_id, n_new: int) -> bool:
        return all(need <= pool.num_free for need, pool in zip(self.pages_needed(request_id, n_new), self.pools))

    def free_pages(self) -> list:
        """Pages per group that can be taken now (kept prefixes give theirs up when asked)."""
        return [p.num_free for p in self.pools]

    def reserve(self, request_id, n_new: int) -> None:
        """Takes the pages for the next n_new tokens in every group, or none at all
        (OutOfPages)."""
        if n_new < 0:
            raise CacheError("cannot reserve a negative number of tokens")
        rc = self.get(request_id)
        need = self.pages_needed(request_id, n_new)
        for n, pool, g in zip(need, self.pools, range(len(self.pools))):
            if n > pool.num_free:
                raise OutOfPages(f"request {request_id!r} needs {n} more pages in cache group {g}, "
                                 f"{pool.num_free} are free")
        for g, n in enumerate(need):
            for _ in range(n):
                rc._append(g, self.pools[g].take(request_id))

    def commit(self, request_id, n_new: int) -> None:
        """The step has written n_new tokens: advance the length and return the
        pages that a window has passed."""
        rc = self.get(request_id)
        if any(self._blocks_for(rc.length + n_new) > len(t) for t in rc.tables):
            raise CacheError(f"request {request_id!r}: commit of {n_new} tokens beyond the reserved pages")
        rc.length += n_new
        for g, spec in enumerate(self.groups):
            if spec.kind != "window":
                continue
            # the next query sits at position >= length and reads keys >= length - window + 1
            first_needed = max(0, rc.length - spec.window + 1)
            dead_until = first_needed // self.page_size        # blocks < dead_until are never read again
            table = rc.tables[g]
            for b in range(rc.first_live_block[g], min(dead_until, len(table))):
                if table[b] >= 0:
                    self.pools[g].give_back(table[b], request_id)
                    table[b] = -1
                    rc.arrays[g][b] = 0
            rc.first_live_block[g] = max(rc.first_live_block[g], min(dead_until, len(table)))

    def truncate(self, request_id, length: int) -> None:
        """Forget tokens at and after `length` (full groups give back whole pages
        beyond it; the rows left in a kept page are overwritten later, as the
        reference's Truncate leaves stale rows, forward.go:31-34).  Window groups
        cannot go back past what they have released."""
        rc = self.get(request_id)
        if not 0 <= length <= rc.length:
            raise CacheError(f"cannot truncate request {request_id!r} from {rc.length} to {length}")
        keep = self._blocks_for(length)
        for g, spec in enumerate(self.groups):
            table = rc.tables[g]
            if spec.kind == "window" and length > 0 and any(
                    table[b] < 0 for b in range(max(0, (length - spec.window) // self.page_size), min(keep, len(table)))):
                raise CacheError("a window group has already released pages this truncation needs")
            while len(table) > keep:
                page = table.pop()
                if page >= 0:
                    self.pools[g].give_back(page, request_id)
            rc.first_live_block[g] = min(rc.first_live_block[g], len(table))
        rc.length = length

    def block_table(self, request_id, group: int) -> list:
        return self.get(request_id).tables[group]

    # ---------------------------------------------------------- invariants
    def check(self) -> None:
        """No page lost, held twice or freed twice; every table entry is owned by its request."""
        for g, pool in enumerate(self.pools):
            held = []
            for rid, rc in self.requests.items():
                for page in rc.tables[g]:
                    if page >= 0:
                        if pool.owner_of(page) != rid:
                            raise CacheError(f"group {g}: page {page} in the table of {rid!r} is owned by "
                                             f"{pool.owner_of(page)!r}")
                        held.append(page)
            for pages, tokens in self._kept.values():
                if pool.owner_of(pages[g]) != KEPT or len(tokens) != self.page_size:
                    raise CacheError(f"group {g}: kept page {pages[g]} is owned by {pool.owner_of(pages[g])!r}")
                held.append(pages[g])
            if len(held) != len(set(held)):
                raise CacheError(f"group {g}: a page is held twice")
            free = list(pool._free)
            if len(free) != len(set(free)):
                raise CacheError(f"group {g}: a page is on the free list twice")
            if set(free) & set(held):
                raise CacheError(f"group {g}: a page is both free and held")
            if len(free) + len(held) != pool.num_pages:
                raise CacheError(f"group {g}: {pool.num_pages - len(free) - len(held)} page(s) lost")
            for page in free:
                if pool.owner_of(page) is not None:
                    raise CacheError(f"group {g}: free page {page} has an owner")
        slots = [rc.slot for rc in self.requests.values()]
        if len(slots) != len(set(slots)) or set(slots) & set(self._free_slots) \
                or len(slots) + len(self._free_slots) != self.max_requests:
            raise CacheError("state slots are inconsistent")
