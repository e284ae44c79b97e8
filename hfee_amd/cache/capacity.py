"""How many pages the cache gets.

The reference gives every slot a dense array for its whole context when the slot is first
used (/root/reference/internal/llm/forward.go:18-26) and clamps the context to what the
model was trained for (/root/reference/internal/llm/runner.go:72); memory is whatever
that multiplies out to.  Here the pool is sized from the device's free memory: the weights
and their second copies in tiles are there first (the copies stop while a fifth of the
memory is still free), then the cache takes what is left, less the workspace of the largest
step and a reserve; a pool that was asked for by number and does not fit is refused with
the bytes it needs and the bytes there are, before anything is allocated.

Only arithmetic here, so that it can be tested without a GPU.
"""
from __future__ import annotations

from .manager import CacheError

# the part of the device's memory that stays free for whatever else the process holds
# (the allocator's slack, kernel libraries, captured graphs)
RESERVE_FRACTION = 0.05


def workspace_bytes(max_batch_tokens: int, vocab: int, widest: int) -> int:
    """An upper estimate of the step workspace: for every row of the largest step float32
    logits, and sixteen bytes for each output of the widest product (its float32 sums, its
    bfloat16 results and the buffers of the neighbouring parts)."""
    return max_batch_tokens * (4 * vocab + 16 * widest)


def budget(free: int, total: int, workspace: int) -> int:
    """Bytes the cache may take when `free` of the device's `total` bytes are free now."""
    return free - workspace - int(RESERVE_FRACTION * total)


def pages_that_fit(free: int, total: int, workspace: int, bytes_per_page: int, state_bytes: int = 0) -> int:
    """The pages (of all groups and cache layers together: one page id a group) that the budget holds."""
    if bytes_per_page <= 0:
        return 0
    return max(0, (budget(free, total, workspace) - state_bytes) // bytes_per_page)


def require_room(need: int, what: str, free: int, total: int, workspace: int, hint: str = "") -> None:
    """Raises CacheError, naming the bytes needed and the bytes there are, if `need` bytes of
    cache do not fit."""
    room = budget(free, total, workspace)
    if need > room:
        raise CacheError(
            f"{what} needs {need:,} bytes, but {room:,} bytes are there for it: {free:,} of the device's "
            f"{total:,} bytes are free, {workspace:,} are kept for the workspace of the largest step and "
            f"{int(RESERVE_FRACTION * total):,} in reserve{hint}")


def choose_pages(requested, wanted_at_most: int, free: int, total: int, workspace: int, bytes_per_page: int,
                 state_bytes: int = 0) -> int:
    """requested: a number of pages that the caller insists on, or None.  wanted_at_most: what
    every request slot at its full context would take (more is never used).  Raises CacheError
    where the request, or a single page, does not fit."""
    fit = pages_that_fit(free, total, workspace, bytes_per_page, state_bytes)
    if requested is not None:
        require_room(requested * bytes_per_page + state_bytes, f"the cache of {requested} pages ({bytes_per_page:,} bytes a page)",
                     free, total, workspace, f"; {fit} pages would fit")
        return requested
    if fit < 1:
        require_room(bytes_per_page + state_bytes, f"no page of the cache fits: one page ({bytes_per_page:,} bytes)",
                     free, total, workspace)
    return min(fit, wanted_at_most)
