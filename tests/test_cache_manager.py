"""The cache manager: no page lost, held twice or freed twice, under random orders
of requests; windows give pages back; state slots are exclusive (CPU)."""
import random

import pytest

from hfee_amd.cache import CacheError, CacheGroupSpec, CacheManager, OutOfPages, PagePool

FULL = CacheGroupSpec("full", (2, 2, 16), cache_layers=(0, 1))
WIN = CacheGroupSpec("window", (2, 2, 16), cache_layers=(2,), window=40)


def test_pool_refuses_double_free_and_foreign_free():
    p = PagePool(3)
    a, b = p.take("x"), p.take("y")
    assert (a, b) == (0, 1) and p.num_free == 1
    p.give_back(a, "x")
    with pytest.raises(CacheError, match="freed twice"):
        p.give_back(a, "x")
    with pytest.raises(CacheError, match="belongs to"):
        p.give_back(b, "x")
    assert p.take("z") == a, "the page freed last is handed out first"
    p.take("z")
    with pytest.raises(OutOfPages):
        p.take("z")


def test_reserve_commit_release_and_reuse():
    m = CacheManager([FULL], 16, 6, max_requests=2)
    a = m.admit("a")
    assert m.pages_needed("a", 17) == [2]
    m.reserve("a", 17)
    m.commit("a", 17)
    assert a.length == 17 and m.pages_needed("a", 15) == [0] and m.pages_needed("a", 16) == [1]
    m.admit("b")
    with pytest.raises(OutOfPages):
        m.reserve("b", 16 * 4 + 1)
    assert m.free_pages() == [4], "a failed reservation takes nothing"
    m.reserve("b", 64)
    with pytest.raises(CacheError, match="beyond the reserved pages"):
        m.commit("a", 16)
    with pytest.raises(CacheError, match="state slots"):
        m.admit("c")
    held = list(m.block_table("a", 0))
    m.release("a")
    m.check()
    c = m.admit("c")
    assert c.slot == a.slot
    m.reserve("c", 20)
    assert sorted(m.block_table("c", 0)) == sorted(held), "released pages are used again"
    with pytest.raises(CacheError, match="not live"):
        m.release("a")
    m.check()


def test_window_group_gives_back_pages_the_window_has_passed():
    m = CacheManager([FULL, WIN], 16, [32, 12], max_requests=1)
    m.admit("r")
    n = 0
    for portion in (50, 1, 1, 30, 7, 1, 100, 1, 1):
        m.reserve("r", portion)
        m.commit("r", portion)
        n += portion
        m.check()
        full, win = m.block_table("r", 0), m.block_table("r", 1)
        assert all(p >= 0 for p in full) and len(full) == (n + 15) // 16
        first_needed = max(0, n - 40 + 1)
        for b, page in enumerate(win):
            if (b + 1) * 16 <= first_needed:
                assert page == -1, f"block {b} is behind the window and still held"
            else:
                assert page >= 0, f"block {b} is inside the window and gone"
    assert m.free_pages()[1] >= 12 - 4
    m.release("r")
    m.check()
    assert m.free_pages() == [32, 12]


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_every_invariant(seed):
    rng = random.Random(seed)
    m = CacheManager([FULL, WIN], 16, [40, 12], max_requests=5)
    live, counter = {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.num_free_slots:
            counter += 1
            m.admit(counter)
            live[counter] = 0
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 5, 16, 17, 33, 64])
            if m.can_reserve(rid, n):
                m.reserve(rid, n)
                if rng.random() < 0.9:
                    m.commit(rid, n)
                    live[rid] += n
            else:
                with pytest.raises(OutOfPages):
                    m.reserve(rid, n)
        elif op < 0.9 and live:
            rid = rng.choice(list(live))
            if live[rid] and rng.random() < 0.5:
                try:
                    keep = rng.randrange(live[rid] + 1)
                    m.truncate(rid, keep)
                    live[rid] = keep
                except CacheError:
                    pass          # a window group cannot go back past released pages
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        m.check()
        for rid, n in live.items():
            assert m.get(rid).length == n
    for rid in list(live):
        m.release(rid)
    m.check()
    assert m.free_pages() == [40, 12] and m.num_free_slots == 5


# ------------------------------------------------------- prefixes kept between requests
def keeping(pages=16, requests=4, groups=1):
    specs = [CacheGroupSpec("full", (2, 1, 16), (g,)) for g in range(groups)]
    return CacheManager(specs, 16, pages, requests, keep_prefixes=True)


def run_whole(m, rid, tokens):
    rc = m.admit(rid, tokens)
    m.reserve(rid, len(tokens) - rc.length)
    m.commit(rid, len(tokens) - rc.length)
    return rc


def test_full_pages_of_a_released_request_wait_for_one_that_begins_alike():
    m = keeping(pages=8, groups=2)
    a = list(range(100, 140))                         # 40 tokens: two full pages and a half
    rc = run_whole(m, "a", a)
    pages = [list(t) for t in rc.tables]
    m.release("a", a)
    m.check()
    assert m.num_kept_pages == 2 and m.free_pages() == [8, 8]          # kept pages count as free
    # the same 32 tokens and then others: both pages come back, as this request's own, in every group
    rc = m.admit("b", a[:32] + [7, 8, 9])
    assert rc.length == rc.reused == 32 and [t[:2] for t in rc.tables] == [p[:2] for p in pages]
    assert m.num_kept_pages == 0 and m.pages_needed("b", 3) == [1, 1]
    m.check()
    m.release("b", a[:32])
    # exactly the kept tokens: one token must still be run (runner.go:219), so the second page stays
    rc = m.admit("c", a[:32])
    assert rc.length == 16 and m.num_kept_pages == 1
    m.release("c", a[:16])
    m.check()
    # the first page differs in its last token: nothing is taken, although the second page's own tokens agree
    rc = m.admit("d", a[:15] + [0] + a[16:40])
    assert rc.length == 0 and m.num_kept_pages == 2
    m.release("d")
    # a page is known by everything before it as well: these 16 tokens behind another beginning are another page
    rc = m.admit("e", [1] * 16 + a[16:40])
    assert rc.length == 0
    m.release("e")
    m.check()


def test_kept_pages_give_way_when_pages_are_needed_the_deepest_of_the_oldest_first():
    m = keeping(pages=4)
    a, b = list(range(200, 232)) + [1], list(range(300, 316)) + [1]
    run_whole(m, "a", a)                      # pages 0, 1, 2
    m.release("a", a)                         # two kept
    run_whole(m, "b", b)                      # two more pages
    m.release("b", b)                         # one kept
    assert m.num_kept_pages == 3 and m.free_pages() == [4]
    m.admit("c")
    m.reserve("c", 32)                        # one page is free, the other comes from a's second page
    assert m.num_kept_pages == 2
    m.check()
    assert m.admit("a2", a).length == 16      # a's first page is still there, its second is gone
    assert m.admit("b2", b).length == 16
    m.check()
    m.release("a2"), m.release("b2")
    with pytest.raises(OutOfPages):
        m.reserve("c", 80)                    # five pages: nothing kept is left to give way
    m.release("c", None)
    m.drop_kept()
    assert m.free_pages() == [4] and m.num_kept_pages == 0
    m.check()


def test_the_same_prefix_is_kept_once():
    m = keeping(pages=8)
    a = list(range(50, 83))
    run_whole(m, "a", a)
    m.admit("b")                              # the same tokens run again beside it (nothing was kept yet)
    m.reserve("b", 33), m.commit("b", 33)
    m.release("a", a), m.release("b", a)
    assert m.num_kept_pages == 2 and len(m.pools[0]._free) == 6
    m.check()


def test_prefixes_are_not_kept_where_a_window_has_given_pages_back():
    with pytest.raises(CacheError, match="every cache group keeps every token"):
        CacheManager([CacheGroupSpec("window", (2, 1, 16), (0,), window=32)], 16, 8, 2, keep_prefixes=True)


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_with_kept_prefixes(seed):
    """Requests from a small family of prompts that begin alike come and go in random order on
    few pages.  A model of the memory (what was written where) shows that every position of a
    live request, taken over or written, holds that request's token, and check() that no page
    is lost, held twice or both kept and owned."""
    rng = random.Random(seed)
    ps = 16
    m = keeping(pages=12, requests=3)
    stems = [[rng.randrange(1000) for _ in range(70)] for _ in range(2)]
    content, live, n = {}, {}, 0          # (page, slot) -> token; rid -> its tokens
    reused = 0
    for _ in range(400):
        if live and (len(live) == 3 or rng.random() < 0.4):
            rid = rng.choice(sorted(live))
            rc = m.get(rid)
            assert [content[(rc.tables[0][p // ps], p % ps)] for p in range(rc.length)] == live[rid][:rc.length]
            m.release(rid, live[rid] if rng.random() < 0.8 else None)
            del live[rid]
        else:
            stem = rng.choice(stems)
            tokens = stem[:rng.randrange(1, 70)] + [rng.randrange(1000) for _ in range(rng.randrange(0, 20))]
            rid, n = n, n + 1
            rc = m.admit(rid, tokens)
            assert rc.length % ps == 0 and rc.length < len(tokens)
            reused += rc.length
            try:
                m.reserve(rid, len(tokens) - rc.length)
            except OutOfPages:
                m.release(rid, tokens)            # only what it took over can stay behind
                m.check()
                continue
            for p in range(rc.length, len(tokens)):
                content[(rc.tables[0][p // ps], p % ps)] = tokens[p]
            m.commit(rid, len(tokens) - rc.length)
            live[rid] = tokens
        m.check()
    assert reused > 0


def test_the_pool_is_sized_from_the_free_memory():
    """The arithmetic of `capacity`: by default the pool is what every slot at its full context
    takes, or what fits if that is less; a number that was asked for and does not fit is refused
    with the bytes it needs and the bytes there are; a pool of no page is refused."""
    from hfee_amd.cache import capacity
    from hfee_amd.cache.manager import CacheError
    gib = 1 << 30
    total = 288 * gib
    page = 2 << 20                                     # the 8B shape: 128 KiB a token, 16 tokens
    work = capacity.workspace_bytes(2048, 128256, 28672)
    assert work == 2048 * (4 * 128256 + 16 * 28672)
    reserve = int(capacity.RESERVE_FRACTION * total)
    # plenty of room: the slots' full contexts decide
    assert capacity.choose_pages(None, 8 * 512, 200 * gib, total, work, page) == 8 * 512
    # little room: what fits, to the page
    free = 30 * gib
    fit = (free - work - reserve) // page
    assert capacity.pages_that_fit(free, total, work, page) == fit and 0 < fit < 64 * 8192 // 16
    assert capacity.choose_pages(None, 64 * 8192 // 16, free, total, work, page) == fit
    assert capacity.choose_pages(fit, 1, free, total, work, page) == fit          # asked for: taken as it is
    with pytest.raises(CacheError) as e:
        capacity.choose_pages(fit + 1, 1, free, total, work, page)
    msg = str(e.value)
    assert f"needs {(fit + 1) * page:,} bytes" in msg and f"{free:,}" in msg and f"{fit} pages would fit" in msg
    # the states' bytes come off first
    spare = (free - work - reserve) % page
    assert capacity.pages_that_fit(free, total, work, page, state_bytes=3 * page + spare) == fit - 3
    assert capacity.pages_that_fit(free, total, work, page, state_bytes=3 * page + spare + 1) == fit - 4
    with pytest.raises(CacheError, match="no page of the cache fits"):
        capacity.choose_pages(None, 100, work + reserve + page - 1, total, work, page)
    assert capacity.choose_pages(None, 100, work + reserve + page, total, work, page) == 1
