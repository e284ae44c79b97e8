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
