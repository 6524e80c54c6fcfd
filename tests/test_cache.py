"""The cache manager on the host (no GPU): the reference's allocator vectors
(engine/kv/kv_test.go:5-70), all-or-nothing reservations, windows, slots, and
random orders of requests with the invariants checked after every operation."""

import random

import pytest

from kllm_amd.cache import (FREED, CacheError, CacheManager, GroupSpec, OutOfPages, PagePool,
                            SlotPool)


def manager(num_pages, page_size, window=0, slots=8):
    return CacheManager([GroupSpec("g", page_size, num_pages, window)], slots)


def test_reference_reserve_commit_release():
    m = manager(8, 4)                                # engine/kv/kv_test.go:5-38
    m.open("s")
    m.reserve("s", 5)
    assert len(m.table("s", 0)) == 2 and m.pools[0].free_pages == 6
    m.commit("s", 5)
    m.reserve("s", 3)
    assert len(m.table("s", 0)) == 2
    m.commit("s", 3)
    m.reserve("s", 1)
    assert len(m.table("s", 0)) == 3 and m.pools[0].free_pages == 5
    m.release("s")
    assert m.pools[0].free_pages == 8 and "s" not in m
    m.check_invariants()


def test_reference_out_of_blocks_and_recycling():
    m = manager(2, 4)                                # engine/kv/kv_test.go:40-53
    m.open(1), m.open(2)
    m.reserve(1, 8)
    with pytest.raises(OutOfPages):
        m.reserve(2, 1)
    m.release(1)
    m.reserve(2, 1)
    m.check_invariants()


def test_reference_tables_are_distinct_and_low_ids_first():
    m = manager(4, 2)                                # engine/kv/kv_test.go:55-70
    m.open(1), m.open(2)
    m.reserve(1, 4), m.reserve(2, 4)
    assert m.table(1, 0) == [0, 1] and m.table(2, 0) == [2, 3]     # engine/kv/kv.go:17-21
    m.check_invariants()


def test_reservation_is_all_or_nothing():
    m = CacheManager([GroupSpec("a", 4, 8), GroupSpec("b", 4, 2)], 4)
    m.open("r")
    with pytest.raises(OutOfPages):
        m.reserve("r", 12)                           # group b has 2 pages only
    assert m.pools[0].free_pages == 8 and m.pools[1].free_pages == 2
    assert m.table("r", 0) == [] and m.get("r").reserved == 0
    m.reserve("r", 8)
    m.cancel("r")                                    # a failed step gives everything back
    assert m.pools[0].free_pages == 8 and m.pools[1].free_pages == 2
    m.check_invariants()


def test_lifo_reuse_of_freed_pages():
    m = manager(6, 2)
    m.open("a"), m.open("b")
    m.reserve("a", 4), m.commit("a", 4)              # pages 0, 1
    m.reserve("b", 2), m.commit("b", 2)              # page 2
    m.release("a")
    m.open("c")
    m.reserve("c", 6)
    assert m.table("c", 0) == [1, 0, 3]              # freed pages come back first, last in first out
    m.check_invariants()


def test_misuse_is_an_error():
    m = manager(4, 4)
    with pytest.raises(CacheError):
        m.reserve("nobody", 1)
    m.open("a")
    with pytest.raises(CacheError):
        m.open("a")
    with pytest.raises(CacheError):
        m.commit("a", 1)                             # nothing reserved
    m.reserve("a", 2)
    with pytest.raises(CacheError):
        m.commit("a", 3)
    pool = PagePool(3, 4)
    ids = pool.alloc(2)
    pool.free(ids)
    with pytest.raises(CacheError, match="twice"):
        pool.free([ids[0]])
    with pytest.raises(CacheError):
        pool.free([7])
    with pytest.raises(OutOfPages):
        pool.alloc(4)
    assert pool.free_pages == 3


def test_slots():
    m = manager(4, 4, slots=2)
    a, b = m.open("a"), m.open("b")
    assert {a.slot, b.slot} == {0, 1}
    with pytest.raises(OutOfPages):
        m.open("c")
    m.release("a")
    assert m.open("c").slot == a.slot
    s = SlotPool(1)
    x = s.alloc()
    s.free(x)
    with pytest.raises(CacheError):
        s.free(x)


def test_window_gives_pages_back_once_passed():
    m = manager(8, 4, window=6)
    m.open("r")
    m.reserve("r", 5), m.commit("r", 5)              # next token at 5 reads keys 0..5
    assert m.table("r", 0) == [0, 1]
    m.reserve("r", 5), m.commit("r", 5)              # length 10: next reads 5..10 -> page 0 passed
    assert m.table("r", 0) == [FREED, 1, 2] and m.pools[0].free_pages == 6
    m.reserve("r", 1), m.commit("r", 1)              # length 11: reads 6..11, page 1 (4..7) still needed
    assert m.table("r", 0) == [FREED, 1, 2]
    m.reserve("r", 2), m.commit("r", 2)              # length 13: reads 8..13, page 1 passed
    assert m.table("r", 0) == [FREED, FREED, 2, 0]   # and page 0 is used again
    m.check_invariants()
    m.release("r")
    assert m.pools[0].free_pages == 8


def test_window_lets_a_long_request_live_in_a_small_pool():
    m = manager(4, 4, window=5)
    m.open("r")
    for _ in range(200):
        m.reserve("r", 1), m.commit("r", 1)
        m.check_invariants()
        assert m.pools[0].used_pages <= 3


def test_groups_have_pools_of_their_own():
    m = CacheManager([GroupSpec("all", 4, 10), GroupSpec("win", 4, 10, window=4)], 4)
    m.open("r")
    m.reserve("r", 20), m.commit("r", 20)
    assert len(m.table("r", 0)) == 5 and m.pools[0].used_pages == 5
    assert m.pools[1].used_pages == 1 and m.table("r", 1)[:4] == [FREED] * 4
    st = m.stats()
    assert st["groups"][0]["used"] == 5 and st["groups"][1]["high_water"] == 5
    m.release("r")
    m.check_invariants()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_lose_no_page(seed):
    rng = random.Random(seed)
    groups = [GroupSpec("all", 4, 24), GroupSpec("win", 8, 10, window=rng.choice([5, 9, 16]))]
    m = CacheManager(groups, 5)
    live, next_id = {}, 0
    for _ in range(600):
        op = rng.random()
        try:
            if op < 0.15 and len(live) < 5:
                m.open(next_id)
                live[next_id] = 0
                next_id += 1
            elif op < 0.75 and live:
                r = rng.choice(list(live))
                n = rng.choice([1, 1, 1, 2, 3, 7, 13])
                m.reserve(r, n)
                if rng.random() < 0.1:
                    m.cancel(r)
                else:
                    k = n if rng.random() < 0.8 else rng.randint(1, n)
                    m.commit(r, k)
                    live[r] += k
                    if k < n:
                        m.cancel(r)
            elif live:
                r = rng.choice(list(live))
                m.release(r)
                del live[r]
        except OutOfPages:
            pass
        m.check_invariants()
        for r, n in live.items():
            rc = m.get(r)
            assert rc.length == n and rc.reserved == 0
            assert len(rc.tables[0]) == -(-n // 4) and FREED not in rc.tables[0]
            w = groups[1].window
            held = [p for p in rc.tables[1] if p != FREED]
            assert len(held) <= (w + 8 - 1) // 8 + 1
    for r in list(live):
        m.release(r)
    assert all(p.free_pages == p.num_pages for p in m.pools) and m.slots.free_slots == 5


@pytest.mark.parametrize("page_size,window,step", [(4, 5, 1), (4, 6, 5), (8, 9, 13), (16, 20, 64), (16, 1, 2), (4, 16, 3)])
def test_a_windowed_request_never_holds_more_than_pages_for_tokens_says(page_size, window, step):
    """The bound that sizes a windowed group's pool and admits long requests:
    random portions of at most ``step`` tokens, pages counted while reserved."""
    from kllm_amd.cache.manager import window_pages
    rng = random.Random(page_size * 1000 + window * 10 + step)
    total = 40 * page_size
    bound = window_pages(total, step, page_size, window)
    assert bound <= -(-(step + window - 1) // page_size) + 1 and bound < -(-total // page_size)
    m = CacheManager([GroupSpec("win", page_size, bound, window=window)], 2)
    assert m.pages_for_tokens(total, step) == [bound] and m.pages_for_tokens(total) == [-(-total // page_size)]
    m.open("r")
    done, most = 0, 0
    while done < total:
        n = min(rng.randint(1, step), total - done)
        m.reserve("r", n)                       # never OutOfPages: the pool is exactly the bound
        most = max(most, m.pools[0].used_pages)
        m.commit("r", n)
        done += n
        m.check_invariants()
    assert most <= bound
    assert most >= bound - 1                    # and the bound is not loose by more than a page
    assert window_pages(total, step, page_size, 0) == -(-total // page_size)
